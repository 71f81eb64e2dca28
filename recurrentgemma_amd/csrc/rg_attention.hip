// The small steps of the local-attention block around its matrix products
// (recurrentgemma/torch/modules.py:52-83 rotary embedding, :152-183 positions
// held by the ring cache, :186-216 ring update, :462-474 masked softmax): one
// kernel each instead of a few dozen elementwise launches per block and
// decoded token.  The products themselves (projections, scores, weighted sum
// of the values) stay batched GEMMs of the caller.  Every step rounds to the
// activation dtype where the reference's chain of tensor ops does.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

__device__ __forceinline__ float position_as_float(const void* pos, int kind,
                                                   int64_t i) {
  return kind == kSegI64 ? (float)reinterpret_cast<const int64_t*>(pos)[i]
                         : (float)reinterpret_cast<const int32_t*>(pos)[i];
}

// x, out [rows, n, hd]; positions [rows]; inv_freq [hd / 4] float32.
// First half of the head dimension: element i pairs with element i + hd/4,
// rotated by position * inv_freq[i]; second half copied.
// A second tensor (x2, out2 [rows, n2, hd], same positions: the keys beside
// the queries) takes the elements from `total` up to `total + total2`.
template <typename T>
__global__ void __launch_bounds__(256)
rope_kernel(const T* __restrict__ x, const void* __restrict__ pos,
            int pos_kind, const float* __restrict__ inv_freq,
            T* __restrict__ out, int64_t total, int n, int hd,
            const T* __restrict__ x2, T* __restrict__ out2, int64_t total2,
            int n2) {
  // products and their sum are separate tensors in the reference: no fused
  // multiply-add (matters in float32, where nothing is rounded in between)
#pragma clang fp contract(off)
  int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= total) {
    e -= total;
    if (e >= total2) return;
    x = x2;
    out = out2;
    n = n2;
  }
  const int d = (int)(e % hd);
  const int half = hd / 2, quarter = hd / 4;
  if (d >= half) {
    out[e] = x[e];
    return;
  }
  const int64_t row = e / ((int64_t)n * hd);
  const int i = d % quarter;
  const float angle = position_as_float(pos, pos_kind, row) * inv_freq[i];
  const float s = round_act<T>(sinf(angle)), c = round_act<T>(cosf(angle));
  const int64_t base = e - d;
  const float lo = load_scalar<T>(x + base + i);
  const float hi = load_scalar<T>(x + base + i + quarter);
  const float v = d < quarter
                      ? round_act<T>(lo * c) - round_act<T>(hi * s)
                      : round_act<T>(hi * c) + round_act<T>(lo * s);
  store_scalar<T>(out + e, v);
}

// bf16, head_dim a multiple of 32: eight elements (16 bytes) per access.  A
// head is hd/32 rotate items (elements i .. i+7 of the first quarter with
// their partners in the second, both read and written by one thread) and
// hd/16 copy items (second half).  A thread owns one item of one row for
// every head of x and of x2: the eight sines and cosines of a rotate item
// depend on the row and the item only, and are formed once for all heads
// (eleven times fewer than per head at ten query heads and one key head).
// Same arithmetic per element as rope_kernel.
__global__ void __launch_bounds__(256)
rope_bf16_vec_kernel(const uint16_t* __restrict__ x,
                     const void* __restrict__ pos, int pos_kind,
                     const float* __restrict__ inv_freq,
                     uint16_t* __restrict__ out, int64_t rows, int n, int hd,
                     const uint16_t* __restrict__ x2,
                     uint16_t* __restrict__ out2, int n2) {
#pragma clang fp contract(off)
  const int per_head = hd / 32 + hd / 16;
  const int64_t item = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = item / per_head;
  const int which = (int)(item - row * per_head);
  if (row >= rows) return;
  const int quarter = hd / 4;
  if (which >= hd / 32) {  // copy
    const int off = hd / 2 + 8 * (which - hd / 32);
    for (int h = 0; h < n; ++h) {
      const int64_t at = (row * n + h) * hd + off;
      *reinterpret_cast<u32x4*>(out + at) =
          *reinterpret_cast<const u32x4*>(x + at);
    }
    for (int h = 0; h < n2; ++h) {
      const int64_t at = (row * n2 + h) * hd + off;
      *reinterpret_cast<u32x4*>(out2 + at) =
          *reinterpret_cast<const u32x4*>(x2 + at);
    }
    return;
  }
  const int i0 = 8 * which;
  const float p = position_as_float(pos, pos_kind, row);
  float sn[8], cs[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float angle = p * inv_freq[i0 + e];
    sn[e] = round_to_bf16(sinf(angle));
    cs[e] = round_to_bf16(cosf(angle));
  }
  auto rotate = [&](const uint16_t* src, uint16_t* dst) {
    const u32x4 lo4 = *reinterpret_cast<const u32x4*>(src);
    const u32x4 hi4 = *reinterpret_cast<const u32x4*>(src + quarter);
    u32x4 olo, ohi;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float vlo[2], vhi[2];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const float lo = e == 0 ? __uint_as_float(lo4[k] << 16)
                                : __uint_as_float(lo4[k] & 0xffff0000u);
        const float hi = e == 0 ? __uint_as_float(hi4[k] << 16)
                                : __uint_as_float(hi4[k] & 0xffff0000u);
        const float s = sn[2 * k + e], c = cs[2 * k + e];
        vlo[e] = round_to_bf16(lo * c) - round_to_bf16(hi * s);
        vhi[e] = round_to_bf16(hi * c) + round_to_bf16(lo * s);
      }
      olo[k] = pack_bf16x2(vlo[0], vlo[1]);
      ohi[k] = pack_bf16x2(vhi[0], vhi[1]);
    }
    *reinterpret_cast<u32x4*>(dst) = olo;
    *reinterpret_cast<u32x4*>(dst + quarter) = ohi;
  };
  for (int h = 0; h < n; ++h) {
    const int64_t at = (row * n + h) * hd + i0;
    rotate(x + at, out + at);
  }
  for (int h = 0; h < n2; ++h) {
    const int64_t at = (row * n2 + h) * hd + i0;
    rotate(x2 + at, out2 + at);
  }
}

__device__ __forceinline__ float block_reduce(float v, float* scratch,
                                              bool take_max) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = take_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads();  // scratch may still be read from the previous reduction
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  const float a = scratch[0], b = scratch[1], c = scratch[2], d = scratch[3];
  return take_max ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : (a + b) + (c + d);
}

// One workgroup per (row, head).  scores [B, heads, window]: q . k of the ring
// slots as the caller's batched product left them (activation dtype,
// unscaled); q [B, heads, hd], k_new [B, hd] (both after the rotary
// embedding); num_tokens [B] tokens seen before this one; probs
// [B, heads, window + 1]: softmax over the visible ring slots and, last
// column, the new token itself.  Slot j holds the largest position congruent
// to j below num_tokens, so it is visible iff it was ever written: j <
// num_tokens, or the ring has wrapped.
template <typename T>
__global__ void __launch_bounds__(256)
attn_decode_probs_kernel(const T* __restrict__ scores, const T* __restrict__ q,
                         const T* __restrict__ k_new,
                         const int32_t* __restrict__ num_tokens,
                         T* __restrict__ probs, int heads, int hd, int window,
                         float scale) {
  __shared__ float scratch[4];
  const int b = blockIdx.x / heads;
  const int nt = num_tokens[b];
  const T* srow = scores + (int64_t)blockIdx.x * window;
  const T* qrow = q + (int64_t)blockIdx.x * hd;
  const T* krow = k_new + (int64_t)b * hd;
  T* prow = probs + (int64_t)blockIdx.x * (window + 1);
  float dot = 0.0f;
  for (int d = threadIdx.x; d < hd; d += 256)
    dot += load_scalar<T>(qrow + d) * load_scalar<T>(krow + d);
  dot = block_reduce(dot, scratch, false);
  const float self = round_act<T>(round_act<T>(dot) * scale);
  const bool wrapped = nt >= window;
  if (window <= 8 * 256) {
    // the usual window (2048): every thread keeps its eight scores, read once
    float sv[8];
    float mx = self;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = threadIdx.x + 256 * i;
      const bool visible = j < window && (wrapped || j < nt);
      sv[i] = visible ? round_act<T>(load_scalar<T>(srow + (j < window ? j : 0)) *
                                     scale)
                      : -__builtin_inff();
      mx = fmaxf(mx, sv[i]);
    }
    mx = block_reduce(mx, scratch, true);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      sv[i] = expf(sv[i] - mx);  // (exp(-inf) = 0 for the slots not visible)
      sum += sv[i];
    }
    const float self_e = expf(self - mx);
    if (threadIdx.x == 0) sum += self_e;
    sum = block_reduce(sum, scratch, false);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = threadIdx.x + 256 * i;
      if (j < window) store_scalar<T>(prow + j, sv[i] * inv);
    }
    if (threadIdx.x == 0) store_scalar<T>(prow + window, self_e * inv);
    return;
  }
  float mx = self;
  for (int j = threadIdx.x; j < window; j += 256)
    if (wrapped || j < nt)
      mx = fmaxf(mx, round_act<T>(load_scalar<T>(srow + j) * scale));
  mx = block_reduce(mx, scratch, true);
  float sum = 0.0f;
  for (int j = threadIdx.x; j < window; j += 256)
    if (wrapped || j < nt)
      sum += expf(round_act<T>(load_scalar<T>(srow + j) * scale) - mx);
  if (threadIdx.x == 0) sum += expf(self - mx);
  sum = block_reduce(sum, scratch, false);
  const float inv = 1.0f / sum;
  for (int j = threadIdx.x; j < window; j += 256) {
    float p = 0.0f;
    if (wrapped || j < nt)
      p = expf(round_act<T>(load_scalar<T>(srow + j) * scale) - mx) * inv;
    store_scalar<T>(prow + j, p);
  }
  if (threadIdx.x == 0) store_scalar<T>(prow + window, expf(self - mx) * inv);
}

// One workgroup per row.  from_ring [B, heads, hd]: probs[..., :window] times
// the ring's values (the caller's batched product); adds the new token's share
// probs[..., window] * v_new, then (update != 0) stores the new key and value
// in slot num_tokens % window and counts the token.
template <typename T>
__global__ void __launch_bounds__(256)
attn_decode_finish_kernel(const T* __restrict__ from_ring,
                          const T* __restrict__ probs,
                          const T* __restrict__ k_new,
                          const T* __restrict__ v_new, T* __restrict__ out,
                          T* __restrict__ ring_k, T* __restrict__ ring_v,
                          int32_t* __restrict__ num_tokens, int heads, int hd,
                          int window, int update) {
  const int b = blockIdx.x;
  const int nt = num_tokens[b];
  const T* vrow = v_new + (int64_t)b * hd;
  for (int e = threadIdx.x; e < heads * hd; e += 256) {
    const int h = e / hd, d = e % hd;
    const float p = load_scalar<T>(
        probs + ((int64_t)b * heads + h) * (window + 1) + window);
    const int64_t at = (int64_t)b * heads * hd + e;
    store_scalar<T>(out + at, load_scalar<T>(from_ring + at) +
                                  round_act<T>(p * load_scalar<T>(vrow + d)));
  }
  if (!update) return;
  const int64_t slot = ((int64_t)b * window + nt % window) * hd;
  for (int d = threadIdx.x; d < hd; d += 256) {
    ring_k[slot + d] = k_new[(int64_t)b * hd + d];
    ring_v[slot + d] = vrow[d];
  }
  __syncthreads();  // every thread has read num_tokens[b]
  if (threadIdx.x == 0) num_tokens[b] = nt + 1;
}

template <typename F>
hipError_t by_dtype(int dtype, F&& f) {
  if (dtype == 0) f((float*)nullptr);
  else f((uint16_t*)nullptr);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_rope(const void* x, const void* pos, int pos_kind,
                       const float* inv_freq, void* out, int64_t rows, int n,
                       int hd, const void* x2, void* out2, int n2, int dtype,
                       hipStream_t s) {
  const int64_t total = rows * n * hd;
  const int64_t total2 = x2 ? rows * n2 * hd : 0;
  const bool aligned = (((uintptr_t)x | (uintptr_t)out | (uintptr_t)x2 |
                         (uintptr_t)out2) & 15) == 0;
  if (dtype != 0 && hd % 32 == 0 && aligned) {
    const int64_t items = rows * (hd / 32 + hd / 16);
    const int64_t vblocks = (items + 255) / 256;
    if (vblocks > 0x7fffffff) return hipErrorInvalidValue;
    rope_bf16_vec_kernel<<<dim3((unsigned)vblocks), 256, 0, s>>>(
        (const uint16_t*)x, pos, pos_kind, inv_freq, (uint16_t*)out, rows, n,
        hd, (const uint16_t*)x2, (uint16_t*)out2, x2 ? n2 : 0);
    return hipGetLastError();
  }
  const int64_t blocks = (total + total2 + 255) / 256;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  return by_dtype(dtype, [&](auto* tag) {
    typedef std::remove_pointer_t<decltype(tag)> T;
    rope_kernel<T><<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const T*)x, pos, pos_kind, inv_freq, (T*)out, total, n, hd,
        (const T*)x2, (T*)out2, total2, n2);
  });
}

hipError_t launch_attn_decode_probs(const void* scores, const void* q,
                                    const void* k_new,
                                    const int32_t* num_tokens, void* probs,
                                    int B, int heads, int hd, int window,
                                    float scale, int dtype, hipStream_t s) {
  return by_dtype(dtype, [&](auto* tag) {
    typedef std::remove_pointer_t<decltype(tag)> T;
    attn_decode_probs_kernel<T><<<dim3((unsigned)(B * heads)), 256, 0, s>>>(
        (const T*)scores, (const T*)q, (const T*)k_new, num_tokens, (T*)probs,
        heads, hd, window, scale);
  });
}

hipError_t launch_attn_decode_finish(const void* from_ring, const void* probs,
                                     const void* k_new, const void* v_new,
                                     void* out, void* ring_k, void* ring_v,
                                     int32_t* num_tokens, int B, int heads,
                                     int hd, int window, int update, int dtype,
                                     hipStream_t s) {
  return by_dtype(dtype, [&](auto* tag) {
    typedef std::remove_pointer_t<decltype(tag)> T;
    attn_decode_finish_kernel<T><<<dim3((unsigned)B), 256, 0, s>>>(
        (const T*)from_ring, (const T*)probs, (const T*)k_new, (const T*)v_new,
        (T*)out, (T*)ring_k, (T*)ring_v, num_tokens, heads, hd, window, update);
  });
}

}  // namespace rg
