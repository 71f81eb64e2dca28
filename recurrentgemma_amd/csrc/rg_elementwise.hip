// out = a * gelu_tanh(g): the join of the two branches of the recurrent block
// (recurrentgemma/torch/modules.py:627-628 `y = gelu(linear_y(x))`, :289-291
// the tanh approximation, :644 `x = x * y`), one pass instead of torch's gelu
// pass plus multiply pass.  `a` is the RG-LRU output, `g` the linear_y output.
#include <type_traits>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {


// bf16: gelu_mul_bf16 per element, the product rounded once.
// One 16-byte item (eight elements) per thread, streaming loads and stores, no
// loop: measured at 2^29 elements this shape (2^18 workgroups, each one
// contiguous 4 KB of every operand) moves 6.4 TB/s, a grid-stride loop over
// 8192 workgroups 4.7 TB/s.
__global__ void __launch_bounds__(256)
gelu_mul_bf16_kernel(const u32x4* a, const u32x4* __restrict__ g, u32x4* out,
                     int64_t n8,
                     const uint16_t* a_tail, const uint16_t* g_tail,
                     uint16_t* out_tail, int tail) {
  auto one = [](float av, float gv) { return gelu_mul_bf16(av, gv); };
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n8) {
    const u32x4 av = __builtin_nontemporal_load(a + i);
    const u32x4 gv = __builtin_nontemporal_load(g + i);
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = one(__uint_as_float(av[k] << 16),
                           __uint_as_float(gv[k] << 16));
      const float hi = one(__uint_as_float(av[k] & 0xffff0000u),
                           __uint_as_float(gv[k] & 0xffff0000u));
      o[k] = pack_bf16x2(lo, hi);
    }
    __builtin_nontemporal_store(o, out + i);
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < tail)
    out_tail[threadIdx.x] = f32_to_bf16_bits(
        one(bf16_bits_to_f32(a_tail[threadIdx.x]),
            bf16_bits_to_f32(g_tail[threadIdx.x])));
}

// float32: the reference's own formula; four elements per thread.
__global__ void __launch_bounds__(256)
gelu_mul_f32_kernel(const f32x4* a, const f32x4* __restrict__ g, f32x4* out,
                    int64_t n4, const float* a_tail,
                    const float* g_tail, float* out_tail, int tail) {
  auto one = [](float av, float gv) { return gelu_mul_f32(av, gv); };
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n4) {
    const f32x4 av = __builtin_nontemporal_load(a + i);
    const f32x4 gv = __builtin_nontemporal_load(g + i);
    f32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = one(av[k], gv[k]);
    __builtin_nontemporal_store(o, out + i);
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < tail)
    out_tail[threadIdx.x] = one(a_tail[threadIdx.x], g_tail[threadIdx.x]);
}

// The backward pass of the join, out = a * gelu_tanh(g) (modules.py:289-291,
// :627-628, :644), one pass over the three operands:
//   d_a = dout * gelu(g)
//   d_g = (dout * a) * gelu'(g),
//   gelu'(g) = 0.5 (1 + t) + 0.5 g (1 - t^2) sqrt(2/pi) (1 + 3 c1 g^2),
//   t = tanh(sqrt(2/pi) (g + c1 g^3)).
// bf16: gelu(g) and dout * a are rounded to bf16 first, as the tensors they
// are when autograd walks the reference's two ops; each output is rounded
// once.
template <bool BF16>
__device__ __forceinline__ void gelu_mul_backward_one(float dv, float av,
                                                      float gv, float& da,
                                                      float& dg) {
  constexpr float c0 = 0.7978845608028654f;  // sqrt(2/pi)
  constexpr float c1 = 0.044715f;
  const float g2 = gv * gv;
  const float u = c0 * __builtin_fmaf(c1 * g2, gv, gv);
  const float t = BF16 ? __builtin_fmaf(2.0f, sigmoid_fast(2.0f * u), -1.0f)
                       : tanhf(u);
  const float half_g = 0.5f * gv;
  const float gelu = half_g * (1.0f + t);
  const float slope = __builtin_fmaf(
      half_g * __builtin_fmaf(-t, t, 1.0f),
      c0 * __builtin_fmaf(3.0f * c1, g2, 1.0f), 0.5f * (1.0f + t));
  da = dv * (BF16 ? round_to_bf16(gelu) : gelu);
  dg = (BF16 ? round_to_bf16(dv * av) : dv * av) * slope;
}

__global__ void __launch_bounds__(256)
gelu_mul_backward_bf16_kernel(const u32x4* __restrict__ dout,
                              const u32x4* __restrict__ a,
                              const u32x4* __restrict__ g, u32x4* d_a,
                              u32x4* d_g, int64_t n8, const uint16_t* dout_tail,
                              const uint16_t* a_tail, const uint16_t* g_tail,
                              uint16_t* d_a_tail, uint16_t* d_g_tail,
                              int tail) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n8) {
    const u32x4 dv = __builtin_nontemporal_load(dout + i);
    const u32x4 av = __builtin_nontemporal_load(a + i);
    const u32x4 gv = __builtin_nontemporal_load(g + i);
    u32x4 oa, og;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float da_lo, dg_lo, da_hi, dg_hi;
      gelu_mul_backward_one<true>(__uint_as_float(dv[k] << 16),
                                  __uint_as_float(av[k] << 16),
                                  __uint_as_float(gv[k] << 16), da_lo, dg_lo);
      gelu_mul_backward_one<true>(__uint_as_float(dv[k] & 0xffff0000u),
                                  __uint_as_float(av[k] & 0xffff0000u),
                                  __uint_as_float(gv[k] & 0xffff0000u), da_hi,
                                  dg_hi);
      oa[k] = pack_bf16x2(da_lo, da_hi);
      og[k] = pack_bf16x2(dg_lo, dg_hi);
    }
    __builtin_nontemporal_store(oa, d_a + i);
    __builtin_nontemporal_store(og, d_g + i);
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < tail) {
    float da, dg;
    gelu_mul_backward_one<true>(bf16_bits_to_f32(dout_tail[threadIdx.x]),
                                bf16_bits_to_f32(a_tail[threadIdx.x]),
                                bf16_bits_to_f32(g_tail[threadIdx.x]), da, dg);
    d_a_tail[threadIdx.x] = f32_to_bf16_bits(da);
    d_g_tail[threadIdx.x] = f32_to_bf16_bits(dg);
  }
}

__global__ void __launch_bounds__(256)
gelu_mul_backward_f32_kernel(const f32x4* __restrict__ dout,
                             const f32x4* __restrict__ a,
                             const f32x4* __restrict__ g, f32x4* d_a,
                             f32x4* d_g, int64_t n4, const float* dout_tail,
                             const float* a_tail, const float* g_tail,
                             float* d_a_tail, float* d_g_tail, int tail) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n4) {
    const f32x4 dv = __builtin_nontemporal_load(dout + i);
    const f32x4 av = __builtin_nontemporal_load(a + i);
    const f32x4 gv = __builtin_nontemporal_load(g + i);
    f32x4 oa, og;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      float da, dg;
      gelu_mul_backward_one<false>(dv[k], av[k], gv[k], da, dg);
      oa[k] = da;
      og[k] = dg;
    }
    __builtin_nontemporal_store(oa, d_a + i);
    __builtin_nontemporal_store(og, d_g + i);
  }
  if (blockIdx.x == 0 && (int)threadIdx.x < tail)
    gelu_mul_backward_one<false>(dout_tail[threadIdx.x], a_tail[threadIdx.x],
                                 g_tail[threadIdx.x], d_a_tail[threadIdx.x],
                                 d_g_tail[threadIdx.x]);
}

// RMSNorm of the residual stack (recurrentgemma/torch/layers.py:65-73):
//   var = mean(x^2);  out = x * rsqrt(var + eps) * (scale + 1)
// with every step rounded to the activation dtype like the reference's chain
// of tensor ops (for bf16: x^2, the mean, var + eps, the rsqrt, x * rsqrt and
// scale + 1 are each a bf16 tensor there; sums accumulate in float32).  One
// workgroup per row; the row is read twice, the second time from cache.
// ADD: the row normalised is x + addend (rounded to the activation dtype, the
// residual sum of the block, recurrentgemma/torch/modules.py:893-896), which
// is also written to `sum_out`.
template <typename T, bool ADD>
__global__ void __launch_bounds__(256)
rms_norm_kernel(const T* __restrict__ x, const T* __restrict__ addend,
                const T* __restrict__ scale, T* __restrict__ sum_out,
                T* __restrict__ out, int width, float eps) {
  __shared__ float partial[4];
  const int64_t row = (int64_t)blockIdx.x * width;
  const T* xr = x + row;
  T* outr = out + row;
  float sum = 0.0f;
  for (int i = threadIdx.x; i < width; i += 256) {
    float v = load_scalar<T>(xr + i);
    if (ADD) {
      v = round_act<T>(v + load_scalar<T>(addend + row + i));
      store_scalar<T>(sum_out + row + i, v);
    }
    sum += round_act<T>(v * v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
  __syncthreads();
  sum = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float var = round_act<T>(sum * (1.0f / (float)width));
  const float r = round_act<T>(1.0f / sqrtf(round_act<T>(var + eps)));
  for (int i = threadIdx.x; i < width; i += 256) {
    // (with ADD each thread re-reads the sums it stored itself)
    const float v = load_scalar<T>((ADD ? sum_out + row : xr) + i);
    const float g = round_act<T>(load_scalar<T>(scale + i) + 1.0f);
    store_scalar<T>(outr + i, round_act<T>(v * r) * g);
  }
}

// bf16 rows of up to 4096 elements whose width is a multiple of 8: 16-byte
// lanes, the row stays in registers between the two passes (one read, one
// write; the scalar kernel above re-reads through the cache and moved
// 1.7 TB/s on 131 072 rows of 2560).
// The row a linear layer left as fp32 partial sums over slices of its K
// (rg_linear.hip): x = round(sum of the slices, in slice order, + bias).
struct PartialRows {
  const f32x4* sums;     // [slices][rows][width]
  int slices;
  int64_t slice_stride;  // rows * width / 4
  const u32x4* bias;     // [width] or null
};

template <bool ADD, bool FROM_PARTIAL>
__global__ void __launch_bounds__(256)
rms_norm_bf16_rows_kernel(const u32x4* __restrict__ x, PartialRows part,
                          const u32x4* __restrict__ addend,
                          const u32x4* __restrict__ scale,
                          u32x4* __restrict__ sum_out,
                          u32x4* __restrict__ out, int chunks, float inv_width,
                          float eps) {
  __shared__ float partial[4];
  const int64_t row = (int64_t)blockIdx.x * chunks;
  const u32x4* xr = x + row;
  u32x4* outr = out + row;
  u32x4 v[2];
  float sum = 0.0f;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int i = threadIdx.x + c * 256;
    v[c] = u32x4{0u, 0u, 0u, 0u};
    if (!FROM_PARTIAL && i < chunks) v[c] = __builtin_nontemporal_load(xr + i);
    if (FROM_PARTIAL && i < chunks) {
      f32x4 lo = {0.0f, 0.0f, 0.0f, 0.0f}, hi = lo;
      const f32x4* src = part.sums + (row + i) * 2;
      for (int s = 0; s < part.slices; ++s) {
        lo += src[s * part.slice_stride];
        hi += src[s * part.slice_stride + 1];
      }
      if (part.bias) {
        const u32x4 b = part.bias[i];
        lo += f32x4{__uint_as_float(b[0] << 16),
                    __uint_as_float(b[0] & 0xffff0000u),
                    __uint_as_float(b[1] << 16),
                    __uint_as_float(b[1] & 0xffff0000u)};
        hi += f32x4{__uint_as_float(b[2] << 16),
                    __uint_as_float(b[2] & 0xffff0000u),
                    __uint_as_float(b[3] << 16),
                    __uint_as_float(b[3] & 0xffff0000u)};
      }
      v[c] = u32x4{pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]),
                   pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3])};
      if (!ADD) sum_out[row + i] = v[c];
    }
    if (ADD && i < chunks) {
      const u32x4 w = __builtin_nontemporal_load(addend + row + i);
#pragma unroll
      for (int k = 0; k < 4; ++k)
        v[c][k] = pack_bf16x2(
            __uint_as_float(v[c][k] << 16) + __uint_as_float(w[k] << 16),
            __uint_as_float(v[c][k] & 0xffff0000u) +
                __uint_as_float(w[k] & 0xffff0000u));
      sum_out[row + i] = v[c];
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = __uint_as_float(v[c][k] << 16);
      const float hi = __uint_as_float(v[c][k] & 0xffff0000u);
      sum += round_to_bf16(lo * lo);
      sum += round_to_bf16(hi * hi);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
  __syncthreads();
  sum = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float var = round_to_bf16(sum * inv_width);
  const float r = round_to_bf16(1.0f / sqrtf(round_to_bf16(var + eps)));
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int i = threadIdx.x + c * 256;
    if (i >= chunks) continue;
    const u32x4 g = scale[i];
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = round_to_bf16(__uint_as_float(v[c][k] << 16) * r) *
                       round_to_bf16(__uint_as_float(g[k] << 16) + 1.0f);
      const float hi =
          round_to_bf16(__uint_as_float(v[c][k] & 0xffff0000u) * r) *
          round_to_bf16(__uint_as_float(g[k] & 0xffff0000u) + 1.0f);
      o[k] = pack_bf16x2(lo, hi);
    }
    __builtin_nontemporal_store(o, outr + i);
  }
}

// Soft cap of the logits (recurrentgemma/torch/griffin.py:203-206
// `logits = tanh(logits / cap) * cap`): torch's three kernels in one, with
// their roundings (the quotient -- torch multiplies by the reciprocal of a
// scalar divisor --, the tanh and the product each rounded to the dtype).
template <typename T>
__global__ void __launch_bounds__(256)
soft_cap_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t n,
                float inv_cap, float cap) {
  constexpr int kPer = 16 / sizeof(T);
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * kPer;
  auto one = [&](float v) {
    v = round_act<T>(v * inv_cap);
    v = round_act<T>(tanhf(v));
    return round_act<T>(v * cap);
  };
  if (i0 + kPer <= n) {
    alignas(16) T in[kPer];
    alignas(16) T o[kPer];
    *reinterpret_cast<u32x4*>(in) =
        __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + i0));
#pragma unroll
    for (int k = 0; k < kPer; ++k) store_scalar<T>(o + k, one(load_scalar<T>(in + k)));
    __builtin_nontemporal_store(*reinterpret_cast<u32x4*>(o),
                                reinterpret_cast<u32x4*>(out + i0));
  } else {
    for (int64_t i = i0; i < n; ++i)
      store_scalar<T>(out + i, one(load_scalar<T>(x + i)));
  }
}

// Index of the largest element of every row (the first one among equals, a NaN
// counts as larger than everything: torch.argmax's rule; greedy sampling,
// recurrentgemma/torch/sampler.py:126-128).  One workgroup per row.
template <typename T>
__global__ void __launch_bounds__(1024)
argmax_rows_kernel(const T* __restrict__ x, int64_t* __restrict__ out, int n) {
  __shared__ float best_v[16];
  __shared__ int best_i[16];
  const T* row = x + (int64_t)blockIdx.x * n;
  float bv = 0.0f;
  int bi = 0x7fffffff;
  // a beats b: larger, or NaN where b is not; equal values keep the lower index
  auto better = [](float v, int i, float w, int j) {
    if (j == 0x7fffffff) return true;
    const bool vn = v != v, wn = w != w;
    if (vn || wn) return vn && (!wn || i < j);
    return v > w || (v == w && i < j);
  };
  constexpr int kPer = 16 / sizeof(T);
  const int vec_n = ((reinterpret_cast<uintptr_t>(row) & 15) == 0) ? n / kPer : 0;
  for (int c = threadIdx.x; c < vec_n; c += 1024) {
    alignas(16) T in[kPer];
    *reinterpret_cast<u32x4*>(in) =
        __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(row) + c);
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
      const float v = load_scalar<T>(in + k);
      if (better(v, c * kPer + k, bv, bi)) {
        bv = v;
        bi = c * kPer + k;
      }
    }
  }
  for (int i = vec_n * kPer + threadIdx.x; i < n; i += 1024) {
    const float v = load_scalar<T>(row + i);
    if (better(v, i, bv, bi)) {
      bv = v;
      bi = i;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    if (oi != 0x7fffffff && better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    best_v[threadIdx.x >> 6] = bv;
    best_i[threadIdx.x >> 6] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w)
      if (best_i[w] != 0x7fffffff && better(best_v[w], best_i[w], bv, bi)) {
        bv = best_v[w];
        bi = best_i[w];
      }
    out[blockIdx.x] = bi;
  }
}

}  // namespace

hipError_t launch_soft_cap(const void* x, void* out, int64_t n, float cap,
                           int dtype, hipStream_t s) {
  const int per = dtype == 0 ? 4 : 8;
  const int64_t blocks = ((n + per - 1) / per + 255) / 256;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  const float inv = 1.0f / cap;
  if (dtype == 0)
    soft_cap_kernel<float><<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const float*)x, (float*)out, n, inv, cap);
  else
    soft_cap_kernel<uint16_t><<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const uint16_t*)x, (uint16_t*)out, n, inv, cap);
  return hipGetLastError();
}

hipError_t launch_argmax_rows(const void* x, int64_t* out, int rows, int n,
                              int dtype, hipStream_t s) {
  if (dtype == 0)
    argmax_rows_kernel<float><<<dim3((unsigned)rows), 1024, 0, s>>>(
        (const float*)x, out, n);
  else
    argmax_rows_kernel<uint16_t><<<dim3((unsigned)rows), 1024, 0, s>>>(
        (const uint16_t*)x, out, n);
  return hipGetLastError();
}

hipError_t launch_gelu_mul(const void* a, const void* g, void* out, int64_t n,
                           int dtype, hipStream_t s) {
  const int per = dtype == 0 ? 4 : 8;  // elements per 16-byte item
  const int64_t items = n / per;
  const int tail = (int)(n - items * per);
  const int64_t blocks = items > 0 ? (items + 255) / 256 : 1;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  if (dtype == 0) {
    gelu_mul_f32_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const f32x4*)a, (const f32x4*)g, (f32x4*)out, items,
        (const float*)a + items * per, (const float*)g + items * per,
        (float*)out + items * per, tail);
  } else {
    gelu_mul_bf16_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const u32x4*)a, (const u32x4*)g, (u32x4*)out, items,
        (const uint16_t*)a + items * per, (const uint16_t*)g + items * per,
        (uint16_t*)out + items * per, tail);
  }
  return hipGetLastError();
}

hipError_t launch_gelu_mul_backward(const void* dout, const void* a,
                                    const void* g, void* d_a, void* d_g,
                                    int64_t n, int dtype, hipStream_t s) {
  const int per = dtype == 0 ? 4 : 8;  // elements per 16-byte item
  const int64_t items = n / per;
  const int tail = (int)(n - items * per);
  const int64_t blocks = items > 0 ? (items + 255) / 256 : 1;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  const int64_t done = items * per;
  if (dtype == 0) {
    gelu_mul_backward_f32_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const f32x4*)dout, (const f32x4*)a, (const f32x4*)g, (f32x4*)d_a,
        (f32x4*)d_g, items, (const float*)dout + done, (const float*)a + done,
        (const float*)g + done, (float*)d_a + done, (float*)d_g + done, tail);
  } else {
    gelu_mul_backward_bf16_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const u32x4*)dout, (const u32x4*)a, (const u32x4*)g, (u32x4*)d_a,
        (u32x4*)d_g, items, (const uint16_t*)dout + done,
        (const uint16_t*)a + done, (const uint16_t*)g + done,
        (uint16_t*)d_a + done, (uint16_t*)d_g + done, tail);
  }
  return hipGetLastError();
}

hipError_t launch_rms_norm(const void* x, const void* addend, const void* scale,
                           void* sum_out, void* out, int64_t rows, int width,
                           float eps, int dtype, hipStream_t s) {
  if (rows > 0x7fffffff) return hipErrorInvalidValue;
  const bool add = addend != nullptr;
  const bool aligned = (((uintptr_t)x | (uintptr_t)addend | (uintptr_t)scale |
                         (uintptr_t)sum_out | (uintptr_t)out) & 15) == 0;
  const dim3 grid((unsigned)rows);
  if (dtype != 0 && width % 8 == 0 && width <= 4096 && aligned) {
    const int chunks = width / 8;
    const float inv = 1.0f / (float)width;
    const PartialRows none{};
    if (add)
      rms_norm_bf16_rows_kernel<true, false><<<grid, 256, 0, s>>>(
          (const u32x4*)x, none, (const u32x4*)addend, (const u32x4*)scale,
          (u32x4*)sum_out, (u32x4*)out, chunks, inv, eps);
    else
      rms_norm_bf16_rows_kernel<false, false><<<grid, 256, 0, s>>>(
          (const u32x4*)x, none, nullptr, (const u32x4*)scale, nullptr,
          (u32x4*)out, chunks, inv, eps);
    return hipGetLastError();
  }
  auto run = [&](auto* tag) {
    typedef std::remove_pointer_t<decltype(tag)> T;
    if (add)
      rms_norm_kernel<T, true><<<grid, 256, 0, s>>>(
          (const T*)x, (const T*)addend, (const T*)scale, (T*)sum_out, (T*)out,
          width, eps);
    else
      rms_norm_kernel<T, false><<<grid, 256, 0, s>>>(
          (const T*)x, nullptr, (const T*)scale, nullptr, (T*)out, width, eps);
  };
  if (dtype == 0) run((float*)nullptr);
  else run((uint16_t*)nullptr);
  return hipGetLastError();
}

// bf16 rows given as partial sums; the caller has checked width % 8 == 0,
// width <= 4096 and 16-byte alignment.
hipError_t launch_rms_norm_partial(const float* sums, int slices,
                                   const void* bias, const void* addend,
                                   const void* scale, void* sum_out, void* out,
                                   int rows, int width, float eps,
                                   hipStream_t s) {
  const int chunks = width / 8;
  const float inv = 1.0f / (float)width;
  PartialRows part;
  part.sums = (const f32x4*)sums;
  part.slices = slices;
  part.slice_stride = (int64_t)rows * width / 4;
  part.bias = (const u32x4*)bias;
  const dim3 grid((unsigned)rows);
  if (addend)
    rms_norm_bf16_rows_kernel<true, true><<<grid, 256, 0, s>>>(
        nullptr, part, (const u32x4*)addend, (const u32x4*)scale,
        (u32x4*)sum_out, (u32x4*)out, chunks, inv, eps);
  else
    rms_norm_bf16_rows_kernel<false, true><<<grid, 256, 0, s>>>(
        nullptr, part, nullptr, (const u32x4*)scale, (u32x4*)sum_out,
        (u32x4*)out, chunks, inv, eps);
  return hipGetLastError();
}


// ------------------------------------------------------------ clock probe ----
// One wave per CU spins through `iters` rounds of 64 dependent fused
// multiply-adds and notes the shader-clock counter (s_memtime) and the
// constant 100 MHz counter (s_memrealtime) before and after: their ratio is
// the shader clock the GPU runs at right now.  out[0] = shader cycles, out[1] =
// 10 ns ticks (workgroup 0's).
namespace {
__global__ void __launch_bounds__(64) clock_probe_kernel(uint64_t* out,
                                                         int iters) {
  float v = (float)threadIdx.x;
  const uint64_t c0 = __builtin_readcyclecounter();
  const uint64_t r0 = __builtin_amdgcn_s_memrealtime();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int j = 0; j < 64; ++j) v = __builtin_fmaf(v, 0.999f, 0.5f);
    asm volatile("" : "+v"(v));
  }
  const uint64_t c1 = __builtin_readcyclecounter();
  const uint64_t r1 = __builtin_amdgcn_s_memrealtime();
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    out[0] = c1 - c0;
    out[1] = r1 - r0;
    out[2] = (uint64_t)__float_as_uint(v);  // keeps the loop
  }
}
}  // namespace

hipError_t launch_clock_probe(uint64_t* out, int iters, hipStream_t s) {
  clock_probe_kernel<<<256, 64, 0, s>>>(out, iters);
  return hipGetLastError();
}

}  // namespace rg
