// One decoded token of the local-attention block against its ring cache
// (recurrentgemma/torch/modules.py:431-476 with the cache of :152-216), bf16,
// head_dim 256, one shared key/value head: rotary embedding, scores, mask,
// softmax, weighted sum of the values, the new token's own share, ring
// update and token count in two launches that read the ring once.
//
//   attn_decode_chunks_kernel   one workgroup per (row, 256 ring slots); a wave
//       owns 64 slots and walks them in passes of 16: keys and values come
//       from HBM through registers into a wave-private LDS tile; scores
//       S^T = K Q^T on v_mfma_f32_16x16x32_bf16 with the (at most 16) query
//       heads as result columns, so a lane holds four scores of one head,
//       which are, as they lie, its operand of O^T += V^T P^T on
//       v_mfma_f32_16x16x16_bf16; running maximum and sum per head as in any
//       streaming softmax.  The four waves meet in LDS; the chunk leaves its
//       unnormalised sum [heads, 256] with its maximum and denominator.
//   attn_decode_combine_kernel  one workgroup per (head, row): the new
//       token's own score, the chunks weighed against the common maximum, the
//       new token's share, output; then the ring slot and the token count.
//
// Roundings follow the reference's chain of tensor ops where a streaming
// softmax can: scores rounded to bf16, scaled, rounded; softmax in float32;
// probabilities enter the second product as bf16 (unnormalised here,
// normalised there); the sum over the ring rounded to bf16 before the new
// token's rounded share is added.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));

constexpr int kHd = 256;             // head dimension
constexpr int kSlots = kAttnDecodeChunk;  // ring slots per workgroup (256)
constexpr int kWaveSlots = kSlots / 4;    // per wave
constexpr int kPass = 16;            // slots per pass of a wave
constexpr int kPasses = kWaveSlots / kPass;
constexpr int kRowBytes = 528;       // a staged row: 512 bytes + 16 of padding
constexpr int kTileBytes = kPass * kRowBytes;
constexpr int kQBytes = 16 * kRowBytes;   // the queries after the rotary
                                          // embedding, 16 head rows
constexpr int kSumStride = 17;       // floats per row of a wave's O^T in LDS
constexpr int kWaveBytes = kHd * kSumStride * 4;  // >= 2 tiles
static_assert(kWaveBytes >= 2 * kTileBytes, "a wave's tiles share its area");
constexpr int kStatsOff = kQBytes + 4 * kWaveBytes;
constexpr int kChunkLdsBytes = kStatsOff + 4 * 16 * 2 * 4;
constexpr float kNegInf = -__builtin_inff();

__device__ __forceinline__ float position_of_row(const void* pos, int kind,
                                                 int64_t i) {
  return kind == kSegI64 ? (float)reinterpret_cast<const int64_t*>(pos)[i]
                         : (float)reinterpret_cast<const int32_t*>(pos)[i];
}

// LDS traffic between the lanes of one wave: the unit executes a wave's
// instructions in order; this keeps the compiler from reordering them.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Rotary embedding of eight elements i0 .. i0+7 of the first quarter of a
// head with their partners in the second (recurrentgemma/torch/modules.py:
// 52-83; the arithmetic of rope_bf16_vec_kernel, element for element).
__device__ __forceinline__ void rotate8(u32x4 lo4, u32x4 hi4, float position,
                                        const float* inv_freq, int i0,
                                        u32x4& olo, u32x4& ohi) {
#pragma clang fp contract(off)
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    float vlo[2], vhi[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const float lo = e == 0 ? __uint_as_float(lo4[k] << 16)
                              : __uint_as_float(lo4[k] & 0xffff0000u);
      const float hi = e == 0 ? __uint_as_float(hi4[k] << 16)
                              : __uint_as_float(hi4[k] & 0xffff0000u);
      const float angle = position * inv_freq[i0 + 2 * k + e];
      const float s = round_to_bf16(sinf(angle)), c = round_to_bf16(cosf(angle));
      vlo[e] = round_to_bf16(lo * c) - round_to_bf16(hi * s);
      vhi[e] = round_to_bf16(hi * c) + round_to_bf16(lo * s);
    }
    olo[k] = pack_bf16x2(vlo[0], vlo[1]);
    ohi[k] = pack_bf16x2(vhi[0], vhi[1]);
  }
}

__global__ void __launch_bounds__(256, 2)
attn_decode_chunks_kernel(AttnDecodeArgs p) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c = blockIdx.x, b = blockIdx.y;
  const int nt = p.num_tokens[b];
  // slot j holds the largest position congruent to j below nt: visible iff
  // it was ever written
  const int visible_end = nt >= p.window ? p.window : nt;
  const int slot_first = c * kSlots;
  float* const ml = p.part_ml + ((int64_t)b * p.chunks + c) * p.heads * 2;
  if (slot_first >= visible_end) {  // nothing of this chunk is visible
    if (tid < p.heads) {
      ml[2 * tid] = kNegInf;
      ml[2 * tid + 1] = 0.0f;
    }
    return;
  }

  unsigned char* const ktile = lds + kQBytes + wave * kWaveBytes;
  unsigned char* const vtile = ktile + kTileBytes;
  const int wave_first = slot_first + wave * kWaveSlots;
  // passes with a visible slot (wave-uniform)
  int npass = (visible_end - wave_first + kPass - 1) / kPass;
  npass = npass < 0 ? 0 : (npass > kPasses ? kPasses : npass);

  // rows of the ring beyond the window read as zero (and are masked)
  const uint32_t ring_bytes = (uint32_t)p.window * (kHd * 2);
  const __amdgpu_buffer_rsrc_t rk =
      make_rsrc(p.ring_k + (int64_t)b * p.window * kHd, ring_bytes);
  const __amdgpu_buffer_rsrc_t rv =
      make_rsrc(p.ring_v + (int64_t)b * p.window * kHd, ring_bytes);
  // a load instruction covers two rows: lane -> row lane / 32, 16-byte piece
  // lane % 32
  const uint32_t lane_bytes = (uint32_t)(lane >> 5) * (kHd * 2) + 16u * (lane & 31);
  const uint32_t lane_lds = (uint32_t)(lane >> 5) * kRowBytes + 16u * (lane & 31);
  u32x4 kreg[8], vreg[8];
  auto request = [&](const __amdgpu_buffer_rsrc_t& r, u32x4 (&dst)[8], int pass) {
    const uint32_t row0 = (uint32_t)(wave_first + pass * kPass);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      dst[i] = __builtin_amdgcn_raw_buffer_load_b128(
          r, lane_bytes, (row0 + 2 * i) * (kHd * 2), 0);
  };
  auto to_tile = [&](unsigned char* tile, const u32x4 (&src)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      *reinterpret_cast<u32x4*>(tile + lane_lds + 2 * i * kRowBytes) = src[i];
  };

  // the first pass's keys and values are on their way while the queries are
  // rotated
  if (npass > 0) {
    request(rk, kreg, 0);
    request(rv, vreg, 0);
  }

  // ---- queries after the rotary embedding, 16 head rows (zeros past heads)
  {
    const uint16_t* qrow = p.q + (int64_t)b * p.ldq;
    const float position = position_of_row(p.pos, p.pos_kind, b);
    for (int item = tid; item < 16 * 24; item += 256) {
      const int head = item / 24, which = item - head * 24;
      unsigned char* dst = lds + head * kRowBytes;
      const u32x4 zero = {0, 0, 0, 0};
      if (which >= 8) {  // second half of the head: copied
        const int off = kHd / 2 + 8 * (which - 8);
        *reinterpret_cast<u32x4*>(dst + 2 * off) =
            head < p.heads
                ? *reinterpret_cast<const u32x4*>(qrow + head * kHd + off)
                : zero;
      } else {
        const int i0 = 8 * which;
        u32x4 olo = zero, ohi = zero;
        if (head < p.heads)
          rotate8(*reinterpret_cast<const u32x4*>(qrow + head * kHd + i0),
                  *reinterpret_cast<const u32x4*>(qrow + head * kHd + i0 +
                                                  kHd / 4),
                  position, p.inv_freq, i0, olo, ohi);
        *reinterpret_cast<u32x4*>(dst + 2 * i0) = olo;
        *reinterpret_cast<u32x4*>(dst + 2 * (i0 + kHd / 4)) = ohi;
      }
    }
  }
  __syncthreads();

  const int head = lane & 15;  // this lane's column of every result
  const int quad = lane >> 4;  // its group of four rows
  // the queries as the second operand of the scores: head `head`, elements
  // 32 ks + 8 quad + 0..7
  union Frag8 { u32x4 u; bf16x8 v; };
  union Frag4 { u32x2 u; bf16x4 v; };
  Frag8 qf[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks)
    qf[ks].u = *reinterpret_cast<const u32x4*>(lds + head * kRowBytes +
                                               2 * (32 * ks + 8 * quad));

  f32x4 o[16];  // O^T: rows 16 blk + 4 quad + r (head dimension), column head
#pragma unroll
  for (int blk = 0; blk < 16; ++blk) o[blk] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = kNegInf, l_run = 0.0f;

  for (int pass = 0; pass < npass; ++pass) {
    wave_lds_sync();  // the previous pass has read both tiles
    to_tile(ktile, kreg);
    if (pass + 1 < npass) request(rk, kreg, pass + 1);
    wave_lds_sync();
    // ---- scores of 16 slots x 16 heads
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      Frag8 a;
      a.u = *reinterpret_cast<const u32x4*>(ktile + head * kRowBytes +
                                            16 * (4 * ks + quad));
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, qf[ks].v, acc, 0, 0, 0);
    }
    // this lane: slots 4 quad + r of the pass, head `head`
    const int slot0 = wave_first + pass * kPass + 4 * quad;
    float s[4];
    float m_new = m_run;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s[r] = slot0 + r < visible_end
                 ? round_to_bf16(round_to_bf16(acc[r]) * p.scale)
                 : kNegInf;
      m_new = fmaxf(m_new, s[r]);
    }
    m_new = fmaxf(m_new, __shfl_xor(m_new, 16, 64));
    m_new = fmaxf(m_new, __shfl_xor(m_new, 32, 64));
    // (finite: the first slot of a pass that runs is visible)
    const float alpha = __expf(m_run - m_new);
    float pr[4], psum = 0.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pr[r] = __expf(s[r] - m_new);
      psum += pr[r];
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    Frag4 pf;
    pf.u[0] = pack_bf16x2(pr[0], pr[1]);
    pf.u[1] = pack_bf16x2(pr[2], pr[3]);
#pragma unroll
    for (int blk = 0; blk < 16; ++blk) o[blk] *= alpha;
    // ---- values of the same 16 slots
    to_tile(vtile, vreg);
    if (pass + 1 < npass) request(rv, vreg, pass + 1);
    wave_lds_sync();
    const unsigned char* vbase = vtile + 4 * quad * kRowBytes + 2 * head;
#pragma unroll
    for (int blk = 0; blk < 16; ++blk) {
      // V^T: row 16 blk + head (head dimension), slots 4 quad + 0..3
      uint32_t e[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        e[j] = *reinterpret_cast<const uint16_t*>(vbase + j * kRowBytes +
                                                  32 * blk);
      Frag4 a;
      a.u[0] = e[0] | (e[1] << 16);
      a.u[1] = e[2] | (e[3] << 16);
      o[blk] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a.v, pf.v, o[blk], 0,
                                                         0, 0);
    }
  }
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);

  // ---- the four waves meet
  float* const stats = reinterpret_cast<float*>(lds + kStatsOff);
  if (quad == 0) {
    stats[(wave * 16 + head) * 2] = m_run;
    stats[(wave * 16 + head) * 2 + 1] = l_run;
  }
  __syncthreads();  // also: every wave is done with its tiles
  float m_all = kNegInf;
#pragma unroll
  for (int w = 0; w < 4; ++w) m_all = fmaxf(m_all, stats[(w * 16 + head) * 2]);
  // (finite: wave 0's first slot is visible)
  const float f = __expf(m_run - m_all);
  float* const mine = reinterpret_cast<float*>(lds + kQBytes + wave * kWaveBytes);
#pragma unroll
  for (int blk = 0; blk < 16; ++blk)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      mine[(16 * blk + 4 * quad + r) * kSumStride + head] = o[blk][r] * f;
  __syncthreads();
  float* const po =
      p.part_o + ((int64_t)b * p.chunks + c) * p.heads * kHd + tid;
  for (int h = 0; h < p.heads; ++h) {
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w)
      sum += reinterpret_cast<const float*>(lds + kQBytes + w * kWaveBytes)
          [tid * kSumStride + h];
    po[h * kHd] = sum;
  }
  if (tid < p.heads) {
    float m = kNegInf, l = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) m = fmaxf(m, stats[(w * 16 + tid) * 2]);
#pragma unroll
    for (int w = 0; w < 4; ++w)
      l += __expf(stats[(w * 16 + tid) * 2] - m) * stats[(w * 16 + tid) * 2 + 1];
    ml[2 * tid] = m;
    ml[2 * tid + 1] = l;
  }
}

// One workgroup of 256 threads per (head, row); thread t owns element t of the
// head dimension.  The workgroup of head 0 also writes the ring slot and
// counts the token (no other reads the count: what is visible reached this
// kernel as the chunks' maxima and denominators).
__global__ void __launch_bounds__(256)
attn_decode_combine_kernel(AttnDecodeArgs p) {
#pragma clang fp contract(off)
  __shared__ float dots[4];
  __shared__ float weight[kAttnDecodeMaxChunks];
  __shared__ float inv_sum, p_self;
  const int tid = threadIdx.x;
  const int h = blockIdx.x, b = blockIdx.y;
  const uint16_t* qrow = p.q + (int64_t)b * p.ldq + h * kHd;
  const uint16_t* krow = p.k_new + (int64_t)b * p.ldk;
  const uint16_t* vrow = p.v_new + (int64_t)b * p.ldv;

  // ---- rotary embedding of element t of the new key and of this head's
  // query (recurrentgemma/torch/modules.py:52-83; rope_kernel's arithmetic)
  const int quarter = kHd / 4;
  float sn = 0.0f, cs = 1.0f;
  if (tid < kHd / 2) {
    const float angle =
        position_of_row(p.pos, p.pos_kind, b) * p.inv_freq[tid % quarter];
    sn = round_to_bf16(sinf(angle));
    cs = round_to_bf16(cosf(angle));
  }
  auto roped = [&](const uint16_t* row) -> float {
    if (tid >= kHd / 2) return bf16_bits_to_f32(row[tid]);
    const int i = tid % quarter;
    const float lo = bf16_bits_to_f32(row[i]);
    const float hi = bf16_bits_to_f32(row[i + quarter]);
    return round_to_bf16(tid < quarter
                             ? round_to_bf16(lo * cs) - round_to_bf16(hi * sn)
                             : round_to_bf16(hi * cs) + round_to_bf16(lo * sn));
  };
  const float k_mine = roped(krow);
  // ---- the chunks' results for this element, requested before anything
  // waits (a chunk without a visible slot left nothing: its weight is zero
  // and what is read there is dropped)
  const int64_t row_parts = (int64_t)b * p.chunks * p.heads;
  const float* po = p.part_o + (row_parts + h) * kHd + tid;
  const float v_mine = bf16_bits_to_f32(vrow[tid]);
  // ---- the new token's own score
  {
    float d = roped(qrow) * k_mine;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) d += __shfl_xor(d, off, 64);
    if ((tid & 63) == 0) dots[tid >> 6] = d;
  }
  __syncthreads();
  const float dot = (dots[0] + dots[1]) + (dots[2] + dots[3]);
  const float self = round_to_bf16(round_to_bf16(dot) * p.scale);
  const float* ml = p.part_ml + (row_parts + h) * 2;
  if (tid < 64) {
    // lane c: chunk c (c + 64 k for longer tables: chunks <= 64, so one each)
    const bool have = tid < p.chunks;
    const float mc = have ? ml[(int64_t)tid * p.heads * 2] : kNegInf;
    const float lc = have ? ml[(int64_t)tid * p.heads * 2 + 1] : 0.0f;
    float m = fmaxf(self, mc);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    const float w = lc > 0.0f ? expf(mc - m) : 0.0f;
    float sum = w * lc;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    const float e_self = expf(self - m);
    sum += e_self;
    weight[tid] = w;
    if (tid == 0) {
      const float inv = 1.0f / sum;
      inv_sum = inv;
      p_self = round_to_bf16(e_self * inv);
    }
  }
  __syncthreads();
  // ---- output
  float acc = 0.0f;
  for (int c0 = 0; c0 < p.chunks; c0 += 8) {
    float part[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      part[i] = c0 + i < p.chunks && weight[c0 + i] > 0.0f
                    ? po[(int64_t)(c0 + i) * p.heads * kHd]
                    : 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (c0 + i < p.chunks) acc += weight[c0 + i] * part[i];
  }
  const float from_ring = round_to_bf16(acc * inv_sum);
  p.out[((int64_t)b * p.heads + h) * kHd + tid] =
      f32_to_bf16_bits(from_ring + round_to_bf16(p_self * v_mine));
  if (!p.update || h != 0) return;
  const int nt = p.num_tokens[b];
  const int64_t slot = ((int64_t)b * p.window + nt % p.window) * kHd;
  p.ring_k[slot + tid] = f32_to_bf16_bits(k_mine);
  p.ring_v[slot + tid] = vrow[tid];
  __syncthreads();  // every thread has read num_tokens[b]
  if (tid == 0) p.num_tokens[b] = nt + 1;
}

}  // namespace

hipError_t launch_attn_decode_fused(const AttnDecodeArgs& a, hipStream_t s) {
  // needs bf16, head_dim 256, heads <= 16, chunks <= kAttnDecodeMaxChunks
  // (checked by the caller)
  if (a.B > 65535) return hipErrorInvalidValue;
  static OncePerDevice once;
  hipError_t e = set_max_dynamic_lds(
      once, (const void*)attn_decode_chunks_kernel, kChunkLdsBytes);
  if (e != hipSuccess) return e;
  attn_decode_chunks_kernel<<<dim3((unsigned)a.chunks, (unsigned)a.B), 256,
                              kChunkLdsBytes, s>>>(a);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  attn_decode_combine_kernel<<<dim3((unsigned)a.heads, (unsigned)a.B), 256, 0,
                               s>>>(a);
  return hipGetLastError();
}

}  // namespace rg
