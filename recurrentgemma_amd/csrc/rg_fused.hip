// Decode step of the recurrent core in one launch (bf16, 256-wide heads), and
// the re-layout of the gate weights that it and the prefill kernel
// (rg_prefill.hip) share.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;         // head width (K and per-gate N)
constexpr int kLdsStride = 264;  // bf16 elements per staged row (256 + 8 pad)

union Frag {
  bf16x8 v;
  uint16_t u[8];
  f32x4 q;
};

// ---------------------------------------------------------------- decode --
// Gate weights in the order the MFMA B operand is consumed: for head h, wave
// w (32 output channels), k-step ks, gate g and lane l the 8 bf16 values
// w_g[h][16 ks + 8 (l/32) + 0..7][32 w + l%32], 16 bytes per lane, so that a
// kernel fills its 128 weight registers with 32 coalesced 16-byte loads.
// One thread per 16-byte group; run once per set of weights.
__global__ void __launch_bounds__(256)
pack_gate_weights_kernel(const uint16_t* __restrict__ w_x,
                         const uint16_t* __restrict__ w_a,
                         uint16_t* __restrict__ packed, int H) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)H * 8 * 16 * 2 * 64;
  if (idx >= total) return;
  const int l = (int)(idx & 63);
  const int g = (int)((idx >> 6) & 1);
  const int ks = (int)((idx >> 7) & 15);
  const int w = (int)((idx >> 11) & 7);
  const int h = (int)(idx >> 14);
  const uint16_t* src = (g ? w_a : w_x) + (int64_t)h * kBW * kBW +
                        (int64_t)(16 * ks + 8 * (l >> 5)) * kBW + 32 * w + (l & 31);
  Frag f;
#pragma unroll
  for (int e = 0; e < 8; ++e) f.u[e] = src[(int64_t)e * kBW];
  *reinterpret_cast<f32x4*>(packed + idx * 8) = f.q;
}

// One token per sequence row: the same chain (conv step from the carried conv
// state, both gate projections, gate arithmetic, one recurrence step) with the
// 32 rows of a tile being different sequences.  One workgroup per (tile of 32
// rows, head).  Every state element is read and then written by the same
// thread, so the outputs may alias the inputs (in-place caches).
//
// Replaces Conv1D.forward's decode branch (layers.py:469-474, 491-529) and
// RGLRU.forward / rnn_scan with T == 1 (layers.py:313-365, 170-177).
constexpr int kStepRows = 32;
constexpr int kStepRowsPerThread = 8;  // 32 rows x 128 channel pairs / 512

__global__ void __launch_bounds__(512) block_step_bf16_kernel(StepArgs p) {
  __shared__ __align__(16) uint16_t stage[kStepRows * kLdsStride];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b0 = blockIdx.x * kStepRows;
  const int h = blockIdx.y;
  const int B = p.B;
  const int64_t W = p.W;
  const bool upper = lane >= 32;
  const int n0 = wave * 32;
  const int ch = h * kBW + n0 + (lane & 31);

  // ---- loads first: this wave's weights (32 x 16 bytes per lane), the state
  //      of this lane's 16 (row, channel) elements ---------------------------
  Frag bfrag[16][2];
  {
    const f32x4* src = reinterpret_cast<const f32x4*>(p.w_packed) +
                       ((int64_t)(h * 8 + wave) * 16 * 2) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks)
#pragma unroll
      for (int g = 0; g < 2; ++g) bfrag[ks][g].q = src[(ks * 2 + g) * 64];
  }
  float hv[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int64_t b = b0 + 8 * (r >> 2) + (r & 3) + (upper ? 4 : 0);
    hv[r] = b < B ? p.h_in[b * W + ch] : 0.0f;
  }

  // ---- conv step of this tile's rows -> LDS (bf16), new conv state ---------
  {
    const int cp = tid & 127;
    const int rg = tid >> 7;
    const uint32_t c = h * kBW + cp * 2;
    const uint16_t* xin = (const uint16_t*)p.x;
    const uint16_t* cin = (const uint16_t*)p.cache_in;
    uint16_t* cout = (uint16_t*)p.cache_out;
    uint32_t xr[kStepRowsPerThread], s0[kStepRowsPerThread],
        s1[kStepRowsPerThread], s2[kStepRowsPerThread];  // state oldest first
#pragma unroll
    for (int j = 0; j < kStepRowsPerThread; ++j) {
      const int64_t b = b0 + rg * kStepRowsPerThread + j;
      xr[j] = s0[j] = s1[j] = s2[j] = 0u;
      if (b < B) {
        xr[j] = *reinterpret_cast<const uint32_t*>(xin + b * W + c);
        s0[j] = *reinterpret_cast<const uint32_t*>(cin + (b * 3 + 0) * W + c);
        s1[j] = *reinterpret_cast<const uint32_t*>(cin + (b * 3 + 1) * W + c);
        s2[j] = *reinterpret_cast<const uint32_t*>(cin + (b * 3 + 2) * W + c);
      }
    }
    const uint16_t* cw = (const uint16_t*)p.conv_w + c;
    const uint32_t u0 = *reinterpret_cast<const uint32_t*>(cw);
    const uint32_t u1 = *reinterpret_cast<const uint32_t*>(cw + W);
    const uint32_t u2 = *reinterpret_cast<const uint32_t*>(cw + 2 * W);
    const uint32_t u3 = *reinterpret_cast<const uint32_t*>(cw + 3 * W);
    const uint32_t ub =
        *reinterpret_cast<const uint32_t*>((const uint16_t*)p.conv_b + c);
#pragma unroll
    for (int j = 0; j < kStepRowsPerThread; ++j) {
      const int row = rg * kStepRowsPerThread + j;
      const int64_t b = b0 + row;
      float o[2];
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        auto unpack = [&](uint32_t v) {
          return k == 0 ? __uint_as_float(v << 16)
                        : __uint_as_float(v & 0xffff0000u);
        };
        o[k] = conv4(unpack(xr[j]), unpack(s2[j]), unpack(s1[j]), unpack(s0[j]),
                     unpack(u0), unpack(u1), unpack(u2), unpack(u3), unpack(ub));
      }
      *reinterpret_cast<uint32_t*>(stage + (size_t)row * kLdsStride + cp * 2) =
          pack_bf16x2(o[0], o[1]);
      if (b < B) {
        *reinterpret_cast<uint32_t*>(cout + (b * 3 + 0) * W + c) = s1[j];
        *reinterpret_cast<uint32_t*>(cout + (b * 3 + 1) * W + c) = s2[j];
        *reinterpret_cast<uint32_t*>(cout + (b * 3 + 2) * W + c) = xr[j];
      }
    }
  }

  const float bias_x = bf16_bits_to_f32(((const uint16_t*)p.b[0])[ch]);
  const float bias_a = bf16_bits_to_f32(((const uint16_t*)p.b[1])[ch]);
  const float decay =
      (-8.0f * kLog2e) *
      softplus_precise(bf16_bits_to_f32(((const uint16_t*)p.a_param)[ch]));
  // rows of this tile whose position is 0 (document start: forget the state)
  uint32_t m_start;
  {
    const int64_t b = (int64_t)b0 + (lane & 31);
    bool st = false;
    if (b < B) st = is_doc_start(p.segpos, p.seg_kind, b);
    m_start = (uint32_t)__ballot(st);
  }
  __syncthreads();  // the staged tile is complete

  f32x16 acc_x, acc_a;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    acc_x[r] = bias_x;
    acc_a[r] = bias_a;
  }
  const uint16_t* abase =
      stage + (size_t)(lane & 31) * kLdsStride + 8 * (lane >> 5);
#pragma unroll
  for (int ks = 0; ks < 16; ++ks) {
    Frag a;
    a.q = *reinterpret_cast<const f32x4*>(abase + ks * 16);
    acc_x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, bfrag[ks][0].v, acc_x,
                                                    0, 0, 0);
    acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, bfrag[ks][1].v, acc_a,
                                                    0, 0, 0);
  }
  const uint16_t* xcp =
      stage + (size_t)(4 * (lane >> 5)) * kLdsStride + n0 + (lane & 31);
  float* h_out = p.h_out;
  uint16_t* yout = (uint16_t*)p.y;
#pragma unroll
  for (int r = 0; r < 16; r += 2) {
    // pre-activations are a bf16 module output in the reference
    const uint32_t px2 = pack_bf16x2(acc_x[r], acc_x[r + 1]);
    const uint32_t pa2 = pack_bf16x2(acc_a[r], acc_a[r + 1]);
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int rr = r + e;
      const int i = 8 * (rr >> 2) + (rr & 3);
      const int row = i + (upper ? 4 : 0);
      const int64_t b = (int64_t)b0 + row;
      const float xc = bf16_bits_to_f32(xcp[(size_t)i * kLdsStride]);
      const float px = e == 0 ? __uint_as_float(px2 << 16)
                              : __uint_as_float(px2 & 0xffff0000u);
      const float pa = e == 0 ? __uint_as_float(pa2 << 16)
                              : __uint_as_float(pa2 & 0xffff0000u);
      const float gate_x = sigmoid_fast(px);
      const float gate_a = sigmoid_fast(pa);
      float a = __builtin_amdgcn_exp2f(gate_a * decay);
      if ((m_start >> row) & 1u) a = 0.0f;  // the input scale becomes 1 below
      const float mult = __builtin_amdgcn_sqrtf(__builtin_fmaf(-a, a, 1.0f));
      const float xn = (xc * gate_x) * mult;
      const float hn = __builtin_fmaf(a, hv[rr], xn);
      if (b < B) {
        h_out[b * W + ch] = hn;
        yout[b * W + ch] = f32_to_bf16_bits(hn);
      }
    }
  }
}

}  // namespace

hipError_t launch_pack_gate_weights(const void* w_x, const void* w_a,
                                    void* packed, int H, hipStream_t s) {
  const int64_t total = (int64_t)H * 8 * 16 * 2 * 64;
  pack_gate_weights_kernel<<<dim3((unsigned)((total + 255) / 256)), 256, 0, s>>>(
      (const uint16_t*)w_x, (const uint16_t*)w_a, (uint16_t*)packed, H);
  return hipGetLastError();
}

hipError_t launch_block_step_bf16(const StepArgs& a, hipStream_t s) {
  // needs head width 256 (checked by the caller)
  const int tiles = (a.B + kStepRows - 1) / kStepRows;
  if (tiles <= 0 || a.H > 65535) return hipErrorInvalidValue;
  block_step_bf16_kernel<<<dim3((unsigned)tiles, (unsigned)a.H), 512, 0, s>>>(a);
  return hipGetLastError();
}

}  // namespace rg
