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
// ROWS = 32 rows of a tile, or 16 where 32 would leave CUs without a
// workgroup (the matrix instructions then run half empty, which costs
// nothing here: a step is loads and stores).

// GELU: y leaves as y * gelu(gate_branch), the join of the recurrent block's
// two branches (recurrentgemma/torch/modules.py:627-628, 644) with the
// arithmetic and roundings of the stand-alone gelu_mul pass.
template <bool GELU, int ROWS>
__global__ void __launch_bounds__(512) block_step_bf16_kernel(StepArgs p) {
  constexpr int kStepRows = ROWS;
  constexpr int kStepRowsPerThread = ROWS / 8;  // rows x 64 channel quads / 512
  constexpr int kRuns = ROWS / 2;  // of a lane's 16 accumulator rows: in use
  // (32 rows staged whatever ROWS is: the matrix instructions read 32)
  __shared__ __align__(16) uint16_t stage[32 * kLdsStride];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroups go to the eight XCDs in turn (linear id modulo 8), each with
  // an L2 of its own: the (head, row tile) pairs are dealt out so that one
  // XCD gets a contiguous run of pairs in head-major order, i.e. all row
  // tiles of a head fetch its weights through the same L2 (the plain order
  // sends the tiles of a head to eight different ones, and every L2 then
  // pulls in every head's weights).
  const int tiles = (p.B + kStepRows - 1) / kStepRows;
  int pair = blockIdx.x;
  {
    const int per_xcd = (int)gridDim.x / 8;
    if (pair < 8 * per_xcd) pair = (pair & 7) * per_xcd + (pair >> 3);
  }
  const int h = pair / tiles;
  const int b0 = (pair - h * tiles) * kStepRows;
  const int B = p.B;
  const int64_t W = p.W;
  const bool upper = lane >= 32;
  const int n0 = wave * 32;
  const int ch = h * kBW + n0 + (lane & 31);

  // Everything per row goes through descriptors over this tile's rows only:
  // rows past the end of the batch read as zero and their stores are dropped,
  // without a branch around any access.
  const int rows_here = B - b0 < kStepRows ? B - b0 : kStepRows;
  const uint32_t row_bytes = (uint32_t)W * 2u;
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(
      (const uint16_t*)p.x + (int64_t)b0 * W, (uint32_t)rows_here * row_bytes);
  const __amdgpu_buffer_rsrc_t rcin =
      make_rsrc((const uint16_t*)p.cache_in + (int64_t)b0 * 3 * W,
                (uint32_t)rows_here * 3u * row_bytes);
  const __amdgpu_buffer_rsrc_t rcout =
      make_rsrc((uint16_t*)p.cache_out + (int64_t)b0 * 3 * W,
                (uint32_t)rows_here * 3u * row_bytes);
  const __amdgpu_buffer_rsrc_t rhin = make_rsrc(
      p.h_in + (int64_t)b0 * W, (uint32_t)rows_here * 2u * row_bytes);
  const __amdgpu_buffer_rsrc_t rhout = make_rsrc(
      p.h_out + (int64_t)b0 * W, (uint32_t)rows_here * 2u * row_bytes);
  const __amdgpu_buffer_rsrc_t ry = make_rsrc(
      (uint16_t*)p.y + (int64_t)b0 * W, (uint32_t)rows_here * row_bytes);
  const __amdgpu_buffer_rsrc_t rgate =
      make_rsrc((const uint16_t*)p.gate_branch + (int64_t)b0 * W,
                GELU ? (uint32_t)rows_here * row_bytes : 0u);
  // ---- loads, in the order they are needed: the conv step's rows (thread =
  //      four channels of four rows: 8-byte accesses, a wave per access covers
  //      the head's 512 bytes of a row), the small per-channel and per-row
  //      values, this lane's 16 state elements, this wave's weights (32 x 16
  //      bytes per lane).  Loads return in order, so the conv step runs while
  //      the weights are still on their way.
  const int cq = lane;
  const int rg = wave;
  const uint32_t c = h * kBW + cq * 4;
  u32x2 xr[kStepRowsPerThread], s0[kStepRowsPerThread], s1[kStepRowsPerThread],
      s2[kStepRowsPerThread];  // state oldest first
#pragma unroll
  for (int j = 0; j < kStepRowsPerThread; ++j) {
    const uint32_t row = rg * kStepRowsPerThread + j;
    xr[j] = __builtin_amdgcn_raw_buffer_load_b64(rx, 2u * c, row * row_bytes, 0);
    s0[j] = __builtin_amdgcn_raw_buffer_load_b64(
        rcin, 2u * c, (row * 3u + 0u) * row_bytes, 0);
    s1[j] = __builtin_amdgcn_raw_buffer_load_b64(
        rcin, 2u * c, (row * 3u + 1u) * row_bytes, 0);
    s2[j] = __builtin_amdgcn_raw_buffer_load_b64(
        rcin, 2u * c, (row * 3u + 2u) * row_bytes, 0);
  }
  const uint16_t* cw = (const uint16_t*)p.conv_w + c;
  const u32x2 u0 = *reinterpret_cast<const u32x2*>(cw);
  const u32x2 u1 = *reinterpret_cast<const u32x2*>(cw + W);
  const u32x2 u2 = *reinterpret_cast<const u32x2*>(cw + 2 * W);
  const u32x2 u3 = *reinterpret_cast<const u32x2*>(cw + 3 * W);
  const u32x2 ub =
      *reinterpret_cast<const u32x2*>((const uint16_t*)p.conv_b + c);
  __builtin_amdgcn_sched_barrier(0);
  // (the small per-channel and per-row values are requested here, with
  // everything else: asked for where they are used they would cost a memory
  // round trip of their own after the conv step)
  const uint16_t bias_x_raw = ((const uint16_t*)p.b[0])[ch];
  const uint16_t bias_a_raw = ((const uint16_t*)p.b[1])[ch];
  const uint16_t a_param_raw = ((const uint16_t*)p.a_param)[ch];
  // position of row lane % 32: two unconditional 32-bit loads (for int32
  // positions the high half is sent out of range and reads as zero)
  uint32_t seg_lo, seg_hi;
  {
    const bool is64 = p.seg_kind == kSegI64;
    const uint32_t esize = is64 ? 8u : 4u;
    const __amdgpu_buffer_rsrc_t rseg =
        make_rsrc((const char*)p.segpos + (int64_t)b0 * esize,
                  (uint32_t)rows_here * esize);
    const uint32_t off = (uint32_t)(lane & 31) * esize;
    seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
    seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
        rseg, is64 ? off + 4u : kBufferOutOfRange, 0, 0);
  }
  float hv[kRuns];
#pragma unroll
  for (int r = 0; r < kRuns; ++r) {
    // row 8 (r / 4) + r % 4 (+ 4 in the upper half-wave)
    hv[r] = __builtin_bit_cast(
        float,
        __builtin_amdgcn_raw_buffer_load_b32(
            rhin, (uint32_t)ch * 4u + (upper ? 8u * row_bytes : 0u),
            (uint32_t)(8 * (r >> 2) + (r & 3)) * 2u * row_bytes, 0));
  }

  // GELU: the gate branch where this lane stores y (see the output stage)
  uint32_t gate2[kRuns / 2];
  if (GELU) {
    const uint32_t lane_rows = ((lane & 1) ? 1u : 0u) + (upper ? 4u : 0u);
#pragma unroll
    for (int r = 0; r < kRuns; r += 2)
      gate2[r >> 1] = __builtin_amdgcn_raw_buffer_load_b32(
          rgate, (uint32_t)(ch & ~1) * 2u + lane_rows * row_bytes,
          (uint32_t)(8 * (r >> 2) + (r & 3)) * row_bytes, 0);
  }

  Frag bfrag[16][2];
  {
    const f32x4* src = reinterpret_cast<const f32x4*>(p.w_packed) +
                       ((int64_t)(h * 8 + wave) * 16 * 2) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks)
#pragma unroll
      for (int g = 0; g < 2; ++g) bfrag[ks][g].q = src[(ks * 2 + g) * 64];
  }
  // (nothing above may sink below this line: left alone the compiler moves
  // most of the weight and state loads behind the conv step, whose own loads
  // it waits for first, and the kernel pays two memory round trips in a row)
  __builtin_amdgcn_sched_barrier(0);

  // ---- conv step of this tile's rows -> LDS (bf16), new conv state ---------
  {
#pragma unroll
    for (int j = 0; j < kStepRowsPerThread; ++j) {
      const uint32_t row = rg * kStepRowsPerThread + j;
      u32x2 packed;
#pragma unroll
      for (int w2 = 0; w2 < 2; ++w2) {
        // the bf16 kernels' width-4 arithmetic (conv4_dot of rg_common.h):
        // s0, s1, s2 are the state rows x[t-3], x[t-2], x[t-1], xr is x[t]
        uint32_t p_old[2], p_new[2], w10[2], w32[2];
        pair_up(s0[j][w2], s1[j][w2], p_old[0], p_old[1]);
        pair_up(s2[j][w2], xr[j][w2], p_new[0], p_new[1]);
        pair_up(u0[w2], u1[w2], w10[0], w10[1]);
        pair_up(u2[w2], u3[w2], w32[0], w32[1]);
        const float bias2[2] = {__uint_as_float(ub[w2] << 16),
                                __uint_as_float(ub[w2] & 0xffff0000u)};
        float o[2];
        conv4_dot_x2(p_old, p_new, w10, w32, bias2, o);
        packed[w2] = pack_bf16x2(o[0], o[1]);
      }
      *reinterpret_cast<u32x2*>(stage + (size_t)row * kLdsStride + cq * 4) =
          packed;
      __builtin_amdgcn_raw_buffer_store_b64(s1[j], rcout, 2u * c,
                                            (row * 3u + 0u) * row_bytes, 0);
      __builtin_amdgcn_raw_buffer_store_b64(s2[j], rcout, 2u * c,
                                            (row * 3u + 1u) * row_bytes, 0);
      __builtin_amdgcn_raw_buffer_store_b64(xr[j], rcout, 2u * c,
                                            (row * 3u + 2u) * row_bytes, 0);
    }
  }

  const float bias_x = bf16_bits_to_f32(bias_x_raw);
  const float bias_a = bf16_bits_to_f32(bias_a_raw);
  const float decay =
      (-8.0f * kLog2e) * softplus_precise(bf16_bits_to_f32(a_param_raw));
  // rows of this tile whose position is 0 (document start: forget the state)
  const uint32_t m_start = (uint32_t)__ballot((seg_lo | seg_hi) == 0u);
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
  // Outputs: neighbouring lanes hold neighbouring channels of the same rows.
  // Lanes swap in pairs so that the even lane stores both channels of the even
  // row of a row pair and the odd lane both channels of the odd row: 8-byte
  // state and 4-byte y stores, half as many as one store per element.
  const bool odd = lane & 1;
  const uint32_t pair_ch = (uint32_t)(ch & ~1);
#pragma unroll
  for (int r = 0; r < kRuns; r += 2) {
    // pre-activations are a bf16 module output in the reference
    const uint32_t px2 = pack_bf16x2(acc_x[r], acc_x[r + 1]);
    const uint32_t pa2 = pack_bf16x2(acc_a[r], acc_a[r + 1]);
    float hn[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int rr = r + e;
      const int i = 8 * (rr >> 2) + (rr & 3);
      const int row = i + (upper ? 4 : 0);
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
      hn[e] = __builtin_fmaf(a, hv[rr], xn);
    }
    // what the partner lane stores of mine: the even lane keeps row r, the
    // odd lane row r + 1
    const float give = odd ? hn[0] : hn[1];
    const float got = __uint_as_float(__builtin_amdgcn_mov_dpp(
        __float_as_uint(give), 0xB1 /* quad_perm [1,0,3,2] */, 0xf, 0xf, true));
    const float mine = odd ? hn[1] : hn[0];
    const float lo = odd ? got : mine;  // channel pair_ch
    const float hi = odd ? mine : got;  // channel pair_ch + 1
    // row 8 (r / 4) + r % 4, + 1 in the odd lane, + 4 in the upper half-wave
    const uint32_t lane_rows = (odd ? 1u : 0u) + (upper ? 4u : 0u);
    const uint32_t tile_row = (uint32_t)(8 * (r >> 2) + (r & 3));
    __builtin_amdgcn_raw_buffer_store_b64(
        u32x2{__float_as_uint(lo), __float_as_uint(hi)}, rhout,
        pair_ch * 4u + lane_rows * 2u * row_bytes, tile_row * 2u * row_bytes, 0);
    uint32_t y2 = pack_bf16x2(lo, hi);
    if (GELU) {
      const uint32_t g2 = gate2[r >> 1];
      y2 = pack_bf16x2(gelu_mul_bf16(__uint_as_float(y2 << 16),
                                     __uint_as_float(g2 << 16)),
                       gelu_mul_bf16(__uint_as_float(y2 & 0xffff0000u),
                                     __uint_as_float(g2 & 0xffff0000u)));
    }
    __builtin_amdgcn_raw_buffer_store_b32(y2, ry,
                                          pair_ch * 2u + lane_rows * row_bytes,
                                          tile_row * row_bytes, 0);
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
  const int tiles32 = (a.B + 31) / 32;
  if (tiles32 <= 0 || (int64_t)tiles32 * 2 * a.H > 0x7fffffff)
    return hipErrorInvalidValue;
  // tiles of 16 rows while 32 would give fewer workgroups than CUs (256 rows
  // x 16 heads: 128 workgroups 10.2 us, 256 workgroups 9.0 us, 512 of 8 rows
  // 13.6 us a step)
  const bool half = (int64_t)tiles32 * a.H < 256 && a.B > 16;
  const int tiles = half ? (a.B + 15) / 16 : tiles32;
  const dim3 grid((unsigned)(tiles * a.H));
  if (a.gate_branch) {
    if (half) block_step_bf16_kernel<true, 16><<<grid, 512, 0, s>>>(a);
    else block_step_bf16_kernel<true, 32><<<grid, 512, 0, s>>>(a);
  } else {
    if (half) block_step_bf16_kernel<false, 16><<<grid, 512, 0, s>>>(a);
    else block_step_bf16_kernel<false, 32><<<grid, 512, 0, s>>>(a);
  }
  return hipGetLastError();
}

}  // namespace rg
