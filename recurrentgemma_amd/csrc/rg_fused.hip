// Whole recurrent core in one launch (bf16, 256-wide heads): width-4 conv ->
// both gate projections on MFMA -> gate activations -> linear recurrence.
//
// One persistent workgroup per (sequence row b, head h) walks the sequence in
// tiles of 64 tokens.  Neither the conv output nor the gate pre-activations
// ever go to memory: per element the kernel reads x once and writes y once.
//
// Replaces the chain Conv1D.forward -> RGLRU.forward of
// recurrentgemma/torch/modules.py:632-643 (layers.py:447-529, 313-365,
// 140-191) for prefill.
#include <type_traits>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;           // head width (K and per-gate N)
constexpr int kTM = 64;            // tokens per tile
constexpr int kLdsStride = 264;    // bf16 elements per staged row (256 + 8 pad)
constexpr int kRowsPerGroup = 16;  // rows each thread converts per tile
constexpr int kHalo = 3;
constexpr int kRaw = kRowsPerGroup + kHalo;
// Three staged tiles: the one the MFMAs read, the one being written for the
// next tile, and the previous one, which half of the waves still read while
// they finish its gate arithmetic (see the tile loop).
constexpr int kStageBufs = 3;
constexpr size_t kStageLdsBytes =
    (size_t)kStageBufs * kTM * kLdsStride * sizeof(uint16_t);
// Per-wave output patch: 32 tokens x 32 channels in bf16, rows padded to 80
// bytes (16-byte aligned row reads, spread over the banks).
constexpr int kPatchStride = 80;
constexpr size_t kPatchBytesPerWave = 32ull * kPatchStride;
// Conv taps and bias of the 128 channel pairs as floats, 12 per pair (w0..w3
// and bias for both channels, padded): read back at the start of every conv
// so that they do not occupy registers in between.
constexpr size_t kConvTabOffset = kStageLdsBytes + 8 * kPatchBytesPerWave;
// Gate biases and decay constant of the 256 channels (4 floats each, one
// padding), read at the start of the phases that need them.
constexpr size_t kChanTabOffset = kConvTabOffset + 128 * 12 * sizeof(float);
constexpr size_t kFusedLdsBytes = kChanTabOffset + 256 * 4 * sizeof(float);

union Frag {
  bf16x8 v;
  uint16_t u[8];
  f32x4 q;
};

// Build switch for the tile loop: 1 runs waves 4-7 one phase behind waves 0-3
// (matrix phases of one group over vector phases of the other).  Measured at
// B16 T8192 W4096 it is about 3 % slower than keeping all waves in the same
// phase (the vector ALU, not the matrix pipe, bounds the tile), so it is off.
#ifndef RG_FUSED_SKEW
#define RG_FUSED_SKEW 0
#endif
constexpr bool kSkewGroups = RG_FUSED_SKEW != 0;

using WithCuts = std::integral_constant<bool, true>;
using NoCuts = std::integral_constant<bool, false>;

// Broadcast of the two 32-lane halves of a register: lo = the value lanes
// 0-31 hold (in all 64 lanes), hi = the value lanes 32-63 hold.
__device__ __forceinline__ void halves(float v, float& lo, float& hi) {
  const uint32_t u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  lo = __uint_as_float(r[0]);
  hi = __uint_as_float(r[1]);
}

__global__ void __launch_bounds__(512) block_fused_bf16_kernel(FusedArgs p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(lds_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x / p.H;
  const int h = blockIdx.x % p.H;
  const int T_len = p.T;
  const int64_t W = p.W;
  const int ntiles = (T_len + kTM - 1) / kTM;
  const bool upper = lane >= 32;
  // Lane-derived addresses are recomputed from the thread id where they are
  // used (a few integer instructions) instead of being kept in registers for
  // the whole tile: the optimiser cannot see through fresh_tid().
  auto fresh_tid = [&]() {
    int t = tid;
    asm volatile("" : "+v"(t));
    return t;
  };

  // ---- this wave's weights: 32 channels of the head, both gates ----------
  // The weights are [k][n] with n contiguous, the MFMA B operand wants 8
  // consecutive k per lane: either the caller supplies them re-laid-out, or
  // they are transposed through LDS here, 128 k-rows of one gate at a time
  // (coalesced 16-byte global reads, 2-byte LDS reads).
  const int n0 = wave * 32;
  Frag bfrag[16][2];
  if (p.w_packed) {
    // already in operand order (pack_gate_weights_kernel): 32 x 16 bytes
    const f32x4* src = reinterpret_cast<const f32x4*>(p.w_packed) +
                       ((int64_t)(h * 8 + wave) * 16 * 2) * 64 + lane;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks)
#pragma unroll
      for (int g = 0; g < 2; ++g) bfrag[ks][g].q = src[(ks * 2 + g) * 64];
  } else {
#pragma unroll
    for (int g = 0; g < 2; ++g) {
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) {
        const uint16_t* src =
            (const uint16_t*)p.w[g] + ((int64_t)h * kBW + kh * 128) * kBW;
        for (int e = tid; e < 128 * 32; e += 512) {
          const int r = e >> 5, q = e & 31;
          *reinterpret_cast<f32x4*>(lds + (size_t)r * kLdsStride + q * 8) =
              *reinterpret_cast<const f32x4*>(src + (size_t)r * kBW + q * 8);
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          const int n = n0 + (lane & 31);
          const int kb = ks * 16 + 8 * (lane >> 5);
#pragma unroll
          for (int e = 0; e < 8; ++e)
            bfrag[kh * 8 + ks][g].u[e] = lds[(size_t)(kb + e) * kLdsStride + n];
        }
        __syncthreads();
      }
    }
  }
  // Per-lane channel (the MFMA result has channel = lane % 32): gate biases,
  // decay constant -8 softplus(a_param) log2(e), running state.
  const int ch = h * kBW + n0 + (lane & 31);
  auto chan_ptr = [&](int t) {
    return reinterpret_cast<float*>(lds_raw + kChanTabOffset) +
           4 * (n0 + (t & 31));
  };
  if (!upper) {
    float* const chan_tab = chan_ptr(tid);
    f32x4 t = {bf16_bits_to_f32(((const uint16_t*)p.b[0])[ch]),
               bf16_bits_to_f32(((const uint16_t*)p.b[1])[ch]),
               (-8.0f * kLog2e) * softplus_precise(bf16_bits_to_f32(
                                      ((const uint16_t*)p.a_param)[ch])),
               0.0f};
    *reinterpret_cast<f32x4*>(chan_tab) = t;
  }
  float hc = p.h0 ? p.h0[(int64_t)b * W + ch] : 0.0f;

  // ---- addressing ---------------------------------------------------------
  const uint32_t row_bytes = 2u * (uint32_t)p.W;
  const uint32_t seq_bytes = (uint32_t)T_len * row_bytes;  // < 2^31 (launcher)
  const __amdgpu_buffer_rsrc_t rx =
      make_rsrc((const char*)p.x + (int64_t)b * seq_bytes, seq_bytes);
  const __amdgpu_buffer_rsrc_t ry =
      make_rsrc((char*)p.y + (int64_t)b * seq_bytes, seq_bytes);
  const bool seg_is64 = p.seg_kind == kSegI64;
  const uint32_t seg_esize = seg_is64 ? 8u : 4u;
  const __amdgpu_buffer_rsrc_t rseg =
      make_rsrc((const char*)p.segpos + (int64_t)b * T_len * seg_esize,
                (uint32_t)T_len * seg_esize);

  // x staging: thread -> (channel pair, group of 16 tokens)
  const int cp = tid & 127;
  const int rg = __builtin_amdgcn_readfirstlane(tid >> 7);
  const uint32_t c = h * kBW + cp * 2;
  const uint32_t c_bytes = 2u * c;
  float cw0[2], cw1[2], cw2[2], cw3[2], cb[2];
  auto conv_ptr = [&](int t) {
    return reinterpret_cast<float*>(lds_raw + kConvTabOffset) + (t & 127) * 12;
  };
  if (tid < 128) {
    float* const conv_tab = conv_ptr(tid);
    const uint16_t* cw = (const uint16_t*)p.conv_w + c;
    const uint32_t u0 = *reinterpret_cast<const uint32_t*>(cw);
    const uint32_t u1 = *reinterpret_cast<const uint32_t*>(cw + W);
    const uint32_t u2 = *reinterpret_cast<const uint32_t*>(cw + 2 * W);
    const uint32_t u3 = *reinterpret_cast<const uint32_t*>(cw + 3 * W);
    const uint32_t ub =
        *reinterpret_cast<const uint32_t*>((const uint16_t*)p.conv_b + c);
    f32x4 t0 = {__uint_as_float(u0 << 16), __uint_as_float(u0 & 0xffff0000u),
                __uint_as_float(u1 << 16), __uint_as_float(u1 & 0xffff0000u)};
    f32x4 t1 = {__uint_as_float(u2 << 16), __uint_as_float(u2 & 0xffff0000u),
                __uint_as_float(u3 << 16), __uint_as_float(u3 & 0xffff0000u)};
    f32x4 t2 = {__uint_as_float(ub << 16), __uint_as_float(ub & 0xffff0000u),
                0.0f, 0.0f};
    reinterpret_cast<f32x4*>(conv_tab)[0] = t0;
    reinterpret_cast<f32x4*>(conv_tab)[1] = t1;
    reinterpret_cast<f32x4*>(conv_tab)[2] = t2;
  }
  __syncthreads();
  auto load_conv_consts = [&](int t) {
    const float* const conv_tab = conv_ptr(t);
    const f32x4 t0 = reinterpret_cast<const f32x4*>(conv_tab)[0];
    const f32x4 t1 = reinterpret_cast<const f32x4*>(conv_tab)[1];
    const f32x4 t2 = reinterpret_cast<const f32x4*>(conv_tab)[2];
    cw0[0] = t0[0]; cw0[1] = t0[1]; cw1[0] = t0[2]; cw1[1] = t0[3];
    cw2[0] = t1[0]; cw2[1] = t1[1]; cw3[0] = t1[2]; cw3[1] = t1[3];
    cb[0] = t2[0];  cb[1] = t2[1];
  };
  uint32_t raw[kRaw];
  uint32_t seg_lo = 1, seg_hi = 0;

  // Document starts of a tile: lane j looks at token 64*tile + j.  Two
  // unconditional 32-bit loads (for int32 positions the high half is sent out
  // of range and reads as zero); tokens past the end read as zero too and are
  // masked in start_mask().
  auto fetch_seg = [&](int tile) {
    const int t = tile * kTM + lane;
    const uint32_t off =
        (tile < ntiles && t < T_len) ? (uint32_t)t * seg_esize : kBufferOutOfRange;
    seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
    seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
        rseg, seg_is64 ? off + 4u : kBufferOutOfRange, 0, 0);
  };
  auto start_mask = [&](int tile) -> uint64_t {
    uint32_t lo = seg_lo, hi = seg_hi;
    asm volatile("" : "+v"(lo), "+v"(hi));  // test here, a tile after the load
    const int t = tile * kTM + lane;
    return __ballot(tile < ntiles && t < T_len && (lo | hi) == 0u);
  };
  // Rows before the sequence get an out-of-range scalar offset, rows past its
  // end fall outside the descriptor: both read as zero, which is what the
  // conv sees there.
  auto fetch_row = [&](int tile, int j, uint32_t cb_off) {
    const int t = tile * kTM + rg * kRowsPerGroup - kHalo + j;  // uniform
    const uint32_t soff =
        (t < 0 || tile >= ntiles) ? kBufferOutOfRange : (uint32_t)t * row_bytes;
    raw[j] = __builtin_amdgcn_raw_buffer_load_b32(rx, cb_off, soff, 0);
  };
  auto chan_bytes = [&](int t) {  // byte offset of thread t's channel pair
    return 2u * (uint32_t)(h * kBW + (t & 127) * 2);
  };


  // Conv of one tile, one row at a time.  cut bit j: token j of this thread
  // group's 19 rows starts a document; the conv must not look past it.
  uint32_t cut = 0;
  float h0v[2], h1v[2], h2v[2];
  auto stage_dst = [&](int t, int buf) {
    return lds + (size_t)buf * kTM * kLdsStride +
           (size_t)(rg * kRowsPerGroup) * kLdsStride + (t & 127) * 2;
  };
  auto stage_begin = [&](int t, uint64_t m_tile, uint64_t m_before) {
    // rows 16*rg-3 .. 16*rg+15 of the tile; the three rows before the tile
    // are the last three of the previous one
    if (rg == 0)
      cut = ((uint32_t)(m_tile << 3) | (uint32_t)(m_before >> 61)) & 0x7ffffu;
    else
      cut = (uint32_t)(m_tile >> (16 * rg - 3)) & 0x7ffffu;
    h0v[0] = h0v[1] = h1v[0] = h1v[1] = h2v[0] = h2v[1] = 0.0f;
    load_conv_consts(t);
  };
  auto stage_row = [&](int j, uint16_t* dst, auto cuts) {
    constexpr bool CUTS = decltype(cuts)::value;
    float xv[2];
    xv[0] = __uint_as_float(raw[j] << 16);
    xv[1] = __uint_as_float(raw[j] & 0xffff0000u);
    if (CUTS && ((cut >> j) & 1u)) {
      h0v[0] = h0v[1] = h1v[0] = h1v[1] = h2v[0] = h2v[1] = 0.0f;
    }
    if (j >= kHalo) {
      const float o0 = conv4(xv[0], h0v[0], h1v[0], h2v[0], cw0[0], cw1[0],
                             cw2[0], cw3[0], cb[0]);
      const float o1 = conv4(xv[1], h0v[1], h1v[1], h2v[1], cw0[1], cw1[1],
                             cw2[1], cw3[1], cb[1]);
      *reinterpret_cast<uint32_t*>(dst + (size_t)(j - kHalo) * kLdsStride) =
          pack_bf16x2(o0, o1);
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      h2v[k] = h1v[k];
      h1v[k] = h0v[k];
      h0v[k] = xv[k];
    }
  };

  // ---- per-wave output patch ----------------------------------------------
  unsigned char* const patch =
      lds_raw + kStageLdsBytes + (size_t)wave * kPatchBytesPerWave;
  // (written as token 4*(lane/32) + i, channel lane%32; read back as 16-byte
  // row chunks)

  // ---- prologue -------------------------------------------------------------
  uint64_t m_cur = 0;
  {
    fetch_seg(0);
#pragma unroll
    for (int j = 0; j < kRaw; ++j) fetch_row(0, j, c_bytes);
    m_cur = start_mask(0);
    stage_begin(tid, m_cur, 0);
#pragma unroll
    for (int j = 0; j < kRaw; ++j) stage_row(j, stage_dst(tid, 0), WithCuts{});
    fetch_seg(1);
#pragma unroll
    for (int j = 0; j < kRaw; ++j) fetch_row(1, j, c_bytes);
  }
  lds_barrier();

  // Gate arithmetic + recurrence of one 32-token half of a tile.  On entry
  // acc_x / acc_a hold the gate pre-activations (bias included) of tokens
  // i = 8*(r/4) + 4*(lane/32) + r%4 for channel lane%32.  `general` also
  // handles document starts (a = 0, unit input scale) and tokens past the end
  // of the sequence (identity: a = 1, no input).
  auto half_epilogue = [&](int it, int mt, int buf, f32x16& acc_x, f32x16& acc_a,
                           uint64_t m_tile) {
    const bool general = m_tile != 0 || (it + 1) * kTM > T_len;
    int l1 = lane;
    asm volatile("" : "+v"(l1));  // address recomputed per call, not kept
    const uint16_t* xcp = lds + (size_t)buf * kTM * kLdsStride +
                          (size_t)(mt * 32 + 4 * (l1 >> 5)) * kLdsStride + n0 +
                          (l1 & 31);
    const int t_half = it * kTM + mt * 32;  // first token of this half
    const float decay = chan_ptr(l1)[2];
    // `general` (wave-uniform, rare): bit r of these words says that token r
    // of a lane starts a document / lies inside the sequence.
    // kept as wave-uniform words, one pair per lane half
    uint32_t s_lo = 0, s_hi = 0, v_lo = 0xffffu, v_hi = 0xffffu;
    if (general) {
      v_lo = v_hi = 0;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int row = mt * 32 + 8 * g;  // lanes 0-31: row..row+3, 32-63: +4
        s_lo |= ((uint32_t)(m_tile >> row) & 0xfu) << (4 * g);
        s_hi |= ((uint32_t)(m_tile >> (row + 4)) & 0xfu) << (4 * g);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          v_lo |= (uint32_t)(t_half + 8 * g + q < T_len) << (4 * g + q);
          v_hi |= (uint32_t)(t_half + 8 * g + 4 + q < T_len) << (4 * g + q);
        }
      }
    }
    // Pass 1 (straight-line): a = exp2(sigmoid(pa) * decay) -> acc_a,
    // xc * sigmoid(px) -> acc_x.
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      // pre-activations are a bf16 module output in the reference
      const uint32_t px2 = pack_bf16x2(acc_x[r], acc_x[r + 1]);
      const uint32_t pa2 = pack_bf16x2(acc_a[r], acc_a[r + 1]);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int rr = r + e;
        const int i = 8 * (rr >> 2) + (rr & 3);
        const float xc = bf16_bits_to_f32(xcp[(size_t)i * kLdsStride]);
        const float px = e == 0 ? __uint_as_float(px2 << 16)
                                : __uint_as_float(px2 & 0xffff0000u);
        const float pa = e == 0 ? __uint_as_float(pa2 << 16)
                                : __uint_as_float(pa2 & 0xffff0000u);
        const float gate_x = sigmoid_fast(px);
        const float gate_a = sigmoid_fast(pa);
        acc_a[rr] = __builtin_amdgcn_exp2f(gate_a * decay);
        acc_x[rr] = xc * gate_x;
      }
      // eight tokens at a time: enough independent work to cover the latency
      // of the transcendental chains, few enough temporaries to stay in
      // registers
      if ((r & 6) == 6) __builtin_amdgcn_sched_barrier(0);
    }
    // Document start: a = 0; past the end of the sequence: a = 1.  The input
    // scale sqrt(1 - a^2) of pass 2 then comes out as 1 and 0 by itself.
    if (general) {
#pragma unroll
      for (int rr = 0; rr < 16; ++rr) {
        const bool start = upper ? (s_hi >> rr) & 1u : (s_lo >> rr) & 1u;
        const bool valid = upper ? (v_hi >> rr) & 1u : (v_lo >> rr) & 1u;
        acc_a[rr] = start ? 0.0f : acc_a[rr];
        acc_a[rr] = valid ? acc_a[rr] : 1.0f;
      }
    }
    // Pass 2: xn = (xc * gate_x) * sqrt(1 - a^2)
#pragma unroll
    for (int rr = 0; rr < 16; ++rr)
      acc_x[rr] = acc_x[rr] * __builtin_amdgcn_sqrtf(__builtin_fmaf(
                                  -acc_a[rr], acc_a[rr], 1.0f));
    __builtin_amdgcn_sched_barrier(0);
    // Recurrence.  In time order the runs of four tokens alternate between
    // the lane halves: L0 U0 L1 U1 L2 U2 L3 U3 (run g of lanes 0-31 holds
    // tokens 8g..8g+3, of lanes 32-63 tokens 8g+4..8g+7).  Per run the pair
    // (P, Hh): h_out = P h_in + Hh; both halves' pairs are made visible to all
    // lanes, every lane follows the chain and keeps the h_in of its own runs.
    // The run is replayed from its h_in and written to the patch as soon as
    // its h_in is known.
    {
      // lane-derived address, recomputed here rather than kept in a register
      int l2 = lane;
      asm volatile("" : "+v"(l2));
      unsigned char* const patch_w =
          patch + 4 * (l2 >> 5) * kPatchStride + 2 * (l2 & 31);
      float c_run = hc;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float P = acc_a[4 * g], Hh = acc_x[4 * g];
#pragma unroll
        for (int q = 1; q < 4; ++q) {
          Hh = __builtin_fmaf(acc_a[4 * g + q], Hh, acc_x[4 * g + q]);
          P = P * acc_a[4 * g + q];
        }
        float PL, PU, HL, HU;
        halves(P, PL, PU);
        halves(Hh, HL, HU);
        const float after_lower = __builtin_fmaf(PL, c_run, HL);
        float hh = upper ? after_lower : c_run;
        c_run = __builtin_fmaf(PU, after_lower, HU);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          hh = __builtin_fmaf(acc_a[4 * g + q], hh, acc_x[4 * g + q]);
          *reinterpret_cast<uint16_t*>(patch_w + (8 * g + q) * kPatchStride) =
              f32_to_bf16_bits(hh);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      hc = c_run;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    // tokens past the end of the sequence fall outside the descriptor
    {
      int l2 = lane;
      asm volatile("" : "+v"(l2));
      // read side: lane l takes the 16-byte chunk l%4 of tokens l/4, l/4+16
      const unsigned char* patch_r =
          patch + (l2 >> 2) * kPatchStride + 16 * (l2 & 3);
      const uint32_t y_lane_bytes = (uint32_t)(l2 >> 2) * row_bytes +
                                    2u * (h * kBW + n0) + 16u * (l2 & 3);
#pragma unroll
      for (int q = 0; q < 2; ++q) {
        const u32x4 v =
            *reinterpret_cast<const u32x4*>(patch_r + q * 16 * kPatchStride);
        buffer_store_16(v, ry, y_lane_bytes,
                        (uint32_t)(t_half + 16 * q) * row_bytes);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  };

  // ---- tile loop ------------------------------------------------------------
  // Phases of one tile `it` (staged in buffer it % 3):
  //   A   MFMA of tokens 0-31, with the conv of tile it+1 (into buffer
  //       (it+1) % 3) between the matrix instructions
  //   E0  gates + recurrence of tokens 0-31
  //   B   MFMA of tokens 32-63, with the row loads of tile it+2
  //   E1  gates + recurrence of tokens 32-63
  // A and B keep the matrix pipe busy, E0 and E1 the vector ALU.  Each SIMD
  // holds one wave of waves 0-3 and one of waves 4-7; the second group runs one
  // phase behind the first (it finishes E1 of a tile after the barrier that
  // ends the tile), so that on every SIMD a matrix phase of one wave overlaps a
  // vector phase of the other:
  //   waves 0-3:  A(it)    E0(it)  B(it)   E1(it)  | barrier
  //   waves 4-7:  E1(it-1) A(it)   E0(it)  B(it)   | barrier
  auto a_base = [&](int t, int bi, int mt) {
    const int l = t & 63;
    return lds + (size_t)bi * kTM * kLdsStride +
           (size_t)(mt * 32 + (l & 31)) * kLdsStride + 8 * (l >> 5);
  };
  auto a_read = [&](const uint16_t* abase, int ks) {
    Frag a;
    a.q = *reinterpret_cast<const f32x4*>(abase + ks * 16);
    return a;
  };
  auto acc_init = [&](int t, f32x16& acc_x, f32x16& acc_a) {
    const f32x2 bias = *reinterpret_cast<const f32x2*>(chan_ptr(t));
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      acc_x[r] = bias[0];
      acc_a[r] = bias[1];
    }
  };
  auto phase_a = [&](int bi, int bn, uint64_t m_next, uint64_t m_tile,
                     f32x16& acc_x, f32x16& acc_a) {
    const int t1 = fresh_tid();
    const uint16_t* abase = a_base(t1, bi, 0);
    uint16_t* const dst = stage_dst(t1, bn);
    stage_begin(t1, m_next, m_tile);
    acc_init(t1, acc_x, acc_a);
    Frag a[2];
    if (cut == 0) {
#pragma unroll
      for (int j = 0; j < kHalo; ++j) stage_row(j, dst, NoCuts{});
      a[0] = a_read(abase, 0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < 16; ++ks) {
        if (ks < 15) a[(ks + 1) & 1] = a_read(abase, ks + 1);
        acc_x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            a[ks & 1].v, bfrag[ks][0].v, acc_x, 0, 0, 0);
        acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            a[ks & 1].v, bfrag[ks][1].v, acc_a, 0, 0, 0);
        stage_row(kHalo + ks, dst, NoCuts{});
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      // a document starts among the rows of the next tile: conv first, with
      // the history cuts, then the matrix instructions
#pragma unroll
      for (int j = 0; j < kRaw; ++j) stage_row(j, dst, WithCuts{});
      a[0] = a_read(abase, 0);
#pragma unroll
      for (int ks = 0; ks < 16; ++ks) {
        if (ks < 15) a[(ks + 1) & 1] = a_read(abase, ks + 1);
        acc_x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            a[ks & 1].v, bfrag[ks][0].v, acc_x, 0, 0, 0);
        acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            a[ks & 1].v, bfrag[ks][1].v, acc_a, 0, 0, 0);
      }
    }
  };
  auto phase_b = [&](int it, int bi, f32x16& acc_x, f32x16& acc_a) {
    const int t1 = fresh_tid();
    const uint32_t cb_off = chan_bytes(t1);
    const uint16_t* abase = a_base(t1, bi, 1);
    acc_init(t1, acc_x, acc_a);
    Frag a[2];
    a[0] = a_read(abase, 0);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
      if (ks < 15) a[(ks + 1) & 1] = a_read(abase, ks + 1);
      acc_x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          a[ks & 1].v, bfrag[ks][0].v, acc_x, 0, 0, 0);
      acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          a[ks & 1].v, bfrag[ks][1].v, acc_a, 0, 0, 0);
      fetch_row(it + 2, ks, cb_off);
      if (ks + 16 < kRaw) fetch_row(it + 2, ks + 16, cb_off);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  if (!kSkewGroups || wave < 4) {
    int bi = 0;
    for (int it = 0; it < ntiles; ++it) {
      const int bn = bi == kStageBufs - 1 ? 0 : bi + 1;
      const uint64_t m_next = start_mask(it + 1);
      fetch_seg(it + 2);
      f32x16 acc_x, acc_a;
      phase_a(bi, bn, m_next, m_cur, acc_x, acc_a);
      half_epilogue(it, 0, bi, acc_x, acc_a, m_cur);
      phase_b(it, bi, acc_x, acc_a);
      half_epilogue(it, 1, bi, acc_x, acc_a, m_cur);
      // LDS-only barrier: row loads and y stores stay in flight across it
      lds_barrier();
      m_cur = m_next;
      bi = bn;
    }
  } else {
    int bi = 0, bp = 0;
    uint64_t m_prev = 0;
    f32x16 late_x, late_a;  // tokens 32-63 of the previous tile, E1 pending
#pragma unroll
    for (int r = 0; r < 16; ++r) late_x[r] = late_a[r] = 0.0f;
    for (int it = 0; it < ntiles; ++it) {
      const int bn = bi == kStageBufs - 1 ? 0 : bi + 1;
      const uint64_t m_next = start_mask(it + 1);
      fetch_seg(it + 2);
      if (it > 0) half_epilogue(it - 1, 1, bp, late_x, late_a, m_prev);
      f32x16 acc_x, acc_a;
      phase_a(bi, bn, m_next, m_cur, acc_x, acc_a);
      half_epilogue(it, 0, bi, acc_x, acc_a, m_cur);
      phase_b(it, bi, late_x, late_a);
      lds_barrier();
      m_prev = m_cur;
      m_cur = m_next;
      bp = bi;
      bi = bn;
    }
    half_epilogue(ntiles - 1, 1, bp, late_x, late_a, m_prev);
  }

  if (p.h_last && !upper) p.h_last[(int64_t)b * W + ch] = hc;

  // Masked conv state: rows T-3..T-1 of x, each zeroed if a document starts in
  // a later position of the row; rows before the sequence start are zero.
  if (p.cache_out && tid < 128) {
    uint16_t* cache = (uint16_t*)p.cache_out + (int64_t)b * 3 * W + c;
    bool later_start = false;
#pragma unroll
    for (int kk = 2; kk >= 0; --kk) {
      const int t = T_len - 3 + kk;
      uint32_t v = 0;
      if (t >= 0 && !later_start)
        v = __builtin_amdgcn_raw_buffer_load_b32(rx, c_bytes,
                                                 (uint32_t)t * row_bytes, 0);
      *reinterpret_cast<uint32_t*>(cache + (int64_t)kk * W) = v;
      if (t >= 0 && is_doc_start(p.segpos, p.seg_kind, (int64_t)b * T_len + t))
        later_start = true;
    }
  }
}

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

hipError_t launch_block_fused_bf16(const FusedArgs& a, hipStream_t s) {
  // needs head width 256 and a sequence whose rows fit 31-bit byte offsets
  // (checked by the caller)
  const int64_t blocks = (int64_t)a.B * a.H;
  if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
  hipError_t e = hipFuncSetAttribute(
      (const void*)block_fused_bf16_kernel,
      hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFusedLdsBytes);
  if (e != hipSuccess) return e;
  block_fused_bf16_kernel<<<dim3((unsigned)blocks), 512, kFusedLdsBytes, s>>>(a);
  return hipGetLastError();
}

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
