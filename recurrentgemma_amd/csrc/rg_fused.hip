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
constexpr int kRowsPerGroup = 32;  // rows each staging thread converts per tile
constexpr int kHalo = 3;
constexpr int kRaw = kRowsPerGroup + kHalo;
// Two staged tiles: the one the matrix instructions and the gate arithmetic
// read, and the one being written for the next tile (one barrier per tile).
constexpr int kStageBufs = 2;
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

  // x staging: waves 0-3 only, thread -> (channel pair, 32 tokens of the
  // tile).  The issue arbiter of a SIMD serves its older wave first, so waves
  // 4-7 (the younger wave of each SIMD) progress at about two thirds of the
  // rate of waves 0-3 while both run; leaving the conv to waves 0-3 evens out
  // the time the two groups need per tile.
  const bool stager = wave < 4;
  const int cp = tid & 127;
  const int rg = __builtin_amdgcn_readfirstlane((tid >> 7) & 1);
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
  // The same for a tile >= 1 (no row before the sequence): one scalar add per
  // row.  A tile past the end keeps every row out of range (the marker plus a
  // few rows stays above any sequence size).
  auto row_base = [&](int tile) -> uint32_t {
    return tile < ntiles ? (uint32_t)(tile * kTM + rg * kRowsPerGroup - kHalo) *
                               row_bytes
                         : kBufferOutOfRange;
  };
  auto fetch_row_at = [&](uint32_t base, int j, uint32_t cb_off) {
    raw[j] = __builtin_amdgcn_raw_buffer_load_b32(
        rx, cb_off, base + (uint32_t)j * row_bytes, 0);
  };
  auto chan_bytes = [&](int t) {  // byte offset of thread t's channel pair
    return 2u * (uint32_t)(h * kBW + (t & 127) * 2);
  };


  // Conv of one tile, one row at a time.  cut bit j: token j of this thread
  // group's 35 rows starts a document; the conv must not look past it.
  uint64_t cut = 0;
  float h0v[2], h1v[2], h2v[2];
  auto stage_dst = [&](int t, int buf) {
    return lds + (size_t)buf * kTM * kLdsStride +
           (size_t)(rg * kRowsPerGroup) * kLdsStride + (t & 127) * 2;
  };
  auto stage_begin = [&](int t, uint64_t m_tile, uint64_t m_before) {
    // rows 32*rg-3 .. 32*rg+31 of the tile; the three rows before the tile
    // are the last three of the previous one
    if (rg == 0)
      cut = ((m_tile << 3) | (m_before >> 61)) & ((1ull << kRaw) - 1);
    else
      cut = m_tile >> (kRowsPerGroup - kHalo);
    h0v[0] = h0v[1] = h1v[0] = h1v[1] = h2v[0] = h2v[1] = 0.0f;
    load_conv_consts(t);
  };
  auto stage_row = [&](int j, uint16_t* dst, auto cuts) {
    constexpr bool CUTS = decltype(cuts)::value;
    float xv[2];
    xv[0] = __uint_as_float(raw[j] << 16);
    xv[1] = __uint_as_float(raw[j] & 0xffff0000u);
    if (CUTS && ((cut >> j) & 1ull)) {
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
    if (stager) {
#pragma unroll
      for (int j = 0; j < kRaw; ++j) fetch_row(0, j, c_bytes);
    }
    m_cur = start_mask(0);
    if (stager) {
      stage_begin(tid, m_cur, 0);
#pragma unroll
      for (int j = 0; j < kRaw; ++j) stage_row(j, stage_dst(tid, 0), WithCuts{});
    }
    fetch_seg(1);
    if (stager) {
#pragma unroll
      for (int j = 0; j < kRaw; ++j) fetch_row(1, j, c_bytes);
    }
  }
  lds_barrier();

  // Gate pre-activations of one 32-token half of a tile (bias included),
  // rounded to bf16 -- they are a bf16 module output in the reference -- and
  // kept packed: word i holds accumulator registers 2i and 2i+1, i.e. tokens
  // 8*(i/2) + 4*(lane/32) + 2*(i%2) + {0,1} of channel lane%32.
  struct Packed {
    uint32_t x[8], a[8];
  };
  auto pack_acc = [&](const f32x16& acc_x, const f32x16& acc_a, Packed& pk) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pk.x[i] = pack_bf16x2(acc_x[2 * i], acc_x[2 * i + 1]);
      pk.a[i] = pack_bf16x2(acc_a[2 * i], acc_a[2 * i + 1]);
    }
  };

  // Gate arithmetic + recurrence of one 32-token half of a tile, one run of
  // four tokens at a time.  In time order the runs alternate between the lane
  // halves: L0 U0 L1 U1 L2 U2 L3 U3 (run g of lanes 0-31 holds tokens
  // 8g..8g+3, of lanes 32-63 tokens 8g+4..8g+7).  Per run the pair (P, Hh):
  // h_out = P h_in + Hh; both halves' pairs are made visible to all lanes,
  // every lane follows the chain, replays its own run from its h_in and writes
  // it to the wave's patch.  `general` also handles document starts (a = 0,
  // unit input scale) and tokens past the end of the sequence (identity:
  // a = 1, no input).
  // The work of a run is cut into eight chunks, and hook(8g + c) runs after
  // chunk c of run g, pinned there: the caller passes the matrix instructions
  // of the next half tile (32 of them) so that they issue from this wave's own
  // instruction stream, evenly spread under the vector work.
  auto half_epilogue = [&](int it, int mt, int buf, const Packed& pk,
                           uint64_t m_tile, auto&& hook) {
    const bool general = m_tile != 0 || (it + 1) * kTM > T_len;
    int l1 = lane;
    asm volatile("" : "+v"(l1));  // addresses recomputed per call, not kept
    const uint16_t* xcp = lds + (size_t)buf * kTM * kLdsStride +
                          (size_t)(mt * 32 + 4 * (l1 >> 5)) * kLdsStride + n0 +
                          (l1 & 31);
    unsigned char* const patch_w =
        patch + 4 * (l1 >> 5) * kPatchStride + 2 * (l1 & 31);
    // read side of the patch: lane l takes the 16-byte chunk l%4 of tokens
    // l/4 and l/4+16
    const unsigned char* patch_r =
        patch + (l1 >> 2) * kPatchStride + 16 * (l1 & 3);
    const uint32_t y_lane_bytes = (uint32_t)(l1 >> 2) * row_bytes +
                                  2u * (h * kBW + n0) + 16u * (l1 & 3);
    const int t_half = it * kTM + mt * 32;  // first token of this half
    const float decay = chan_ptr(l1)[2];
    // End of a chunk: its memory operations stay on this side, then the hook,
    // fenced for the instruction scheduler.  The values a chunk produces are
    // pinned by keep4() before this is called (pure arithmetic would otherwise
    // drift to its first use).
    auto pinned = [&](int i) {
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      hook(i);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" ::: "memory");
    };
    auto keep4 = [](float (&v)[4]) {
      asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
    };
    float c_run = hc;
    uint16_t xraw[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) xraw[q] = xcp[(size_t)q * kLdsStride];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      // chunk 0: unpack
      float px[4], pa[4], xc[4];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        px[2 * e] = __uint_as_float(pk.x[2 * g + e] << 16);
        px[2 * e + 1] = __uint_as_float(pk.x[2 * g + e] & 0xffff0000u);
        pa[2 * e] = __uint_as_float(pk.a[2 * g + e] << 16);
        pa[2 * e + 1] = __uint_as_float(pk.a[2 * g + e] & 0xffff0000u);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) xc[q] = bf16_bits_to_f32(xraw[q]);
      keep4(px);
      keep4(pa);
      keep4(xc);
      pinned(8 * g + 0);
      // chunks 1, 2: the two sigmoids, eight independent chains
      float ex[4], ea[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        ex[q] = __builtin_amdgcn_exp2f(-kLog2e * px[q]);
        ea[q] = __builtin_amdgcn_exp2f(-kLog2e * pa[q]);
      }
      keep4(ex);
      keep4(ea);
      pinned(8 * g + 1);
      float av[4], xn[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        ex[q] = __builtin_amdgcn_rcpf(1.0f + ex[q]);
        ea[q] = __builtin_amdgcn_rcpf(1.0f + ea[q]);
      }
      keep4(ex);
      keep4(ea);
      pinned(8 * g + 2);
      // chunk 3: a = exp2(sigmoid(pa) * decay), xc * sigmoid(px); the conv
      // outputs of the next run are requested here
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        av[q] = __builtin_amdgcn_exp2f(ea[q] * decay);
        xn[q] = xc[q] * ex[q];
      }
      keep4(av);
      keep4(xn);
      if (g < 3) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          xraw[q] = xcp[(size_t)(8 * (g + 1) + q) * kLdsStride];
      }
      pinned(8 * g + 3);
      // chunk 4: document start: a = 0; past the end of the sequence: a = 1.
      // The input scale sqrt(1 - a^2) then comes out as 1 and 0 by itself.
      if (general) {
        const int row = mt * 32 + 8 * g + (upper ? 4 : 0);
        const uint32_t starts = (uint32_t)(m_tile >> row) & 0xfu;
        const int t_run = t_half + 8 * g + (upper ? 4 : 0);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          av[q] = ((starts >> q) & 1u) ? 0.0f : av[q];
          av[q] = (t_run + q < T_len) ? av[q] : 1.0f;
        }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q)
        xn[q] = xn[q] * __builtin_amdgcn_sqrtf(
                            __builtin_fmaf(-av[q], av[q], 1.0f));
      keep4(av);
      keep4(xn);
      pinned(8 * g + 4);
      // chunk 5: the run as a pair, the chain over both lane halves
      float P = av[0], Hh = xn[0];
#pragma unroll
      for (int q = 1; q < 4; ++q) {
        Hh = __builtin_fmaf(av[q], Hh, xn[q]);
        P = P * av[q];
      }
      float PL, PU, HL, HU;
      halves(P, PL, PU);
      halves(Hh, HL, HU);
      const float after_lower = __builtin_fmaf(PL, c_run, HL);
      float hh = upper ? after_lower : c_run;
      c_run = __builtin_fmaf(PU, after_lower, HU);
      asm volatile("" : "+v"(hh), "+v"(c_run));
      pinned(8 * g + 5);
      // chunk 6: replay from this lane's h_in
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        hh = __builtin_fmaf(av[q], hh, xn[q]);
        *reinterpret_cast<uint16_t*>(patch_w + (8 * g + q) * kPatchStride) =
            f32_to_bf16_bits(hh);
      }
      pinned(8 * g + 6);
      // chunk 7: sixteen finished tokens leave as 16-byte row chunks; tokens
      // past the end of the sequence fall outside the descriptor
      if (g & 1) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const u32x4 v = *reinterpret_cast<const u32x4*>(
            patch_r + (g >> 1) * 16 * kPatchStride);
        buffer_store_16(v, ry, y_lane_bytes,
                        (uint32_t)(t_half + 16 * (g >> 1)) * row_bytes);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        __builtin_amdgcn_wave_barrier();
      }
      pinned(8 * g + 7);
    }
    hc = c_run;
  };

  // ---- tile loop ------------------------------------------------------------
  // Phases of one tile `it` (staged in buffer it % 2):
  //   A   MFMA of tokens 0-31, with the conv of tile it+1 (into buffer
  //       (it+1) % 2) between the matrix instructions
  //   E0  gates + recurrence of tokens 0-31, with the MFMA of tokens 32-63
  //       and the row loads of tile it+2 spread through it
  //   E1  gates + recurrence of tokens 32-63
  // Every matrix instruction issues from a stream that also carries vector
  // work of the same wave, so the matrix pipe runs under the vector ALU
  // whatever the other wave of the SIMD is doing (the issue arbiter serves the
  // older wave first: a wave that only has matrix instructions to issue
  // starves next to one that only has vector instructions).
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
  // A: the matrix instructions of tokens 0-31; waves 0-3 convolve their 32
  // rows of the next tile between them, one row after each instruction.
  auto phase_a = [&](auto staging, int bi, int bn, uint64_t m_next,
                     uint64_t m_tile, f32x16& acc_x, f32x16& acc_a) {
    constexpr bool STAGE = decltype(staging)::value;
    const int t1 = fresh_tid();
    const uint16_t* abase = a_base(t1, bi, 0);
    acc_init(t1, acc_x, acc_a);
    Frag a[2];
    if (STAGE) {
      uint16_t* const dst = stage_dst(t1, bn);
      stage_begin(t1, m_next, m_tile);
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
          stage_row(kHalo + 2 * ks, dst, NoCuts{});
          __builtin_amdgcn_sched_barrier(0);
          acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              a[ks & 1].v, bfrag[ks][1].v, acc_a, 0, 0, 0);
          stage_row(kHalo + 2 * ks + 1, dst, NoCuts{});
          __builtin_amdgcn_sched_barrier(0);
        }
        return;
      }
      // a document starts among the rows of the next tile: conv first, with
      // the history cuts, then the matrix instructions
#pragma unroll
      for (int j = 0; j < kRaw; ++j) stage_row(j, dst, WithCuts{});
    }
    a[0] = a_read(abase, 0);
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
      if (ks < 15) a[(ks + 1) & 1] = a_read(abase, ks + 1);
      acc_x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          a[ks & 1].v, bfrag[ks][0].v, acc_x, 0, 0, 0);
      acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          a[ks & 1].v, bfrag[ks][1].v, acc_a, 0, 0, 0);
    }
  };
  // One of the 32 matrix instructions of a half tile (hook index i): k-step
  // i/2, gate i%2; the operand of the next k-step is requested two hooks ahead.
  auto mfma_step = [&](int i, const uint16_t* abase, Frag (&a)[2],
                       f32x16& acc_x, f32x16& acc_a) {
    const int ks = i >> 1;
    if ((i & 1) == 0) {
      if (ks < 15) a[(ks + 1) & 1] = a_read(abase, ks + 1);
      acc_x = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          a[ks & 1].v, bfrag[ks][0].v, acc_x, 0, 0, 0);
    } else {
      acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          a[ks & 1].v, bfrag[ks][1].v, acc_a, 0, 0, 0);
    }
  };
  // E0 with the matrix instructions of tokens 32-63 spread through it (and,
  // in waves 0-3, the first 19 row loads of tile it+2); leaves the packed
  // pre-activations of tokens 32-63 in `out`.
  constexpr int kRowsInE0 = 19;
  static_assert(kRowsInE0 + 16 == kRaw, "row loads are split over E0 and E1");
  auto phase_e0 = [&](auto staging, int it, int bi, const Packed& pk,
                      uint64_t m_tile, Packed& out) {
    constexpr bool STAGE = decltype(staging)::value;
    const int t1 = fresh_tid();
    const uint32_t cb_off = chan_bytes(t1);
    const uint32_t base = row_base(it + 2);
    const uint16_t* abase = a_base(t1, bi, 1);
    f32x16 acc_x, acc_a;
    acc_init(t1, acc_x, acc_a);
    Frag a[2];
    a[0] = a_read(abase, 0);
    half_epilogue(it, 0, bi, pk, m_tile, [&](int i) {
      mfma_step(i, abase, a, acc_x, acc_a);
      if (STAGE && (i & 1) == 0) fetch_row_at(base, i >> 1, cb_off);
      if (STAGE && (i & 1) == 1 && (i >> 1) + 16 < kRowsInE0)
        fetch_row_at(base, (i >> 1) + 16, cb_off);
    });
    pack_acc(acc_x, acc_a, out);
  };

  // E1; waves 0-3 issue the other 16 row loads of tile it+2 in it.
  auto phase_e1 = [&](auto staging, int it, int bi, const Packed& pk,
                      uint64_t m_tile) {
    constexpr bool STAGE = decltype(staging)::value;
    const int t1 = fresh_tid();
    const uint32_t cb_off = chan_bytes(t1);
    const uint32_t base = row_base(it + 2);
    half_epilogue(it, 1, bi, pk, m_tile, [&](int i) {
      if (STAGE && (i & 1) == 0)
        fetch_row_at(base, kRowsInE0 + (i >> 1), cb_off);
    });
  };

  auto tile_loop = [&](auto staging) {
    int bi = 0;
    for (int it = 0; it < ntiles; ++it) {
      const int bn = bi == kStageBufs - 1 ? 0 : bi + 1;
      const uint64_t m_next = start_mask(it + 1);
      fetch_seg(it + 2);
      Packed pk, pk1;
      {
        f32x16 acc_x, acc_a;
        phase_a(staging, bi, bn, m_next, m_cur, acc_x, acc_a);
        pack_acc(acc_x, acc_a, pk);
      }
      phase_e0(staging, it, bi, pk, m_cur, pk1);
      phase_e1(staging, it, bi, pk1, m_cur);
      // LDS-only barrier: row loads and y stores stay in flight across it
      lds_barrier();
      m_cur = m_next;
      bi = bn;
    }
  };
  if (stager)
    tile_loop(std::true_type{});
  else
    tile_loop(std::false_type{});

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
  static OncePerDevice once;
  hipError_t e = set_max_dynamic_lds(
      once, (const void*)block_fused_bf16_kernel, kFusedLdsBytes);
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
