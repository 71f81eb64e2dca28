// Whole recurrent core of a prefill in one launch (bf16, 256-wide heads):
// width-4 conv -> both gate projections on MFMA -> gate activations -> linear
// recurrence.  Neither the conv output nor the gate pre-activations ever go to
// memory: per element the kernel reads x once and writes y once.
//
// The form with ONE wave per SIMD.  One workgroup of four waves -- each with
// its SIMD's whole register file -- per (sequence row b, head h), or per (b, h,
// chunk of the sequence), walks its tokens in tiles of 64.  Wave w owns 64
// channels of the head for both gates; its 2 x 256 x 64 weights (256
// registers) stay resident for the whole kernel, and the matrix instructions
// of the next 32 tokens are pinned between the pieces of the gate arithmetic
// of the current ones.  A lone wave issues in order, one instruction per four
// cycles at best, and 68 % of the slots at that: the form with two waves per
// SIMD that alternate between a matrix phase and a gate phase
// (rg_prefill_teams.hip) is 10-20 % faster and is what callers with
// re-laid-out weights get.  This form serves weights in the reference layout
// (transposed through LDS in the prologue) and is the second implementation
// that the bit-equality tests hold the other one against.
//
// Replaces the chain Conv1D.forward -> RGLRU.forward of
// recurrentgemma/torch/modules.py:632-643 (layers.py:447-529, 313-365,
// 140-191) for prefill.
#include <type_traits>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;    // head width (K and per-gate N)
constexpr int kTM = 64;     // tokens per tile
constexpr int kWaves = 4;   // waves per workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kNB = 2;      // 32-channel groups per wave
// Conv output of a tile (the MFMA A operand), bf16, rows padded to 264
// elements so that the 16-byte operand reads spread over the banks.
constexpr int kXcStride = 264;
constexpr int kXcRowBytes = kXcStride * 2;
constexpr int kXcTileBytes = kTM * kXcRowBytes;
// Raw x of a tile as the memory pipe writes it into LDS: rows -4 .. 63 of the
// tile (row -4 only keeps the row pairs aligned), 512 bytes each, unpadded.
constexpr int kRawHalo = 4;
constexpr int kRawRows = kTM + kRawHalo;
constexpr int kRawRowBytes = kBW * 2;
constexpr int kRawLoads = kRawRows / 2;  // wave-wide 16-byte loads per tile
// ... shared out evenly: every wave issues the same number of loads without
// looking at its wave number (a branch per load costs a lone wave more than
// the load); the loads beyond kRawLoads are sent out of range and fill rows
// of padding behind the tile with zeros
constexpr int kRawLoadsPerWave = (kRawLoads + kWaves - 1) / kWaves;
constexpr int kRawTileBytes = kRawLoadsPerWave * kWaves * 2 * kRawRowBytes;
// Per-wave output patch: 16 tokens x 64 channels in bf16, rows padded to 144
// bytes (16-byte aligned row reads, spread over the banks).
constexpr int kPatchStride = 144;
constexpr int kPatchBytesPerWave = 16 * kPatchStride;

constexpr int kXcOff = 0;
constexpr int kRawOff = kXcOff + 2 * kXcTileBytes;
constexpr int kPatchOff = kRawOff + 2 * kRawTileBytes;
// Conv taps of the 128 channel pairs, 8 words per pair: the taps of both
// channels as bf16 pairs (w0|w1, w2|w3: operands of the two-element dot
// product), both biases as floats, two words of padding.
constexpr int kConvTabOff = kPatchOff + kWaves * kPatchBytesPerWave;
constexpr int kPrefillLdsBytes = kConvTabOff + 128 * 32;
static_assert(kPrefillLdsBytes <= 160 * 1024, "LDS of one CU");
static_assert(2 * kXcTileBytes >= 128 * kXcRowBytes,
              "the weight transpose borrows the conv-output tiles");

typedef __attribute__((address_space(3))) unsigned char lds_byte;

union Frag {
  bf16x8 v;
  uint16_t u[8];
  f32x4 q;
};

// What one workgroup does with its tiles.  A row cut into chunks takes two
// launches: the first runs chunk 0 as kChunkHead and chunks 1 .. n-2 as
// kChunkSummary side by side, the second chunks 1 .. n-1 as kChunkReplay,
// each starting from the summaries of the chunks before it.
enum PrefillMode {
  kWholeRow = 0,      // a whole row of one head: y, h_last, conv state
  kChunkSummary = 1,  // a chunk from a zero state: (prod a, h_end), no y
  kChunkReplay = 2,   // a chunk from its incoming state: y, ...
  kChunkHead = 3      // chunk 0 from h0: y, and its end state as a summary
};

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding:
// vmcnt in bits 3:0 and 15:14, expcnt 6:4, lgkmcnt 11:8).
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// v_dot2_f32_bf16: a.lo * b.lo + a.hi * b.hi + c on two bf16 pairs, written as
// the three-operand instruction (the builtin selects the accumulate-in-place
// form and copies c into the destination first).  The result of a dot
// instruction may be read by an instruction of another kind only three issue
// slots later, and the compiler does not insert those for inline assembly: the
// helpers below chain whole groups and end with the wait themselves.

// out[c] = bias[c] + p_old[c] . w10[c] + p_new[c] . w32[c] for two channels.
__device__ __forceinline__ void conv_dot_row(const uint32_t (&p_old)[2],
                                             const uint32_t (&p_new)[2],
                                             const uint32_t (&w10)[2],
                                             const uint32_t (&w32)[2],
                                             const float (&bias)[2],
                                             float (&out)[2]) {
  asm("v_dot2_f32_bf16 %0, %2, %6, %10\n\t"
      "v_dot2_f32_bf16 %1, %3, %7, %11\n\t"
      "v_dot2_f32_bf16 %0, %4, %8, %0\n\t"
      "v_dot2_f32_bf16 %1, %5, %9, %1\n\t"
      "s_nop 2"
      : "=&v"(out[0]), "=&v"(out[1])
      : "v"(p_old[0]), "v"(p_old[1]), "v"(p_new[0]), "v"(p_new[1]),
        "v"(w10[0]), "v"(w10[1]), "v"(w32[0]), "v"(w32[1]), "v"(bias[0]),
        "v"(bias[1]));
}
// The same for two rows at once: `even` from (o_old, o_new), `odd` from
// (e_old, e_new).
__device__ __forceinline__ void conv_dot_row_pair(
    const uint32_t (&o_old)[2], const uint32_t (&o_new)[2],
    const uint32_t (&e_old)[2], const uint32_t (&e_new)[2],
    const uint32_t (&w10)[2], const uint32_t (&w32)[2], const float (&bias)[2],
    float (&even)[2], float (&odd)[2]) {
  asm("v_dot2_f32_bf16 %0, %4, %12, %16\n\t"
      "v_dot2_f32_bf16 %1, %5, %13, %17\n\t"
      "v_dot2_f32_bf16 %2, %8, %12, %16\n\t"
      "v_dot2_f32_bf16 %3, %9, %13, %17\n\t"
      "v_dot2_f32_bf16 %0, %6, %14, %0\n\t"
      "v_dot2_f32_bf16 %1, %7, %15, %1\n\t"
      "v_dot2_f32_bf16 %2, %10, %14, %2\n\t"
      "v_dot2_f32_bf16 %3, %11, %15, %3\n\t"
      "s_nop 2"
      : "=&v"(even[0]), "=&v"(even[1]), "=&v"(odd[0]), "=&v"(odd[1])
      : "v"(o_old[0]), "v"(o_old[1]), "v"(o_new[0]), "v"(o_new[1]),
        "v"(e_old[0]), "v"(e_old[1]), "v"(e_new[0]), "v"(e_new[1]),
        "v"(w10[0]), "v"(w10[1]), "v"(w32[0]), "v"(w32[1]), "v"(bias[0]),
        "v"(bias[1]));
}

// The wave's 64 weight fragments (k-step, channel group, gate: fragment F =
// 4 k + 2 group + gate, four registers each) live in the accumulation
// registers a[4F : 4F+3] for the whole kernel -- the second half of a lone
// wave's 512 registers, which only matrix instructions can read directly.
// They are written and read by inline assembly with the register numbers
// spelled out, so that the register allocator never sees them (left to it, it
// moved fragments in and out of ordinary registers inside the tile loop).
#define RG_FRAG_CASES(X)                                                       \
  X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13)    \
  X(14) X(15) X(16) X(17) X(18) X(19) X(20) X(21) X(22) X(23) X(24) X(25)      \
  X(26) X(27) X(28) X(29) X(30) X(31) X(32) X(33) X(34) X(35) X(36) X(37)      \
  X(38) X(39) X(40) X(41) X(42) X(43) X(44) X(45) X(46) X(47) X(48) X(49)      \
  X(50) X(51) X(52) X(53) X(54) X(55) X(56) X(57) X(58) X(59) X(60) X(61)      \
  X(62) X(63)

// fragment F <- v (F is a constant wherever this is inlined: one case stays)
__device__ __forceinline__ void set_weight_frag(int F, f32x4 v) {
  switch (F) {
#define RG_SET_CASE(F)                                                   \
  case F:                                                                \
    asm volatile("v_accvgpr_write_b32 a[" #F "*4], %0\n\t"               \
                 "v_accvgpr_write_b32 a[" #F "*4+1], %1\n\t"             \
                 "v_accvgpr_write_b32 a[" #F "*4+2], %2\n\t"             \
                 "v_accvgpr_write_b32 a[" #F "*4+3], %3"                  \
                 :                                                       \
                 : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3])            \
                 : "a255");                                              \
    break;
    RG_FRAG_CASES(RG_SET_CASE)
#undef RG_SET_CASE
  }
}
// acc = a x fragment F (+ acc unless `first`): v_mfma_f32_32x32x16_bf16 with
// the accumulator in ordinary registers, where the gate arithmetic reads it
// without a copy.  The compiler does not know what the instruction is: the
// caller keeps every reader of `acc` behind wait_for_matrix_results().
__device__ __forceinline__ void mfma_weight_frag(int F, bool first,
                                                 const f32x4& a, f32x16& acc) {
  switch (F) {
#define RG_MFMA_CASE(F)                                                        \
  case F:                                                                      \
    if (first)                                                                 \
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, a[" #F "*4:" #F "*4+3], 0" \
                   : "=&v"(acc)                                                \
                   : "v"(a));                                                  \
    else                                                                       \
      asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, a[" #F "*4:" #F            \
                   "*4+3], %0"                                                 \
                   : "+v"(acc)                                                 \
                   : "v"(a));                                                  \
    break;
    RG_FRAG_CASES(RG_MFMA_CASE)
#undef RG_MFMA_CASE
  }
}

// Accumulators of one 32-token block: [32-channel group][gate], each the
// 32 x 32 result of v_mfma_f32_32x32x16_bf16 (16 registers per lane).
struct BlockAcc {
  f32x16 v[kNB][2];
};

template <int MODE, bool GELU>
__device__ __forceinline__ void prefill_body(const FusedArgs& p,
                                             const int chunk) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  lds_byte* const lds3 = (lds_byte*)lds_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.x / p.H;
  const int h = blockIdx.x % p.H;
  const int T_len = p.T;
  const int64_t W = p.W;
  const int ntiles_all = (T_len + kTM - 1) / kTM;
  const int tile_begin = MODE == kWholeRow ? 0 : chunk * p.tiles_per_chunk;
  int tile_end = MODE == kWholeRow ? ntiles_all : tile_begin + p.tiles_per_chunk;
  if (tile_end > ntiles_all) tile_end = ntiles_all;
  const bool last_chunk = tile_end == ntiles_all;
  const bool upper = lane >= 32;
  const int n0 = wave * (32 * kNB);  // first channel of this wave in the head

  // ---- this wave's weights: 64 channels of the head, both gates ----------
  // The weights are [k][n] with n contiguous, the MFMA B operand wants 8
  // consecutive k per lane: either the caller supplies them re-laid-out
  // (per 32-channel group: k-step, gate, lane, 8 values), or they are
  // transposed through LDS here, 128 k-rows of one gate at a time.
  if (p.w_packed) {
    // 32 fragments at a time: all their loads are in flight before the first
    // is moved (left to itself the compiler waits for every load in turn)
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      const f32x4* src = reinterpret_cast<const f32x4*>(p.w_packed) +
                         ((int64_t)(h * 8 + wave * kNB + nb) * 16 * 2) * 64 +
                         lane;
      f32x4 w[32];
#pragma unroll
      for (int i = 0; i < 32; ++i) w[i] = src[i * 64];
#pragma unroll
      for (int i = 0; i < 32; i += 16)
        asm volatile("" ::"v"(w[i]), "v"(w[i + 1]), "v"(w[i + 2]),
                     "v"(w[i + 3]), "v"(w[i + 4]), "v"(w[i + 5]),
                     "v"(w[i + 6]), "v"(w[i + 7]), "v"(w[i + 8]),
                     "v"(w[i + 9]), "v"(w[i + 10]), "v"(w[i + 11]),
                     "v"(w[i + 12]), "v"(w[i + 13]), "v"(w[i + 14]),
                     "v"(w[i + 15]));
#pragma unroll
      for (int ks = 0; ks < 16; ++ks)
#pragma unroll
        for (int g = 0; g < 2; ++g)
          set_weight_frag(4 * ks + 2 * nb + g, w[ks * 2 + g]);
    }
  } else {
    uint16_t* const lds = reinterpret_cast<uint16_t*>(lds_raw);
#pragma unroll
    for (int g = 0; g < 2; ++g) {
#pragma unroll
      for (int kh = 0; kh < 2; ++kh) {
        const uint16_t* src =
            (const uint16_t*)p.w[g] + ((int64_t)h * kBW + kh * 128) * kBW;
        for (int e = tid; e < 128 * 32; e += kThreads) {
          const int r = e >> 5, q = e & 31;
          *reinterpret_cast<f32x4*>(lds + (size_t)r * kXcStride + q * 8) =
              *reinterpret_cast<const f32x4*>(src + (size_t)r * kBW + q * 8);
        }
        __syncthreads();
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
          for (int ks = 0; ks < 8; ++ks) {
            const int n = n0 + 32 * nb + (lane & 31);
            const int kb = ks * 16 + 8 * (lane >> 5);
            Frag f;
#pragma unroll
            for (int e = 0; e < 8; ++e)
              f.u[e] = lds[(size_t)(kb + e) * kXcStride + n];
            set_weight_frag(4 * (kh * 8 + ks) + 2 * nb + g, f.q);
          }
        __syncthreads();
      }
    }
  }

  // ---- conv table -------------------------------------------------------------
  if (tid < 128) {
    // Without conv weights x is the conv output already (a stand-alone
    // RG-LRU): the table then holds the identity, w3 = 1 and nothing else,
    // which hands every finite x[t] through exactly.
    uint32_t u0 = 0, u1 = 0, u2 = 0, u3 = 0x3f803f80u, ub = 0;
    if (p.conv_w != nullptr) {
      const uint16_t* cw = (const uint16_t*)p.conv_w + h * kBW + tid * 2;
      u0 = *reinterpret_cast<const uint32_t*>(cw);
      u1 = *reinterpret_cast<const uint32_t*>(cw + W);
      u2 = *reinterpret_cast<const uint32_t*>(cw + 2 * W);
      u3 = *reinterpret_cast<const uint32_t*>(cw + 3 * W);
      ub = *reinterpret_cast<const uint32_t*>(
          (const uint16_t*)p.conv_b + h * kBW + tid * 2);
    }
    // w0 multiplies x[t-3], w3 multiplies x[t] (layers.py:514)
    const u32x4 t0 = {(u0 & 0xffffu) | (u1 << 16), (u2 & 0xffffu) | (u3 << 16),
                      (u0 >> 16) | (u1 & 0xffff0000u),
                      (u2 >> 16) | (u3 & 0xffff0000u)};
    const u32x4 t1 = {ub << 16, ub & 0xffff0000u, 0u, 0u};
    *reinterpret_cast<u32x4*>(lds_raw + kConvTabOff + tid * 32) = t0;
    *reinterpret_cast<u32x4*>(lds_raw + kConvTabOff + tid * 32 + 16) = t1;
  }

  // ---- addressing ---------------------------------------------------------
  const uint32_t row_bytes = 2u * (uint32_t)p.W;
  const uint32_t seq_bytes = (uint32_t)T_len * row_bytes;  // < 2^31 (launcher)
  const __amdgpu_buffer_rsrc_t rx =
      make_rsrc((const char*)p.x + (int64_t)b * seq_bytes, seq_bytes);
  const __amdgpu_buffer_rsrc_t ry = make_rsrc(
      (char*)p.y + (int64_t)b * seq_bytes, MODE == kChunkSummary ? 0 : seq_bytes);
  // GELU: the block's other branch, read where y is written
  const __amdgpu_buffer_rsrc_t rgate = make_rsrc(
      (const char*)p.gate_branch + (int64_t)b * seq_bytes,
      GELU && MODE != kChunkSummary ? seq_bytes : 0);
  const bool seg_is64 = p.seg_kind == kSegI64;
  const uint32_t seg_esize = seg_is64 ? 8u : 4u;
  const __amdgpu_buffer_rsrc_t rseg =
      make_rsrc((const char*)p.segpos + (int64_t)b * T_len * seg_esize,
                (uint32_t)T_len * seg_esize);

  // Document starts of a tile: lane j looks at token 64*tile + j.  Two
  // unconditional 32-bit loads (for int32 positions the high half is sent out
  // of range and reads as zero); tokens past the end are masked out.
  uint32_t seg_lo = 1, seg_hi = 0;
  auto fetch_seg = [&](int tile) {
    const int t = tile * kTM + lane;
    const uint32_t off = (tile >= 0 && tile < ntiles_all && t < T_len)
                             ? (uint32_t)t * seg_esize
                             : kBufferOutOfRange;
    seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
    seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
        rseg, seg_is64 ? off + 4u : kBufferOutOfRange, 0, 0);
  };
  auto start_mask = [&](int tile) -> uint64_t {
    uint32_t lo = seg_lo, hi = seg_hi;
    asm volatile("" : "+v"(lo), "+v"(hi));  // test here, a tile after the load
    const int t = tile * kTM + lane;
    return __ballot(tile >= 0 && tile < ntiles_all && t < T_len &&
                    (lo | hi) == 0u);
  };

  // Raw x of one tile -> LDS, written by the memory pipe itself (no
  // registers): 34 wave-wide loads of two rows each, shared out over the
  // waves.  Rows before the sequence and past its end fall outside the
  // descriptor and arrive as zeros.
  const uint32_t dma_lane_off =
      2u * (uint32_t)(h * kBW) + 16u * (uint32_t)(lane & 31);
  auto dma_tile = [&](int tile, int buf) {
    lds_byte* const dst = lds3 + kRawOff + buf * kRawTileBytes;
    const int t0 = tile * kTM - kRawHalo + (lane >> 5);
#pragma unroll
    for (int j = 0; j < kRawLoadsPerWave; ++j) {
      const int i = wave + kWaves * j;
      uint32_t voff = (uint32_t)((t0 + 2 * i) * (int)row_bytes) + dma_lane_off;
      if (kWaves * j + kWaves > kRawLoads)  // the last round only
        voff = i < kRawLoads ? voff : kBufferOutOfRange;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, dst + i * 1024, 16, voff, 0,
                                               0, 0);
    }
  };

  // ---- lane-dependent LDS offsets, kept for the whole kernel ----------------
  // Every LDS access below is one of these plus a compile-time constant (the
  // buffer index of a tile is a template argument of the tile body), so no
  // address arithmetic is left in the tile loop.
  const int rgp = __builtin_amdgcn_readfirstlane(tid >> 7);  // 0..1
  constexpr int kConvRows = 32 / (kThreads / 128);  // rows per thread and half
  // conv: thread -> (channel pair tid % 128, rows kConvRows rgp .. of a 32-row
  // half tile); row r of a tile lies at raw row r + kRawHalo
  const uint32_t conv_raw_lane =
      kRawOff + (uint32_t)(rgp * kConvRows + kRawHalo) * kRawRowBytes +
      (tid & 127) * 4;
  const uint32_t conv_xc_lane =
      kXcOff + (uint32_t)(rgp * kConvRows) * kXcRowBytes + (tid & 127) * 4;
  // gates: lane -> channel n0 + 32 nb + lane % 32, tokens 4 (lane / 32) + ...
  const uint32_t xc_lane = kXcOff + 4u * (lane >> 5) * kXcRowBytes +
                           2u * (uint32_t)(n0 + (lane & 31));
  // MFMA A operand: lane -> token lane % 32, k offset 8 (lane / 32)
  const uint32_t a_lane = kXcOff + (uint32_t)(lane & 31) * kXcRowBytes +
                          16u * (lane >> 5);
  // output patch of this wave: written as token 4 (lane / 32) + q (+ 8 for
  // odd runs), channel 32 nb + lane % 32; read back as 16-byte row chunks,
  // lane l taking chunk l % 8 of tokens l / 8 and l / 8 + 8
  const uint32_t patch_w_lane = kPatchOff + wave * kPatchBytesPerWave +
                                4u * (lane >> 5) * kPatchStride +
                                2u * (lane & 31);
  const uint32_t patch_r_lane = kPatchOff + wave * kPatchBytesPerWave +
                                (uint32_t)(lane >> 3) * kPatchStride +
                                16u * (lane & 7);
  const uint32_t y_lane_bytes = (uint32_t)(lane >> 3) * row_bytes +
                                2u * (uint32_t)(h * kBW + n0) + 16u * (lane & 7);

  // ---- width-4 conv: raw rows (LDS) -> bf16 conv output (LDS) --------------
  // Per channel the rows are paired in time, P_t = (x[t-1], x[t]) as two bf16
  // in one register, and
  //   out[t] = bias + P_{t-2} . (w0, w1) + P_t . (w2, w3)
  // is two v_dot2_f32_bf16.  Two output rows at a time: E = (x[2j], x[2j+1])
  // serves row 2j+1, O = (x[2j-1], x[2j]) (funnel shift of two E) row 2j.
  uint32_t cw10[2], cw32[2];
  float cbias[2];
  uint32_t e_prev[2], o_prev[2];
  auto raw_row = [&](int buf, int half, int r) {
    return *reinterpret_cast<const uint32_t*>(
        lds_raw + conv_raw_lane + buf * kRawTileBytes +
        (half * 32 + r) * kRawRowBytes);
  };
  auto xc_row = [&](int buf, int half, int r) {
    return reinterpret_cast<uint32_t*>(lds_raw + conv_xc_lane +
                                       buf * kXcTileBytes +
                                       (half * 32 + r) * kXcRowBytes);
  };
  constexpr uint32_t kSelLo = 0x05040100u;  // (lo16(earlier), lo16(later))
  constexpr uint32_t kSelHi = 0x07060302u;  // (hi16(earlier), hi16(later))
  auto pair_rows = [&](uint32_t earlier, uint32_t later, uint32_t (&out)[2]) {
    out[0] = __builtin_amdgcn_perm(later, earlier, kSelLo);
    out[1] = __builtin_amdgcn_perm(later, earlier, kSelHi);
  };
  auto conv_pair = [&](uint32_t ra, uint32_t rb, int buf, int half, int j) {
    uint32_t e[2], o[2];
    pair_rows(ra, rb, e);
    float even[2], odd[2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
      o[c] = __builtin_amdgcn_alignbit(e[c], e_prev[c], 16);
    conv_dot_row_pair(o_prev, o, e_prev, e, cw10, cw32, cbias, even, odd);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      e_prev[c] = e[c];
      o_prev[c] = o[c];
    }
    *xc_row(buf, half, 2 * j) = pack_bf16x2(even[0], even[1]);
    *xc_row(buf, half, 2 * j + 1) = pack_bf16x2(odd[0], odd[1]);
  };
  // The same rows one at a time, with the history cut at document starts:
  // bit i of `cuts` says that row i - 3 of these rows starts a document.
  // Same dot products in the same order as the paired form.
  auto conv_rows_with_cuts = [&](int buf, int half, uint32_t cuts) {
    uint32_t r_prev = 0, p1[2] = {0, 0}, p2[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < kConvRows + 3; ++i) {
      const uint32_t r = raw_row(buf, half, i - 3);
      if ((cuts >> i) & 1u) {
        r_prev = 0;
        p1[0] = p1[1] = p2[0] = p2[1] = 0;
      }
      uint32_t pt[2];
      pair_rows(r_prev, r, pt);
      if (i >= 3) {
        float o[2];
        conv_dot_row(p2, pt, cw10, cw32, cbias, o);
        *xc_row(buf, half, i - 3) = pack_bf16x2(o[0], o[1]);
      }
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        p2[c] = p1[c];
        p1[c] = pt[c];
      }
      r_prev = r;
    }
  };
  // Document starts among this thread group's rows (3 before + its own) of
  // half `half` of a tile with start mask m_tile, m_before being the mask of
  // the tile before it.
  auto conv_cuts = [&](int half, uint64_t m_tile, uint64_t m_before) -> uint32_t {
    // first row of the group: 32 half + kConvRows rgp; bit i <- row first - 3 + i
    // (written without a choice between the two forms at run time: a branch
    // costs a lone wave tens of cycles)
    const uint64_t bits =
        half == 0 ? ((m_tile << 3) | (m_before >> 61)) >> (rgp * kConvRows)
                  : m_tile >> (29 + rgp * kConvRows);
    return (uint32_t)bits & ((1u << (kConvRows + 3)) - 1u);
  };

  // ---- MFMA operand reads -----------------------------------------------------
  auto a_read = [&](int buf, int blk, int ks) {
    Frag a;
    a.q = *reinterpret_cast<const f32x4*>(lds_raw + a_lane + buf * kXcTileBytes +
                                          blk * 32 * kXcRowBytes + ks * 32);
    return a;
  };
  // One of the 64 matrix instructions of a 32-token block (index i): k-step
  // i/4, channel group (i/2)%2, gate i%2; the operand of a later k-step is
  // requested ahead (ring of kARing fragments).  The first instruction of each
  // accumulator starts from zero (no accumulator initialisation; the bias is
  // added with the gate arithmetic).
  constexpr int kARing = 3;
  auto mfma_step = [&](int i, int buf, int blk, Frag (&a)[kARing],
                       BlockAcc& acc) {
    const int ks = i >> 2, nb = (i >> 1) & 1, g = i & 1;
    if ((i & 3) == 0 && ks + kARing - 1 < 16)
      a[(ks + kARing - 1) % kARing] = a_read(buf, blk, ks + kARing - 1);
    mfma_weight_frag(i, ks == 0, a[ks % kARing].q, acc.v[nb][g]);
  };
  // The result of a matrix instruction may be read by a vector instruction
  // only after its passes are through (19 issue slots for this shape); the
  // compiler does not count them for inline assembly.
  auto wait_for_matrix_results = [&]() {
    asm volatile("s_nop 15\n\ts_nop 7");
  };
  auto a_ring_begin = [&](int buf, int blk, Frag (&a)[kARing]) {
#pragma unroll
    for (int k = 0; k < kARing - 1; ++k) a[k] = a_read(buf, blk, k);
  };

  // ---- gate arithmetic + recurrence of one 32-token block --------------------
  // The MFMA result gives a lane one channel (lane % 32) of each of its two
  // channel groups and 16 tokens in runs of four that alternate between the
  // lane halves: run g of lanes 0-31 holds tokens 8g..8g+3, of lanes 32-63
  // tokens 8g+4..8g+7.  Per run the recurrence is walked twice: first from the
  // carried state (right for lanes 0-31, whose end value is handed to lanes
  // 32-63 with one permlane32_swap), then again from each half's own incoming
  // state (right for all lanes); the end value of lanes 32-63 is the carry of
  // the next run.  `general` also handles document starts (a = 0, unit input
  // scale) and tokens past the end of the sequence (identity: a = 1, no
  // input).
  // The eight runs of a block (4 runs x 2 channel groups) are cut into eight
  // pieces each, and hook(8 r + c) runs after piece c of run r, pinned there:
  // the caller passes matrix instructions and conv rows so that they issue
  // from this wave's own instruction stream, spread under the gate
  // arithmetic.
  // Finished tokens go through the wave's LDS patch, sixteen at a time, and
  // leave as 16-byte row chunks; the stores are issued a run after the patch
  // was read so that they do not wait for the LDS (y_pending).
  float bias_x[kNB], bias_a[kNB], decay[kNB];  // times -log2(e), see prologue
  float hc[kNB] = {0.0f, 0.0f};    // carried state of this lane's channels
  float prod[kNB] = {1.0f, 1.0f};  // kChunkSummary: product of a, own tokens
  u32x4 y_pending[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  u32x4 g_pending[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};  // GELU: same positions
  uint32_t y_pending_row = kBufferOutOfRange;  // byte offset of its first row
  auto flush_y_half = [&](int j) {
    if (GELU) {
      // y * gelu(gate branch), each factor a bf16 tensor as in the reference
      // (recurrentgemma/torch/modules.py:627-628, 644): the arithmetic and
      // roundings of the stand-alone gelu_mul pass
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float lo = gelu_mul_bf16(__uint_as_float(y_pending[j][k] << 16),
                                       __uint_as_float(g_pending[j][k] << 16));
        const float hi =
            gelu_mul_bf16(__uint_as_float(y_pending[j][k] & 0xffff0000u),
                          __uint_as_float(g_pending[j][k] & 0xffff0000u));
        y_pending[j][k] = pack_bf16x2(lo, hi);
      }
    }
    buffer_store_16(y_pending[j], ry, y_lane_bytes,
                    y_pending_row + (uint32_t)(8 * j) * row_bytes);
  };
  auto flush_y = [&]() {
    flush_y_half(0);
    flush_y_half(1);
  };
  auto gate_block = [&](int it, int blk, auto BI, const BlockAcc& acc,
                        uint64_t m_tile, auto&& hook) {
    constexpr int bi = decltype(BI)::value;
    const bool general = m_tile != 0 || (it + 1) * kTM > T_len;
    const int t_blk = it * kTM + blk * 32;  // first token of this block
    auto xc_at = [&](int nb, int r) {
      return *reinterpret_cast<const uint16_t*>(
          lds_raw + xc_lane + bi * kXcTileBytes + (blk * 32 + r) * kXcRowBytes +
          64 * nb);
    };
    auto pinned = [&](int i) {
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      hook(i);
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" ::: "memory");
    };
    uint16_t xraw[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) xraw[q] = xc_at(0, q);
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const int g = r >> 1, nb = r & 1;
      const f32x16& acc_x = acc.v[nb][0];
      const f32x16& acc_a = acc.v[nb][1];
      // piece 0: exponents of both sigmoids, -log2(e) (pre-activation + bias)
      float sx[4], sa[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        sx[q] = __builtin_fmaf(acc_x[4 * g + q], -kLog2e, bias_x[nb]);
        sa[q] = __builtin_fmaf(acc_a[4 * g + q], -kLog2e, bias_a[nb]);
      }
      pinned(8 * r + 0);
      // pieces 1, 2: the two sigmoids, eight independent chains
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        sx[q] = __builtin_amdgcn_exp2f(sx[q]);
        sa[q] = __builtin_amdgcn_exp2f(sa[q]);
      }
      pinned(8 * r + 1);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        sx[q] = __builtin_amdgcn_rcpf(1.0f + sx[q]);
        sa[q] = __builtin_amdgcn_rcpf(1.0f + sa[q]);
      }
      // the sixteen tokens read back from the patch two runs ago leave now
      if (MODE != kChunkSummary && (r & 3) == 1) flush_y();
      pinned(8 * r + 2);
      // piece 3: a = exp2(sigmoid(pa) * decay), xc * sigmoid(px); the conv
      // outputs of the next run are requested here
      float av[4], xn[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        av[q] = __builtin_amdgcn_exp2f(sa[q] * decay[nb]);
        xn[q] = bf16_bits_to_f32(xraw[q]) * sx[q];
      }
      if (r < 7) {
        const int g1 = (r + 1) >> 1, nb1 = (r + 1) & 1;
#pragma unroll
        for (int q = 0; q < 4; ++q) xraw[q] = xc_at(nb1, 8 * g1 + q);
      }
      pinned(8 * r + 3);
      // piece 4: document start: a = 0; past the end of the sequence: a = 1,
      // no input.  The input scale sqrt(1 - a^2) comes out as 1 at a start.
      if (__builtin_expect(general, 0)) {
        // (kept a branch: as selects it would cost the common case 3.5 vector
        // instructions per element)
        // (the lane's row offset passes through an empty statement here so
        // that what is computed from it -- the shifted mask, four token
        // numbers -- stays inside the branch: hoisted above it, as the
        // compiler does otherwise, it is five vector instructions per run on
        // the path that needs none of them)
        int half_rows = upper ? 4 : 0;
        asm volatile("" : "+v"(half_rows));
        const int row = blk * 32 + 8 * g + half_rows;
        const uint32_t starts = (uint32_t)(m_tile >> row) & 0xfu;
        const int t_run = t_blk + 8 * g + half_rows;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          av[q] = ((starts >> q) & 1u) ? 0.0f : av[q];
          av[q] = (t_run + q < T_len) ? av[q] : 1.0f;
          xn[q] = (t_run + q < T_len) ? xn[q] : 0.0f;
        }
      }
#pragma unroll
      for (int q = 0; q < 4; ++q)
        xn[q] = xn[q] *
                __builtin_amdgcn_sqrtf(__builtin_fmaf(-av[q], av[q], 1.0f));
      pinned(8 * r + 4);
      // piece 5: first walk, from the carried state; lanes 32-63 then start
      // from the end value of lanes 0-31
      float e1 = hc[nb];
#pragma unroll
      for (int q = 0; q < 4; ++q) e1 = __builtin_fmaf(av[q], e1, xn[q]);
      float hh;
      {
        const auto sw = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(hc[nb]), __float_as_uint(e1), false, false);
        hh = __uint_as_float(sw[0]);  // lanes 0-31: carry, 32-63: e1 of 0-31
      }
      asm volatile("" : "+v"(hh));
      pinned(8 * r + 5);
      // piece 6: second walk, right for every lane
      float hv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        hh = __builtin_fmaf(av[q], hh, xn[q]);
        hv[q] = hh;
      }
      {
        const auto sw = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(hh), __float_as_uint(hh), false, false);
        hc[nb] = __uint_as_float(sw[1]);  // all lanes: end value of 32-63
      }
      if (MODE == kChunkSummary) {
#pragma unroll
        for (int q = 0; q < 4; ++q) prod[nb] *= av[q];
      } else {
        const uint32_t y01 = pack_bf16x2(hv[0], hv[1]);
        const uint32_t y23 = pack_bf16x2(hv[2], hv[3]);
        unsigned char* const pw = lds_raw + patch_w_lane +
                                  (8 * (g & 1)) * kPatchStride + 64 * nb;
        *reinterpret_cast<uint16_t*>(pw) = (uint16_t)y01;
        *reinterpret_cast<uint16_t*>(pw + kPatchStride) = (uint16_t)(y01 >> 16);
        *reinterpret_cast<uint16_t*>(pw + 2 * kPatchStride) = (uint16_t)y23;
        *reinterpret_cast<uint16_t*>(pw + 3 * kPatchStride) =
            (uint16_t)(y23 >> 16);
      }
      asm volatile("" : "+v"(hc[nb]));
      pinned(8 * r + 6);
      // piece 7: sixteen finished tokens (both channel groups) are read back
      // as 16-byte row chunks (the LDS unit executes a wave's instructions in
      // order: the reads see this wave's writes above, the next run's writes
      // come after them); tokens past the end of the sequence fall outside the
      // descriptor when they are stored
      if (MODE != kChunkSummary && (r & 3) == 3) {
        __builtin_amdgcn_wave_barrier();
        typedef const __attribute__((address_space(3))) u32x4 lds_u32x4;
        y_pending[0] = *reinterpret_cast<lds_u32x4*>(lds3 + patch_r_lane);
        y_pending[1] = *reinterpret_cast<lds_u32x4*>(lds3 + patch_r_lane +
                                                     8 * kPatchStride);
        __builtin_amdgcn_wave_barrier();
        y_pending_row = (uint32_t)(t_blk + 16 * (g >> 1)) * row_bytes;
        if (GELU) {
          g_pending[0] = __builtin_amdgcn_raw_buffer_load_b128(
              rgate, y_lane_bytes + y_pending_row, 0, 0);
          g_pending[1] = __builtin_amdgcn_raw_buffer_load_b128(
              rgate, y_lane_bytes + y_pending_row + 8u * row_bytes, 0, 0);
        }
      }
      pinned(8 * r + 7);
    }
  };

  // ---- prologue -------------------------------------------------------------
#pragma unroll
  for (int nb = 0; nb < kNB; ++nb) {
    const int ch = h * kBW + n0 + 32 * nb + (lane & 31);  // this lane's channel
    bias_x[nb] = -kLog2e * bf16_bits_to_f32(((const uint16_t*)p.b[0])[ch]);
    bias_a[nb] = -kLog2e * bf16_bits_to_f32(((const uint16_t*)p.b[1])[ch]);
    decay[nb] =
        (-8.0f * kLog2e) *
        softplus_precise(bf16_bits_to_f32(((const uint16_t*)p.a_param)[ch]));
    if (MODE == kChunkReplay) {
      // state at the start of this chunk from the summaries of the chunks
      // before it: h <- P[k] h + H[k] (the scan operator of
      // recurrentgemma/jax/scan.py:161-187 over chunks); chunk 0 has P = 0
      // and H = its end state
      float hin = 0.0f;
      const float* sp = p.ws_p + (int64_t)b * p.chunks * W + ch;
      const float* sh = p.ws_h + (int64_t)b * p.chunks * W + ch;
      for (int k = 0; k < chunk; ++k)
        hin = __builtin_fmaf(sp[(int64_t)k * W], hin, sh[(int64_t)k * W]);
      hc[nb] = hin;
    } else if ((MODE == kWholeRow || MODE == kChunkHead) && p.h0) {
      hc[nb] = p.h0[(int64_t)b * W + ch];
    }
  }
  uint64_t m_before, m_cur;
  fetch_seg(tile_begin - 1);
  m_before = start_mask(tile_begin - 1);
  fetch_seg(tile_begin);
  m_cur = start_mask(tile_begin);
  fetch_seg(tile_begin + 1);
  dma_tile(tile_begin, 0);
  dma_tile(tile_begin + 1, 1);
  wait_vmcnt<0>();
  __syncthreads();  // conv table, raw tiles
  {
    const u32x4 t0 = *reinterpret_cast<const u32x4*>(lds_raw + kConvTabOff +
                                                     (tid & 127) * 32);
    const u32x2 t1 = *reinterpret_cast<const u32x2*>(lds_raw + kConvTabOff +
                                                     (tid & 127) * 32 + 16);
    cw10[0] = t0[0]; cw32[0] = t0[1]; cw10[1] = t0[2]; cw32[1] = t0[3];
    cbias[0] = __uint_as_float(t1[0]);
    cbias[1] = __uint_as_float(t1[1]);
  }
  BlockAcc acc0;  // block 0 of the current tile
  {
#pragma unroll
    for (int half = 0; half < 2; ++half)
      conv_rows_with_cuts(0, half, conv_cuts(half, m_cur, m_before));
    lds_barrier();
    Frag a[kARing];
    a_ring_begin(0, 0, a);
    // (spelled out 64 times: left as a loop the compiler keeps the fragment
    // number a run-time value, and then copies accumulators around right
    // behind the matrix instructions, before their results have landed)
#define RG_PROLOGUE_STEP(F) mfma_step(F, 0, 0, a, acc0);
    RG_FRAG_CASES(RG_PROLOGUE_STEP)
#undef RG_PROLOGUE_STEP
    wait_for_matrix_results();
  }

  // ---- tile loop ------------------------------------------------------------
  // Tile `it` has its conv output in buffer BI, block 0's pre-activations in
  // acc0; raw x of tile it+1 is in raw buffer BI^1.
  //   P0  gates + recurrence of block 0; the matrix instructions of block 1;
  //       conv of rows 0-31 of tile it+1; the loads of tile it+2 start
  //   P1  gates + recurrence of block 1; the matrix instructions of block 0
  //       of tile it+1; conv of rows 32-63 of tile it+1
  // with one LDS-only barrier before each.  The buffer index alternates, so
  // the loop body is written for both values and run in turn.
  auto tile_body = [&](auto BI, int it) {
    constexpr int bi = decltype(BI)::value;
    constexpr int bn = bi ^ 1;
    const uint64_t m_next = start_mask(it + 1);
    fetch_seg(it + 2);
    dma_tile(it + 2, bi);  // raw buffer bi held tile `it`: consumed
    BlockAcc acc1;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const uint32_t cuts = conv_cuts(half, m_next, m_cur);
      // half 0: block 1 of this tile (buffer bi); half 1: block 0 of the
      // next tile (buffer bn)
      Frag a[kARing];
      a_ring_begin(half == 0 ? bi : bn, half == 0 ? 1 : 0, a);
      // this thread's raw rows, read a run ahead: the three rows before its
      // own first, then one pair per run.  The rows are convolved as if no
      // document started among them; a half tile where one does is redone
      // with the history cuts after the phase (one branch per phase instead
      // of one per hook).
      uint32_t halo[3], ra = 0, rb = 0, ra_next, rb_next;
#pragma unroll
      for (int r = 0; r < 3; ++r) halo[r] = raw_row(bn, half, r - 3);
      ra_next = raw_row(bn, half, 0);
      rb_next = raw_row(bn, half, 1);
      auto hook = [&](int i) {
        if (half == 0)
          mfma_step(i, bi, 1, a, acc1);
        else
          mfma_step(i, bn, 0, a, acc0);

        // row pair j of this thread's kConvRows / 2: its two raw rows were
        // requested a run earlier, the pair after it is requested now
        const int j = i >> 3;
        if ((i & 7) == 3) {
          if (j == 0) {
            pair_rows(halo[0], halo[1], o_prev);
            pair_rows(halo[1], halo[2], e_prev);
          }
          ra = ra_next;
          rb = rb_next;
          if (2 * j + 3 < kConvRows) {
            ra_next = raw_row(bn, half, 2 * j + 2);
            rb_next = raw_row(bn, half, 2 * j + 3);
          }
        }
        if ((i & 7) == 7 && j < kConvRows / 2) conv_pair(ra, rb, bn, half, j);
      };
      if (half == 0)
        gate_block(it, 0, BI, acc0, m_cur, hook);
      else
        gate_block(it, 1, BI, acc1, m_cur, hook);
      if (__builtin_expect(cuts != 0, 0)) conv_rows_with_cuts(bn, half, cuts);
      wait_for_matrix_results();
      // Between the phases the waves hand each other conv outputs, written by
      // ordinary LDS stores: the barrier waits for those alone.  (The
      // compiler's workgroup fence on LDS also waits for the memory pipe's
      // own LDS writes -- the raw rows of tile it+2 requested at the top of
      // this tile -- which nobody reads before the end of the tile: half a
      // tile is not always enough for them to arrive.)
      if (half == 0)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    // the loads of tile it+2 were issued before this tile's eight y stores
    if (MODE == kChunkSummary)
      wait_vmcnt<0>();
    else
      wait_vmcnt<8>();
    lds_barrier();
    m_cur = m_next;
  };
  // (measurement aid: one workgroup notes how long its tile loop takes on the
  // shader clock and on the constant 100 MHz counter -- their ratio is the
  // clock the GPU runs this kernel at)
  const bool timed = p.timing != nullptr && blockIdx.x == 0 && blockIdx.y == 0;
  uint64_t clk0 = 0, tick0 = 0;
  if (timed) {
    clk0 = __builtin_readcyclecounter();
    tick0 = __builtin_amdgcn_s_memrealtime();
  }
  for (int it = tile_begin; it < tile_end; it += 2) {
    tile_body(std::integral_constant<int, 0>{}, it);
    if (it + 1 < tile_end) tile_body(std::integral_constant<int, 1>{}, it + 1);
  }
  if (timed) {
    const uint64_t clk1 = __builtin_readcyclecounter();
    const uint64_t tick1 = __builtin_amdgcn_s_memrealtime();
    if (tid == 0) {
      p.timing[0] = clk1 - clk0;
      p.timing[1] = tick1 - tick0;
    }
  }
  if (MODE != kChunkSummary) flush_y();  // the last sixteen tokens

  if (MODE == kChunkSummary) {
    // this chunk from a zero state: h_end = prod(a) * h_in + hc
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      const auto sw = __builtin_amdgcn_permlane32_swap(
          __float_as_uint(prod[nb]), __float_as_uint(prod[nb]), false, false);
      const float total = __uint_as_float(sw[0]) * __uint_as_float(sw[1]);
      if (!upper) {
        const int ch = h * kBW + n0 + 32 * nb + (lane & 31);
        const int64_t at = ((int64_t)b * p.chunks + chunk) * W + ch;
        p.ws_p[at] = total;
        p.ws_h[at] = hc[nb];
      }
    }
    return;
  }
  if (MODE == kChunkHead) {
    // whatever came before the row is in hc already: a summary with a zero
    // product makes the carry kernel take hc as the next chunk's start
    if (!upper) {
#pragma unroll
      for (int nb = 0; nb < kNB; ++nb) {
        const int ch = h * kBW + n0 + 32 * nb + (lane & 31);
        const int64_t at = (int64_t)b * p.chunks * W + ch;
        p.ws_p[at] = 0.0f;
        p.ws_h[at] = hc[nb];
      }
    }
    return;
  }
  if (!last_chunk) return;
  if (p.h_last && !upper) {
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
      p.h_last[(int64_t)b * W + h * kBW + n0 + 32 * nb + (lane & 31)] = hc[nb];
  }

  // Masked conv state: rows T-3..T-1 of x, each zeroed if a document starts in
  // a later position of the row; rows before the sequence start are zero.
  if (p.cache_out && tid < 128) {
    const uint32_t c = h * kBW + tid * 2;
    uint16_t* cache = (uint16_t*)p.cache_out + (int64_t)b * 3 * W + c;
    bool later_start = false;
#pragma unroll
    for (int kk = 2; kk >= 0; --kk) {
      const int t = T_len - 3 + kk;
      uint32_t v = 0;
      if (t >= 0 && !later_start)
        v = __builtin_amdgcn_raw_buffer_load_b32(rx, 2u * c,
                                                 (uint32_t)t * row_bytes, 0);
      *reinterpret_cast<uint32_t*>(cache + (int64_t)kk * W) = v;
      if (t >= 0 && is_doc_start(p.segpos, p.seg_kind, (int64_t)b * T_len + t))
        later_start = true;
    }
  }
}

enum PrefillPass { kPassWholeRows = 0, kPassFirst = 1, kPassReplay = 2 };

// blockIdx.x: (row, head); blockIdx.y: which chunk (kPassFirst: chunk 0 with
// its outputs beside the summaries of chunks 1 .. n-2; kPassReplay: chunks
// 1 .. n-1).
// GELU: y is written as y * gelu(gate_branch), the join of the recurrent
// block's two branches, instead of the plain RG-LRU output.
template <int PASS, bool GELU>
__global__ void __launch_bounds__(kThreads) block_prefill_bf16_kernel(
    FusedArgs p) {
  if (PASS == kPassWholeRows) {
    prefill_body<kWholeRow, GELU>(p, 0);
  } else if (PASS == kPassReplay) {
    prefill_body<kChunkReplay, GELU>(p, (int)blockIdx.y + 1);
  } else if (blockIdx.y == 0) {
    prefill_body<kChunkHead, GELU>(p, 0);
  } else {
    prefill_body<kChunkSummary, false>(p, (int)blockIdx.y);
  }
}

template <int PASS, bool GELU>
hipError_t launch_pass_as(const FusedArgs& a, int grid_y, hipStream_t s) {
  static OncePerDevice once;
  hipError_t e = set_max_dynamic_lds(
      once, (const void*)block_prefill_bf16_kernel<PASS, GELU>,
      kPrefillLdsBytes);
  if (e != hipSuccess) return e;
  block_prefill_bf16_kernel<PASS, GELU>
      <<<dim3((unsigned)(a.B * a.H), (unsigned)grid_y), kThreads,
         kPrefillLdsBytes, s>>>(a);
  return hipGetLastError();
}

template <int PASS>
hipError_t launch_pass(const FusedArgs& a, int grid_y, hipStream_t s) {
  if (a.gate_branch) return launch_pass_as<PASS, true>(a, grid_y, s);
  return launch_pass_as<PASS, false>(a, grid_y, s);
}

}  // namespace

// Into how many chunks of whole tiles the sequences of this shape are cut
// (1: not cut).  One workgroup per (row, head) leaves CUs idle below 256
// groups.  Cut into n chunks a row takes two launches of n-1 workgroups, each
// as long as one chunk (every chunk but the first and the last is computed
// twice): 2/n of the uncut time, which pays from n = 3 on.
void prefill_chunk_plan(int B, int H, int T, int* chunks, int* tiles_per_chunk) {
  const int ntiles = (T + kTM - 1) / kTM;
  *chunks = 1;
  *tiles_per_chunk = ntiles;
  const int64_t groups = (int64_t)B * H;
  // (measured at W2560 H10 with the two-wave kernel, us, chunks / whole rows:
  // T384 10-120 pairs even; T512 10 pairs 35/43, 80 pairs 45/49, 120 pairs
  // 54/51; T768 10 pairs 37/61, 120 pairs 69/73; T1024 10 pairs 38/78, 120
  // pairs 89/92; T4096 10 pairs 58/288, 80 pairs 231/298, 120 pairs 307/314)
  if (groups > 128 || ntiles < 8 || (ntiles < 12 && groups > 96)) return;
  int want = (int)(256 / groups) + 1;  // workgroups per launch and row, + 1
  if (want > ntiles / 2) want = ntiles / 2;
  if (want < 3) return;
  const int per = (ntiles + want - 1) / want;
  const int n = (ntiles + per - 1) / per;
  if (n < 3) return;
  *tiles_per_chunk = per;
  *chunks = n;
}

hipError_t launch_block_prefill_bf16(const FusedArgs& a, hipStream_t s) {
  // needs head width 256 and a sequence whose rows fit 31-bit byte offsets
  // (checked by the caller)
  const int64_t blocks = (int64_t)a.B * a.H;
  if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
  // with re-laid-out weights: the form with two waves per SIMD
  // (rg_prefill_teams.hip), a tenth to a fifth faster
  if (a.w_packed) return launch_block_prefill_teams_bf16(a, s);
  if (a.chunks <= 1) return launch_pass<kPassWholeRows>(a, 1, s);
  if (a.chunks < 3 || a.chunks > 65535) return hipErrorInvalidValue;
  hipError_t e = launch_pass<kPassFirst>(a, a.chunks - 1, s);
  if (e != hipSuccess) return e;
  return launch_pass<kPassReplay>(a, a.chunks - 1, s);
}

}  // namespace rg
