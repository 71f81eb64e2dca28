// Whole recurrent core of a prefill in one launch (bf16, 256-wide heads), the
// form with TWO waves per SIMD that take turns at the matrix unit and at the
// vector unit.
//
// One workgroup of eight waves per (sequence row b, head h).  Wave w owns 32
// channels of the head for both gates; its 2 x 256 x 32 weights (128
// accumulation registers) stay resident.  The waves form two teams (0-3 and
// 4-7, one wave of each per SIMD) that walk the sequence in blocks of 32
// tokens, each block in two phases:
//   M  the 32 matrix instructions of the block (pre-activations of both
//      gates), with little else to issue: this wave's share of the conv of
//      the next block, the stores of the block before, the next loads, and
//      at the end a part of the gate arithmetic;
//   G  the rest of the gate arithmetic and the recurrence of the block:
//      vector instructions only.
// Team 1 runs one phase behind team 0, a workgroup barrier after every phase
// keeps it there: while one wave of a SIMD is in G the other is in M, so the
// matrix instructions and their operand reads issue in the gaps of the other
// wave's arithmetic instead of in its own instruction stream.  (With both
// waves of a SIMD in the same phase the kernel is a fifth slower; with the
// wave in M not raised in priority over the one in G, a tenth.)  Same
// arithmetic in the same order as the one-wave-per-SIMD form in rg_prefill.hip:
// the two give bit-identical results.
//
// Whole rows and rows in chunks, with or without the block's GELU join; needs
// the weights re-laid-out (rg_pack_gate_weights): the launcher in
// rg_prefill.hip sends callers without them to the other form.
//
// Replaces the chain Conv1D.forward -> RGLRU.forward of
// recurrentgemma/torch/modules.py:632-643 (layers.py:447-529, 313-365,
// 140-191) for prefill.
#include <type_traits>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;   // head width (K and per-gate N)
constexpr int kBT = 32;    // tokens per block
constexpr int kTM = 64;    // tokens per raw tile (two blocks)
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
// Conv output of a block (the MFMA A operand), bf16, rows padded to 264
// elements; a ring of three blocks (a block is written over two phases, read
// over the three after them, and a new one starts every second phase).
constexpr int kXcStride = 264;
constexpr int kXcRowBytes = kXcStride * 2;
constexpr int kXcBlockBytes = kBT * kXcRowBytes;
constexpr int kXcRing = 3;
// Raw x of a 64-token tile as the memory pipe writes it into LDS: rows -4 ..
// 63 of the tile, 512 bytes each; two tiles.
constexpr int kRawHalo = 4;
constexpr int kRawRows = kTM + kRawHalo;
constexpr int kRawRowBytes = kBW * 2;
constexpr int kRawLoads = kRawRows / 2;
constexpr int kRawLoadsPerWave = (kRawLoads + kWaves - 1) / kWaves;
constexpr int kRawTileBytes = kRawLoadsPerWave * kWaves * 2 * kRawRowBytes;
// Per-wave output patch: 16 tokens x 32 channels in bf16, rows padded to 80
// bytes.
constexpr int kPatchStride = 80;
constexpr int kPatchBytesPerWave = 16 * kPatchStride;

constexpr int kXcOff = 0;
constexpr int kRawOff = kXcOff + kXcRing * kXcBlockBytes;
constexpr int kPatchOff = kRawOff + 2 * kRawTileBytes;
constexpr int kConvTabOff = kPatchOff + kWaves * kPatchBytesPerWave;
constexpr int kTeamsLdsBytes = kConvTabOff + 128 * 32;
static_assert(kTeamsLdsBytes <= 160 * 1024, "LDS of one CU");
// Ring of MFMA A operands read ahead of their matrix instruction.
constexpr int kARing = 4;
// How many of a lane's sixteen tokens have their input-gate sigmoid computed
// at the end of phase M, the rest at the top of phase G (measured at B16 T8192
// W4096: 0 -> 778 us, 8 -> 764 us, 12 -> 779 us a launch), and the same for the
// recurrence gate (any part of it there was slower).
constexpr int kTailXPlain = 8;
constexpr int kTailAPlain = 0;
// ... and with the GELU join in phase G (B16 T8192 W4096: 1057-1062 us a launch
// for 8-16 input-gate and 0-8 recurrence-gate sigmoids here: no difference)
constexpr int kTailXJoined = 16;
constexpr int kTailAJoined = 4;
// Priority of a wave while it issues its matrix instructions (the wave in
// phase G stays at 0 and fills the gaps).
constexpr int kMatrixPriority = 1;

typedef __attribute__((address_space(3))) unsigned char lds_byte;
typedef __attribute__((address_space(3))) uint32_t lds_u32;
typedef __attribute__((address_space(3))) uint16_t lds_u16;
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
typedef __attribute__((address_space(3))) f32x4 lds_f32x4;

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// out[c] = bias[c] + p_old[c] . w10[c] + p_new[c] . w32[c] for two channels
// (v_dot2_f32_bf16; its result may be read by an instruction of another kind
// only three issue slots later).
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

// The wave's 32 weight fragments (fragment F = 2 k-step + gate, four registers
// each) live in the accumulation registers a[4F : 4F+3], written and read by
// inline assembly with the register numbers spelled out.
#define RG_TFRAG_CASES(X)                                                     \
  X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13)   \
  X(14) X(15) X(16) X(17) X(18) X(19) X(20) X(21) X(22) X(23) X(24) X(25)     \
  X(26) X(27) X(28) X(29) X(30) X(31)

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
                 : "a127");                                              \
    break;
    RG_TFRAG_CASES(RG_SET_CASE)
#undef RG_SET_CASE
  }
}
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
    RG_TFRAG_CASES(RG_MFMA_CASE)
#undef RG_MFMA_CASE
  }
}

__device__ __forceinline__ void phase_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}

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

// GELU: y is written as y * gelu(gate_branch), the join of the recurrent
// block's two branches (recurrentgemma/torch/modules.py:627-628, 644),
// instead of the plain RG-LRU output.
template <int MODE, bool GELU>
__device__ __forceinline__ void prefill_teams_body(const FusedArgs& p,
                                                   const int chunk) {
  // how much of the gate arithmetic runs at the end of phase M (with the
  // join, phase G carries 17 more vector slots per element)
  constexpr int kTailX = GELU ? kTailXJoined : kTailXPlain;
  constexpr int kTailA = GELU ? kTailAJoined : kTailAPlain;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  lds_byte* const lds3 = (lds_byte*)lds_raw;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int team = wave >> 2;
  const int in_team = wave & 3;
  const int b = blockIdx.x / p.H;
  const int h = blockIdx.x % p.H;
  const int T_len = p.T;
  const int64_t W = p.W;
  const int ntiles = (T_len + kTM - 1) / kTM;  // of the whole row
  const int tile_begin = MODE == kWholeRow ? 0 : chunk * p.tiles_per_chunk;
  int tile_end = MODE == kWholeRow ? ntiles : tile_begin + p.tiles_per_chunk;
  if (tile_end > ntiles) tile_end = ntiles;
  const bool last_chunk = tile_end == ntiles;
  const bool upper = lane >= 32;
  const int n0 = wave * 32;  // first channel of this wave in the head

  // ---- addressing -----------------------------------------------------------
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

  // Document starts of a tile: lane j looks at token 64*tile + j.
  uint32_t seg_lo = 1, seg_hi = 0;
  auto fetch_seg = [&](int tile) {
    const int t = tile * kTM + lane;
    const uint32_t off = (tile >= 0 && tile < ntiles && t < T_len)
                             ? (uint32_t)t * seg_esize
                             : kBufferOutOfRange;
    seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
    seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
        rseg, seg_is64 ? off + 4u : kBufferOutOfRange, 0, 0);
  };
  auto start_mask = [&](int tile) -> uint64_t {
    uint32_t lo = seg_lo, hi = seg_hi;
    asm volatile("" : "+v"(lo), "+v"(hi));
    const int t = tile * kTM + lane;
    return __ballot(tile >= 0 && tile < ntiles && t < T_len && (lo | hi) == 0u);
  };

  // Raw x of one tile -> LDS by the memory pipe: 34 wave-wide loads of two
  // rows each, five per wave (the six beyond 34 are sent out of range and
  // fill padding rows with zeros).
  const uint32_t dma_lane_off =
      2u * (uint32_t)(h * kBW) + 16u * (uint32_t)(lane & 31);
  auto dma_tile = [&](int tile, int j) {  // this wave's load j of the tile
    lds_byte* const dst = lds3 + kRawOff + (tile & 1) * kRawTileBytes;
    const int t0 = tile * kTM - kRawHalo + (lane >> 5);
    const int i = wave + kWaves * j;
    uint32_t voff = (uint32_t)((t0 + 2 * i) * (int)row_bytes) + dma_lane_off;
    if (kWaves * j + kWaves > kRawLoads)
      voff = i < kRawLoads ? voff : kBufferOutOfRange;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, dst + i * 1024, 16, voff, 0, 0,
                                             0);
  };

  // ---- lane-dependent LDS offsets -------------------------------------------
  // conv: thread -> (channel pair tid % 128, rows 8 rg4 .. 8 rg4 + 7 of a
  // block); team 0 holds row groups 0 and 1, team 1 groups 2 and 3.  Row r of
  // a tile lies at raw row r + kRawHalo; the lane offset points three rows
  // before the group's first.
  const int rg4 = team * 2 + (in_team >> 1);  // 0..3
  const int conv_pair_of_lane = (in_team & 1) * 64 + lane;
  constexpr int kConvRows = 8;
  const uint32_t conv_raw_lane =
      kRawOff + (uint32_t)(rg4 * kConvRows + kRawHalo - 3) * kRawRowBytes +
      conv_pair_of_lane * 4;
  const uint32_t conv_xc_lane =
      kXcOff + (uint32_t)(rg4 * kConvRows) * kXcRowBytes + conv_pair_of_lane * 4;
  // gates: lane -> channel n0 + lane % 32, tokens 4 (lane / 32) + ...
  const uint32_t xc_lane = kXcOff + 4u * (lane >> 5) * kXcRowBytes +
                           2u * (uint32_t)(n0 + (lane & 31));
  // MFMA A operand: lane -> token lane % 32, k offset 8 (lane / 32)
  const uint32_t a_lane =
      kXcOff + (uint32_t)(lane & 31) * kXcRowBytes + 16u * (lane >> 5);
  // output patch of this wave: written as token 4 (lane / 32) + q (+ 8 for
  // odd runs), channel lane % 32; read back as 16-byte row chunks, lane l
  // taking chunk l % 4 of token l / 4
  const uint32_t patch_w_lane = kPatchOff + wave * kPatchBytesPerWave +
                                4u * (lane >> 5) * kPatchStride +
                                2u * (lane & 31);
  const uint32_t patch_r_lane = kPatchOff + wave * kPatchBytesPerWave +
                                (uint32_t)(lane >> 2) * kPatchStride +
                                16u * (lane & 3);
  const uint32_t y_lane_bytes = (uint32_t)(lane >> 2) * row_bytes +
                                2u * (uint32_t)(h * kBW + n0) + 16u * (lane & 3);

  // ---- width-4 conv ---------------------------------------------------------
  uint32_t cw10[2], cw32[2];
  float cbias[2];
  constexpr uint32_t kSelLo = 0x05040100u;
  constexpr uint32_t kSelHi = 0x07060302u;
  auto pair_rows = [&](uint32_t earlier, uint32_t later, uint32_t (&out)[2]) {
    out[0] = __builtin_amdgcn_perm(later, earlier, kSelLo);
    out[1] = __builtin_amdgcn_perm(later, earlier, kSelHi);
  };
  // rows 8 rg4 .. +7 of block kb, raw rows -> conv output, in steps that the
  // caller spreads between its matrix instructions: the eleven raw rows
  // (three of them history), then four row pairs.  The rows are convolved as
  // if no document started among them; where one does they are redone with
  // the history cut (bit i of `cuts`: row i - 3 of these rows starts a
  // document), the same dot products in the same order.
  struct ConvRows {
    uint32_t raw[kConvRows + 3];
    uint32_t e_prev[2], o_prev[2];
    uint32_t xc_at;
  };
  auto conv_load = [&](int kb, ConvRows& cr) {
    const uint32_t raw_at = conv_raw_lane +
                            (uint32_t)((kb >> 1) & 1) * kRawTileBytes +
                            (uint32_t)(kb & 1) * (32 * kRawRowBytes);
    cr.xc_at = conv_xc_lane + (uint32_t)(kb % kXcRing) * kXcBlockBytes;
#pragma unroll
    for (int i = 0; i < kConvRows + 3; ++i)
      cr.raw[i] = *reinterpret_cast<lds_u32*>(lds3 + raw_at + i * kRawRowBytes);
  };
  auto conv_pair = [&](ConvRows& cr, int j) {
    if (j == 0) {
      pair_rows(cr.raw[0], cr.raw[1], cr.o_prev);
      pair_rows(cr.raw[1], cr.raw[2], cr.e_prev);
    }
    uint32_t e[2], o[2];
    pair_rows(cr.raw[3 + 2 * j], cr.raw[4 + 2 * j], e);
    float even[2], odd[2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
      o[c] = __builtin_amdgcn_alignbit(e[c], cr.e_prev[c], 16);
    conv_dot_row_pair(cr.o_prev, o, cr.e_prev, e, cw10, cw32, cbias, even, odd);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      cr.e_prev[c] = e[c];
      cr.o_prev[c] = o[c];
    }
    *reinterpret_cast<lds_u32*>(lds3 + cr.xc_at + (2 * j) * kXcRowBytes) =
        pack_bf16x2(even[0], even[1]);
    *reinterpret_cast<lds_u32*>(lds3 + cr.xc_at + (2 * j + 1) * kXcRowBytes) =
        pack_bf16x2(odd[0], odd[1]);
  };
  auto conv_with_cuts = [&](const ConvRows& cr, uint32_t cuts) {
    uint32_t r_prev = 0, p1[2] = {0, 0}, p2[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < kConvRows + 3; ++i) {
      const uint32_t r = cr.raw[i];
      if ((cuts >> i) & 1u) {
        r_prev = 0;
        p1[0] = p1[1] = p2[0] = p2[1] = 0;
      }
      uint32_t pt[2];
      pair_rows(r_prev, r, pt);
      if (i >= 3) {
        float o[2];
        conv_dot_row(p2, pt, cw10, cw32, cbias, o);
        *reinterpret_cast<lds_u32*>(lds3 + cr.xc_at + (i - 3) * kXcRowBytes) =
            pack_bf16x2(o[0], o[1]);
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
  // block kb: m_tile is the start mask of the block's tile, m_before that of
  // the tile before it.
  auto conv_cuts = [&](int kb, uint64_t m_tile, uint64_t m_before) -> uint32_t {
    const uint64_t lo = ((m_tile << 3) | (m_before >> 61)) >> (rg4 * kConvRows);
    const uint64_t hi = m_tile >> (29 + rg4 * kConvRows);
    const uint64_t bits = (kb & 1) ? hi : lo;
    return (uint32_t)bits & ((1u << (kConvRows + 3)) - 1u);
  };

  // ---- state ------------------------------------------------------------------
  const int ch = h * kBW + n0 + (lane & 31);  // this lane's channel
  const float bias_x = -kLog2e * bf16_bits_to_f32(((const uint16_t*)p.b[0])[ch]);
  const float bias_a = -kLog2e * bf16_bits_to_f32(((const uint16_t*)p.b[1])[ch]);
  const float decay =
      (-8.0f * kLog2e) *
      softplus_precise(bf16_bits_to_f32(((const uint16_t*)p.a_param)[ch]));
  float hc = 0.0f;    // carried state of this lane's channel
  float prod = 1.0f;  // kChunkSummary: product of a over this lane's tokens
  if (MODE == kChunkReplay) {
    // state at the start of this chunk from the summaries of the chunks
    // before it: h <- P[k] h + H[k] (the scan operator of
    // recurrentgemma/jax/scan.py:161-187 over chunks); chunk 0 has P = 0 and
    // H = its end state
    const float* sp = p.ws_p + (int64_t)b * p.chunks * W + ch;
    const float* sh = p.ws_h + (int64_t)b * p.chunks * W + ch;
    for (int k = 0; k < chunk; ++k)
      hc = __builtin_fmaf(sp[(int64_t)k * W], hc, sh[(int64_t)k * W]);
  } else if ((MODE == kWholeRow || MODE == kChunkHead) && p.h0) {
    hc = p.h0[(int64_t)b * W + ch];
  }
  f32x16 acc_x, acc_a;
  // conv outputs of the block in phase G, this lane's tokens, as floats
  uint32_t xr[16];
  u32x4 y_pending[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
  uint32_t y_pending_row = kBufferOutOfRange;
  // start masks of the tile before the current G block's, of its own, and of
  // the next
  uint64_t m_prev, m_cur, m_next;

  // gate arithmetic on accumulator elements [i0, i1), in place: the input
  // gate's sigmoid; a = exp2(sigmoid(recurrence gate) * decay)
  auto gate_x = [&](int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
      acc_x[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_x[i], -kLog2e, bias_x));
#pragma unroll
    for (int i = i0; i < i1; ++i)
      acc_x[i] = __builtin_amdgcn_rcpf(1.0f + acc_x[i]);
  };
  auto gate_a = [&](int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
      acc_a[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(acc_a[i], -kLog2e, bias_a));
#pragma unroll
    for (int i = i0; i < i1; ++i)
      acc_a[i] = __builtin_amdgcn_rcpf(1.0f + acc_a[i]);
#pragma unroll
    for (int i = i0; i < i1; ++i)
      acc_a[i] = __builtin_amdgcn_exp2f(acc_a[i] * decay);
  };
  // ---- phase M of block kb ----------------------------------------------------
  auto phase_m = [&](int kb, auto ODD) {
    constexpr bool odd = decltype(ODD)::value;  // kb % 2, at compile time
    // team 1 reads raw rows that it asked for itself two phases ago (team 0
    // waits for its own at the top of phase G)
    if (!odd && team == 1) wait_vmcnt<0>();
    const uint32_t a_at = a_lane + (uint32_t)(kb % kXcRing) * kXcBlockBytes;
    auto a_read = [&](int ks) {
      return *reinterpret_cast<lds_f32x4*>(lds3 + a_at + ks * 32);
    };
    f32x4 a[kARing];
#pragma unroll
    for (int k = 0; k < kARing - 1; ++k) a[k] = a_read(k);
    // the tokens of the block before leave now
    buffer_store_16(y_pending[0], ry, y_lane_bytes, y_pending_row);
    buffer_store_16(y_pending[1], ry, y_lane_bytes,
                    y_pending_row + 16u * row_bytes);
    const uint32_t cuts = odd ? conv_cuts(kb + 1, m_next, m_cur)
                              : conv_cuts(kb + 1, m_cur, m_prev);
    ConvRows cr;
    // the block's conv outputs for the gate arithmetic, this lane's sixteen
    // tokens: each into the high half of a zeroed register -- the bf16 value
    // as a float without a shift
    const uint32_t x_at = xc_lane + (uint32_t)(kb % kXcRing) * kXcBlockBytes;
#define RG_XR(i)                                                            \
  asm volatile("v_mov_b32 %0, 0\n\tds_read_u16_d16_hi %0, %1 offset:%2"      \
               : "=&v"(xr[i])                                                \
               : "v"(x_at), "n"((8 * ((i) >> 2) + ((i) & 3)) * kXcRowBytes));
    __builtin_amdgcn_s_setprio(kMatrixPriority);
    // The 32 matrix instructions of the block, with this wave's conv rows of
    // the next block and (every second block) the loads of the tile after the
    // next between them.
#pragma unroll
    for (int ks = 0; ks < 16; ++ks) {
      if (ks + kARing - 1 < 16)
        a[(ks + kARing - 1) % kARing] = a_read(ks + kARing - 1);
      mfma_weight_frag(2 * ks, ks == 0, a[ks % kARing], acc_x);
      mfma_weight_frag(2 * ks + 1, ks == 0, a[ks % kARing], acc_a);
      if (ks == 0) conv_load(kb + 1, cr);
      if (ks >= 3 && ks % 3 == 0 && ks / 3 - 1 < kConvRows / 2)
        conv_pair(cr, ks / 3 - 1);
      // (late in the loop, when the conv rows have left their registers)
      if (ks == 13) { RG_XR(0) RG_XR(1) RG_XR(2) RG_XR(3) RG_XR(4) }
      if (ks == 14) { RG_XR(5) RG_XR(6) RG_XR(7) RG_XR(8) RG_XR(9) RG_XR(10) }
      if (ks == 15) { RG_XR(11) RG_XR(12) RG_XR(13) RG_XR(14) RG_XR(15) }
      if (odd) {
        if (ks == 4) dma_tile((kb >> 1) + 2, 0);
        if (ks == 7) dma_tile((kb >> 1) + 2, 1);
        if (ks == 10) dma_tile((kb >> 1) + 2, 2);
        if (ks == 13) dma_tile((kb >> 1) + 2, 3);
        if (ks == 14) dma_tile((kb >> 1) + 2, 4);
        if (ks == 15) fetch_seg((kb >> 1) + 2);
      }
    }
#undef RG_XR
    __builtin_amdgcn_s_setprio(0);
    if (__builtin_expect(cuts != 0, 0)) conv_with_cuts(cr, cuts);
    // the last matrix results land (19 issue slots); every reader of the
    // accumulators is ordered behind this statement
    asm volatile("s_nop 15\n\ts_nop 7" : "+v"(acc_x), "+v"(acc_a));
    // part of the gate arithmetic here, the rest in phase G: split so that
    // the two phases take about as long
    gate_x(0, kTailX);
    gate_a(0, kTailA);
    // (computed here, before the barrier: nothing else orders them)
    asm volatile("" : "+v"(acc_x), "+v"(acc_a));
  };

  // ---- phase G of block kb ----------------------------------------------------
  // The MFMA result gives a lane one channel (lane % 32) and 16 tokens in runs
  // of four that alternate between the lane halves: run g of lanes 0-31 holds
  // tokens 8g..8g+3, of lanes 32-63 tokens 8g+4..8g+7.  Per run the recurrence
  // is walked twice: from the carried state (right for lanes 0-31, whose end
  // value goes to lanes 32-63 with one permlane32_swap), then again from each
  // half's own incoming state.
  auto phase_g_as = [&](int kb, auto GENERAL) {
    constexpr bool general = decltype(GENERAL)::value;
    const int t_blk = kb * kBT;
    u32x4 g_pending[2];
    if (GELU) {
      // the gate-branch values at the positions of this block's outputs:
      // asked for now, used at the end of the phase
      g_pending[0] = __builtin_amdgcn_raw_buffer_load_b128(
          rgate, y_lane_bytes + (uint32_t)t_blk * row_bytes, 0, 0);
      g_pending[1] = __builtin_amdgcn_raw_buffer_load_b128(
          rgate, y_lane_bytes + (uint32_t)(t_blk + 16) * row_bytes, 0, 0);
    }
    gate_x(kTailX, 16);
    gate_a(kTailA, 16);
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float av[4], xn[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        av[q] = acc_a[4 * g + q];
        xn[q] = __uint_as_float(xr[4 * g + q]) * acc_x[4 * g + q];
      }
      if (general) {
        // document start: a = 0; past the end of the sequence: a = 1, no
        // input.  The input scale sqrt(1 - a^2) comes out as 1 at a start.
        const int half_rows = upper ? 4 : 0;
        const int row = (kb & 1) * 32 + 8 * g + half_rows;
        const uint32_t starts = (uint32_t)(m_cur >> row) & 0xfu;
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
      float e1 = hc;
#pragma unroll
      for (int q = 0; q < 4; ++q) e1 = __builtin_fmaf(av[q], e1, xn[q]);
      float hh;
      {
        const auto sw = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(hc), __float_as_uint(e1), false, false);
        hh = __uint_as_float(sw[0]);  // lanes 0-31: carry, 32-63: e1 of 0-31
      }
      float hv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        hh = __builtin_fmaf(av[q], hh, xn[q]);
        hv[q] = hh;
      }
      {
        const auto sw = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(hh), __float_as_uint(hh), false, false);
        hc = __uint_as_float(sw[1]);  // all lanes: end value of 32-63
      }
      if (MODE == kChunkSummary) {
#pragma unroll
        for (int q = 0; q < 4; ++q) prod *= av[q];
        continue;
      }
      const uint32_t y01 = pack_bf16x2(hv[0], hv[1]);
      const uint32_t y23 = pack_bf16x2(hv[2], hv[3]);
      // the four tokens into the wave's patch: the low halves of the packed
      // pairs, and the high halves as they are
      const uint32_t pw = patch_w_lane + (8 * (g & 1)) * kPatchStride;
      asm volatile(
          "ds_write_b16 %0, %1\n\t"
          "ds_write_b16_d16_hi %0, %1 offset:%3\n\t"
          "ds_write_b16 %0, %2 offset:%4\n\t"
          "ds_write_b16_d16_hi %0, %2 offset:%5"
          :
          : "v"(pw), "v"(y01), "v"(y23), "n"(kPatchStride),
            "n"(2 * kPatchStride), "n"(3 * kPatchStride)
          : "memory");
      if (g & 1) {
        // sixteen finished tokens are read back as 16-byte row chunks (the
        // LDS unit executes a wave's instructions in order)
        y_pending[g >> 1] = *reinterpret_cast<lds_u32x4*>(lds3 + patch_r_lane);
        asm volatile("" ::: "memory");
      }
    }
    if (GELU) {
      // y * gelu(gate branch), each factor a bf16 tensor as in the reference:
      // the arithmetic and roundings of the stand-alone gelu_mul pass
#pragma unroll
      for (int j = 0; j < 2; ++j)
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
    y_pending_row = (uint32_t)t_blk * row_bytes;
  };
  auto phase_g = [&](int kb, auto ODD) {
    constexpr bool odd = decltype(ODD)::value;
    if (!odd && team == 0) wait_vmcnt<2>();
    if (__builtin_expect(m_cur != 0 || (kb + 1) * kBT > T_len, 0))
      phase_g_as(kb, std::true_type{});
    else
      phase_g_as(kb, std::false_type{});
    if (odd) {
      m_prev = m_cur;
      m_cur = m_next;
      m_next = start_mask((kb >> 1) + 2);
    }
  };

  // ---- prologue -------------------------------------------------------------
  // Everything the first phases need is requested before anything waits: the
  // raw rows of the first two tiles, the positions of three tiles, then the
  // weights and the conv taps (one memory round trip after the other would
  // cost a launch of short chunks a tenth of its time).
#pragma unroll
  for (int j = 0; j < kRawLoadsPerWave; ++j) {
    dma_tile(tile_begin, j);
    dma_tile(tile_begin + 1, j);
  }
  uint32_t first_lo[3], first_hi[3];
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    fetch_seg(tile_begin - 1 + k);
    first_lo[k] = seg_lo;
    first_hi[k] = seg_hi;
  }
  // ---- this wave's weights: 32 channels of the head, both gates ------------
  {
    const f32x4* src = reinterpret_cast<const f32x4*>(p.w_packed) +
                       ((int64_t)(h * 8 + wave) * 16 * 2) * 64 + lane;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      f32x4 w[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) w[i] = src[(16 * half + i) * 64];
      asm volatile("" ::"v"(w[0]), "v"(w[1]), "v"(w[2]), "v"(w[3]), "v"(w[4]),
                   "v"(w[5]), "v"(w[6]), "v"(w[7]), "v"(w[8]), "v"(w[9]),
                   "v"(w[10]), "v"(w[11]), "v"(w[12]), "v"(w[13]), "v"(w[14]),
                   "v"(w[15]));
#pragma unroll
      for (int i = 0; i < 16; ++i) set_weight_frag(16 * half + i, w[i]);
    }
  }

  // ---- conv table ---------------------------------------------------------
  if (tid < 128) {
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

  seg_lo = first_lo[0]; seg_hi = first_hi[0];
  m_prev = start_mask(tile_begin - 1);
  seg_lo = first_lo[1]; seg_hi = first_hi[1];
  m_cur = start_mask(tile_begin);
  seg_lo = first_lo[2]; seg_hi = first_hi[2];
  m_next = start_mask(tile_begin + 1);
  wait_vmcnt<0>();
  __syncthreads();  // conv table, raw tiles
  {
    const u32x4 t0 = *reinterpret_cast<const u32x4*>(lds_raw + kConvTabOff +
                                                     conv_pair_of_lane * 32);
    const u32x2 t1 = *reinterpret_cast<const u32x2*>(lds_raw + kConvTabOff +
                                                     conv_pair_of_lane * 32 + 16);
    cw10[0] = t0[0]; cw32[0] = t0[1]; cw10[1] = t0[2]; cw32[1] = t0[3];
    cbias[0] = __uint_as_float(t1[0]);
    cbias[1] = __uint_as_float(t1[1]);
  }
  {
    ConvRows cr;
    conv_load(2 * tile_begin, cr);
    conv_with_cuts(cr, conv_cuts(2 * tile_begin, m_cur, m_prev));
  }
  phase_barrier();

  const bool timed = p.timing != nullptr && blockIdx.x == 0 && blockIdx.y == 0;
  uint64_t clk0 = 0, tick0 = 0;
  if (timed) {
    clk0 = __builtin_readcyclecounter();
    tick0 = __builtin_amdgcn_s_memrealtime();
  }
  // team 1 runs one phase behind team 0
  if (team == 1) phase_barrier();
  // (whole tiles: a block past the end of the sequence is all identity, and
  // its stores fall outside the descriptor)
  for (int kb = 2 * tile_begin; kb < 2 * tile_end; kb += 2) {
    phase_m(kb, std::false_type{});
    phase_barrier();
    phase_g(kb, std::false_type{});
    phase_barrier();
    phase_m(kb + 1, std::true_type{});
    phase_barrier();
    phase_g(kb + 1, std::true_type{});
    phase_barrier();
  }
  if (team == 0) phase_barrier();
  if (timed) {
    const uint64_t clk1 = __builtin_readcyclecounter();
    const uint64_t tick1 = __builtin_amdgcn_s_memrealtime();
    if (tid == 0) {
      p.timing[0] = clk1 - clk0;
      p.timing[1] = tick1 - tick0;
    }
  }
  buffer_store_16(y_pending[0], ry, y_lane_bytes, y_pending_row);
  buffer_store_16(y_pending[1], ry, y_lane_bytes, y_pending_row + 16u * row_bytes);

  if (MODE == kChunkSummary) {
    // this chunk from a zero state: h_end = prod(a) * h_in + hc
    const auto sw = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(prod), __float_as_uint(prod), false, false);
    const float total = __uint_as_float(sw[0]) * __uint_as_float(sw[1]);
    if (!upper) {
      const int64_t at = ((int64_t)b * p.chunks + chunk) * W + ch;
      p.ws_p[at] = total;
      p.ws_h[at] = hc;
    }
    return;
  }
  if (MODE == kChunkHead) {
    // whatever came before the row is in hc already: a summary with a zero
    // product makes the replay take hc as the next chunk's start
    if (!upper) {
      const int64_t at = (int64_t)b * p.chunks * W + ch;
      p.ws_p[at] = 0.0f;
      p.ws_h[at] = hc;
    }
    return;
  }
  if (!last_chunk) return;
  if (p.h_last && !upper) p.h_last[(int64_t)b * W + ch] = hc;

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
template <int PASS, bool GELU>
__global__ void __launch_bounds__(kThreads) block_prefill_teams_bf16_kernel(
    FusedArgs p) {
  if (PASS == kPassWholeRows) {
    prefill_teams_body<kWholeRow, GELU>(p, 0);
  } else if (PASS == kPassReplay) {
    prefill_teams_body<kChunkReplay, GELU>(p, (int)blockIdx.y + 1);
  } else if (blockIdx.y == 0) {
    prefill_teams_body<kChunkHead, GELU>(p, 0);
  } else {
    prefill_teams_body<kChunkSummary, false>(p, (int)blockIdx.y);
  }
}

template <int PASS, bool GELU>
hipError_t launch_teams_pass_as(const FusedArgs& a, int grid_y, hipStream_t s) {
  static OncePerDevice once;
  hipError_t e = set_max_dynamic_lds(
      once, (const void*)block_prefill_teams_bf16_kernel<PASS, GELU>,
      kTeamsLdsBytes);
  if (e != hipSuccess) return e;
  block_prefill_teams_bf16_kernel<PASS, GELU>
      <<<dim3((unsigned)(a.B * a.H), (unsigned)grid_y), kThreads, kTeamsLdsBytes,
         s>>>(a);
  return hipGetLastError();
}

template <int PASS>
hipError_t launch_teams_pass(const FusedArgs& a, int grid_y, hipStream_t s) {
  if (a.gate_branch) return launch_teams_pass_as<PASS, true>(a, grid_y, s);
  return launch_teams_pass_as<PASS, false>(a, grid_y, s);
}

}  // namespace

hipError_t launch_block_prefill_teams_bf16(const FusedArgs& a, hipStream_t s) {
  const int64_t blocks = (int64_t)a.B * a.H;
  if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
  if (!a.w_packed) return hipErrorInvalidValue;
  if (a.chunks <= 1) return launch_teams_pass<kPassWholeRows>(a, 1, s);
  if (a.chunks < 3 || a.chunks > 65535) return hipErrorInvalidValue;
  hipError_t e = launch_teams_pass<kPassFirst>(a, a.chunks - 1, s);
  if (e != hipSuccess) return e;
  return launch_teams_pass<kPassReplay>(a, a.chunks - 1, s);
}

}  // namespace rg
