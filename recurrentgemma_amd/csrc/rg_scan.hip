// Fused Conv1D(width 4) + RG-LRU gating + linear recurrence for gfx950.
//
// Work decomposition.  Lanes map to channels (CH adjacent channels per lane),
// so every global access of a wave is one contiguous row segment.  A workgroup
// owns one batch row and one slab of 64*CH channels and walks the sequence in
// steps of nw*KL tokens (nw = waves in the group).  Inside a step, wave v
// takes the KL consecutive tokens [v*KL, (v+1)*KL):
//
//   phase 1  each wave reads x / gate pre-activations for its tokens, applies
//            the conv, the sigmoids, a = exp(-8 softplus(L) sigmoid(ga)) and
//            the sqrt(1-a^2) input scale, keeps the (a_t, xn_t) pairs in
//            registers and reduces them with the scan operator
//            (a2,b2) o (a1,b1) = (a2 a1, a2 b1 + b2) to one pair (P, Hloc);
//   exchange the nw pairs go through LDS; wave v folds the pairs of waves
//            0..v-1 onto the carry of the previous step to get its own
//            incoming state;
//   phase 2  each wave replays h = a_t h + xn_t from that state and writes y.
//
// The carry into the next step is the last wave's final h.  A document start
// (segment_pos == 0) sets a = 0 and the input scale to 1 and cuts the conv
// history, which is exactly the reference's masking rule; steps that contain
// one are recomputed on a separate, rarely taken path so that the common path
// is straight-line code.  Tokens past the end of the sequence are computed on
// a re-read of the last valid row; their stores are dropped and their results
// can only reach state that nothing reads any more.
//
// The kernel is bound by the memory system, not by arithmetic: on MI355X the
// achieved rate depends on the bytes per lane and the step length (8 bytes per
// lane and short steps stream best) and on marking the streamed rows
// non-temporal.
//
// Addressing.  All row traffic goes through buffer instructions: a scalar
// resource descriptor based at the wave's first token of the step, a per-lane
// byte offset that never changes, and a scalar row offset.  No per-access
// vector address arithmetic is needed.  The hardware range check covers the
// scalar offset as well, which is used twice: lanes past the last channel
// carry a huge lane offset and rows past the end of the sequence a huge scalar
// offset, so their loads return 0 and their stores are dropped.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kMaxNW = 16;  // waves per workgroup
constexpr uint32_t kOutOfRange = 0x80000000u;
// cache policy of the streamed rows: non-temporal (read or written once)
constexpr int kStream = 2;


// Buffer access of CH adjacent channels.  Raw keeps bf16 values packed until
// they are used.
template <typename T, int CH>
struct Buf;
template <>
struct Buf<uint16_t, 4> {
  typedef u32x2 Raw;
  template <int AUX>
  __device__ static Raw load(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                             uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, AUX);
  }
  __device__ static void unpack(Raw u, float (&v)[4]) {
    v[0] = __uint_as_float(u.x << 16);
    v[1] = __uint_as_float(u.x & 0xffff0000u);
    v[2] = __uint_as_float(u.y << 16);
    v[3] = __uint_as_float(u.y & 0xffff0000u);
  }
  template <int AUX>
  __device__ static void store(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                               uint32_t soff, const float (&v)[4]) {
    u32x2 u = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
    __builtin_amdgcn_raw_buffer_store_b64(u, r, voff, soff, AUX);
  }
  // round to bf16, two channels per convert
  __device__ static void round(float (&v)[4]) {
    u32x2 u = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
    unpack(u, v);
  }
};
template <>
struct Buf<uint16_t, 2> {
  typedef uint32_t Raw;
  template <int AUX>
  __device__ static Raw load(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                             uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, AUX);
  }
  __device__ static void unpack(Raw u, float (&v)[2]) {
    v[0] = __uint_as_float(u << 16);
    v[1] = __uint_as_float(u & 0xffff0000u);
  }
  template <int AUX>
  __device__ static void store(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                               uint32_t soff, const float (&v)[2]) {
    __builtin_amdgcn_raw_buffer_store_b32(pack_bf16x2(v[0], v[1]), r, voff,
                                          soff, AUX);
  }
  __device__ static void round(float (&v)[2]) {
    unpack(pack_bf16x2(v[0], v[1]), v);
  }
};
template <>
struct Buf<uint16_t, 1> {
  typedef uint16_t Raw;
  template <int AUX>
  __device__ static Raw load(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                             uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, AUX);
  }
  __device__ static void unpack(Raw u, float (&v)[1]) {
    v[0] = bf16_bits_to_f32(u);
  }
  template <int AUX>
  __device__ static void store(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                               uint32_t soff, const float (&v)[1]) {
    __builtin_amdgcn_raw_buffer_store_b16(f32_to_bf16_bits(v[0]), r, voff, soff,
                                          AUX);
  }
  __device__ static void round(float (&v)[1]) { v[0] = round_to_bf16(v[0]); }
};
template <>
struct Buf<float, 2> {
  typedef u32x2 Raw;
  template <int AUX>
  __device__ static Raw load(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                             uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, AUX);
  }
  __device__ static void unpack(Raw u, float (&v)[2]) {
    v[0] = __uint_as_float(u.x);
    v[1] = __uint_as_float(u.y);
  }
  template <int AUX>
  __device__ static void store(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                               uint32_t soff, const float (&v)[2]) {
    u32x2 u = {__float_as_uint(v[0]), __float_as_uint(v[1])};
    __builtin_amdgcn_raw_buffer_store_b64(u, r, voff, soff, AUX);
  }
  __device__ static void round(float (&)[2]) {}
};
template <>
struct Buf<float, 1> {
  typedef uint32_t Raw;
  template <int AUX>
  __device__ static Raw load(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                             uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, AUX);
  }
  __device__ static void unpack(Raw u, float (&v)[1]) {
    v[0] = __uint_as_float(u);
  }
  template <int AUX>
  __device__ static void store(__amdgpu_buffer_rsrc_t r, uint32_t voff,
                               uint32_t soff, const float (&v)[1]) {
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v[0]), r, voff, soff,
                                          AUX);
  }
  __device__ static void round(float (&)[1]) {}
};

template <int CH>
struct ChanConst {
  // float32: the four taps as floats.  bf16: the taps stay packed in pairs,
  // w10 = (w0, w1) and w32 = (w2, w3), the operands of the two-element dot
  // product (w0..w3 unused and optimised away)
  float w0[CH], w1[CH], w2[CH], w3[CH], bias[CH];
  uint32_t w10[CH], w32[CH];
  float decay[CH];  // FAST: -8 softplus(L) log2(e);  precise: softplus(L)
};

// ---- width-4 conv on packed bf16 rows (conv4_dot of rg_common.h) ----------
// A row of a lane is CH bf16 channels in CH/2 registers; per channel the rows
// are paired in time, P_t = (x[t-1], x[t]).
template <int CH>
struct PairRow {
  uint32_t p[CH];  // per channel: (x[t-1], x[t])
};
__device__ __forceinline__ PairRow<4> pair_rows(u32x2 earlier, u32x2 later) {
  PairRow<4> r;
  pair_up(earlier.x, later.x, r.p[0], r.p[1]);
  pair_up(earlier.y, later.y, r.p[2], r.p[3]);
  return r;
}
__device__ __forceinline__ PairRow<2> pair_rows(uint32_t earlier,
                                                uint32_t later) {
  PairRow<2> r;
  pair_up(earlier, later, r.p[0], r.p[1]);
  return r;
}
__device__ __forceinline__ void conv_dot(const PairRow<2>& older,
                                         const PairRow<2>& newer,
                                         const ChanConst<2>& k,
                                         float (&out)[2]) {
  conv4_dot_x2(older.p, newer.p, k.w10, k.w32, k.bias, out);
}
__device__ __forceinline__ void conv_dot(const PairRow<4>& older,
                                         const PairRow<4>& newer,
                                         const ChanConst<4>& k,
                                         float (&out)[4]) {
  conv4_dot_x4(older.p, newer.p, k.w10, k.w32, k.bias, out);
}
// Whether this instantiation convolves packed rows with dot products.
template <typename T, int CH, bool CONV>
constexpr bool kPackedConv = CONV && sizeof(T) == 2 && (CH == 2 || CH == 4);


// Where a wave's rows for one step live: descriptors based at the wave's first
// token (clamped into the sequence) and the scalar row offset of each token,
// with tokens past the end of the sequence redirected to the last valid row.
template <int KL>
struct StepAddr {
  __amdgpu_buffer_rsrc_t rx, rgx, rga, rhalo;
  int first;  // clamped first token
  int last;   // last token of the sequence (T-1)
  uint32_t row_bytes;
  bool has_halo;  // three look-back rows exist (first token >= 3)
  __device__ __forceinline__ uint32_t soff(int i) const {
    const int t = first + i < last ? first + i : last;
    return (uint32_t)(t - first) * row_bytes;
  }
};

template <int KL>
__device__ __forceinline__ StepAddr<KL> step_addr(const char* xrow,
                                                  const char* gxrow,
                                                  const char* garow, int t0,
                                                  int T_len,
                                                  uint32_t row_bytes) {
  StepAddr<KL> a;
  a.last = T_len - 1;
  a.first = t0 < a.last ? t0 : a.last;
  a.row_bytes = row_bytes;
  const int64_t tok_bytes = (int64_t)a.first * row_bytes;
  const uint32_t span_bytes = (uint32_t)KL * row_bytes;
  a.rx = make_rsrc(xrow + tok_bytes, span_bytes);
  a.rgx = make_rsrc(gxrow + tok_bytes, span_bytes);
  a.rga = make_rsrc(garow + tok_bytes, span_bytes);
  a.has_halo = a.first >= 3;
  a.rhalo =
      make_rsrc(xrow + tok_bytes - (a.has_halo ? 3 : 0) * (int64_t)row_bytes,
                3 * row_bytes);
  return a;
}

// Raw inputs of one wave for one step, as loaded (bf16 values still packed).
template <typename T, int CH, int KL>
struct Tile {
  typename Buf<T, CH>::Raw x[KL], gx[KL], ga[KL], halo[3];
};

template <typename T, int CH, int KL, bool PLAIN>
__device__ __forceinline__ void load_token(Tile<T, CH, KL>& tl, int i,
                                           const StepAddr<KL>& a,
                                           uint32_t voff) {
  using B = Buf<T, CH>;
  const uint32_t so = a.soff(i);
  tl.x[i] = B::template load<kStream>(a.rx, voff, so);
  if (!PLAIN) tl.gx[i] = B::template load<kStream>(a.rgx, voff, so);
  tl.ga[i] = B::template load<kStream>(a.rga, voff, so);
}

template <typename T, int CH, int KL, bool CONV>
__device__ __forceinline__ void load_halo(Tile<T, CH, KL>& tl,
                                          const StepAddr<KL>& a,
                                          uint32_t voff) {
  using B = Buf<T, CH>;
  if (CONV && a.has_halo) {
#pragma unroll
    for (int s = 0; s < 3; ++s)  // halo[s] = x[first-1-s]
      tl.halo[s] =
          B::template load<0>(a.rhalo, voff, (uint32_t)(2 - s) * a.row_bytes);
  } else {
#pragma unroll
    for (int s = 0; s < 3; ++s) tl.halo[s] = typename B::Raw{};
  }
}

// Raw segment value this lane looks at for the step starting at token t0
// (token t0-3+lane).  One member per encoding, each written by its own guarded
// load and defaulting to "no document start": the three are never merged into
// one register, so issuing the load does not wait for anything.
struct SegRaw {
  int64_t v64;
  int32_t v32;
  uint32_t v8;
};

template <int KL, bool CONV>
__device__ __forceinline__ SegRaw load_seg(const ScanArgs& p, int64_t row0,
                                           int t0, int T_len, int lane) {
  const int t = t0 - 3 + lane;
  const bool look =
      lane < KL + 3 && (CONV || lane >= 3) && t >= 0 && t < T_len;
  SegRaw r;
  r.v64 = 1;
  r.v32 = 1;
  r.v8 = 0;
  if (look && p.seg_kind == kSegI64)
    r.v64 = reinterpret_cast<const int64_t*>(p.segpos)[row0 + t];
  if (look && p.seg_kind == kSegI32)
    r.v32 = reinterpret_cast<const int32_t*>(p.segpos)[row0 + t];
  if (look && p.seg_kind == kSegMaskU8)
    r.v8 = reinterpret_cast<const uint8_t*>(p.segpos)[row0 + t];
  return r;
}

// bit j = token t0-3+j starts a document.  The empty asm pins the comparison
// to the call site: without it the compiler tests the value right behind its
// load, i.e. waits for that load before the rows of the step are even
// requested.
__device__ __forceinline__ uint32_t doc_starts(SegRaw seg) {
  uint32_t lo = (uint32_t)seg.v64, hi = (uint32_t)((uint64_t)seg.v64 >> 32);
  asm volatile("" : "+v"(lo), "+v"(hi), "+v"(seg.v32), "+v"(seg.v8));
  const bool st = ((lo | hi) == 0u) | (seg.v32 == 0) | (seg.v8 != 0u);
  return (uint32_t)__ballot(st);
}

// Keeps a rarely taken, wave-uniform block a real branch (the compiler would
// otherwise turn it into per-lane selects that every token pays for).
#define RG_RARE_BLOCK() asm volatile("" ::: "memory")

// Gating arithmetic of one token: (xc, gate pre-activations) -> (a, xn).
template <int CH, bool FAST, bool PLAIN>
__device__ __forceinline__ void gate_math(const float (&xc)[CH],
                                          const float (&gxv)[CH],
                                          const float (&gav)[CH],
                                          const float (&decay)[CH], bool start,
                                          float (&a)[CH], float (&xn)[CH]) {
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    float mult, gate_x;
    if (PLAIN) {
      a[ch] = gav[ch];
      mult = 1.0f;
      gate_x = 1.0f;
    } else if (FAST) {
      gate_x = sigmoid_fast(gxv[ch]);
      const float gate_a = sigmoid_fast(gav[ch]);
      a[ch] = __builtin_amdgcn_exp2f(gate_a * decay[ch]);
      mult = __builtin_amdgcn_sqrtf(__builtin_fmaf(-a[ch], a[ch], 1.0f));
    } else {
      gate_x = sigmoid_precise(gxv[ch]);
      const float gate_a = sigmoid_precise(gav[ch]);
      const float log_a = (-8.0f * gate_a) * decay[ch];
      a[ch] = expf(log_a);
      mult = sqrtf(1.0f - expf(2.0f * log_a));
    }
    if (start) {  // only the slow path passes a non-constant `start`
      a[ch] = 0.0f;
      mult = 1.0f;
    }
    xn[ch] = PLAIN ? xc[ch] : (xc[ch] * gate_x) * mult;
  }
}

// Phase 1, hot path: straight-line code for a step without a document start
// among the wave's tokens or its three look-back tokens.  As soon as a token's
// raw inputs have been unpacked, the same registers are reloaded with that
// token's row of the NEXT step (`next`), so the next step's rows are in flight
// for a whole step without a second set of registers.  After the last step
// the reload is redundant but harmless: `next` is clamped into the sequence.
template <typename T, int CH, int KL, bool CONV, bool FAST, bool PLAIN>
__device__ __forceinline__ void phase1(
    Tile<T, CH, KL>& tl, const StepAddr<KL>& next, uint32_t voff,
    const ChanConst<CH>& k, float (&a_)[KL][CH], float (&xn_)[KL][CH],
    float (&P)[CH], float (&H)[CH], bool halo_from_memory) {
  using B = Buf<T, CH>;
  constexpr bool PACKED = kPackedConv<T, CH, CONV>;
  float hist[3][CH];
  PairRow<CH> pp2, pp1;  // PACKED: the pairs ending one and two rows back
  typename B::Raw prev_row{};
  if constexpr (PACKED) {
    pp2 = pair_rows(tl.halo[2], tl.halo[1]);
    pp1 = pair_rows(tl.halo[1], tl.halo[0]);
    prev_row = tl.halo[0];
  } else {
#pragma unroll
    for (int s = 0; s < 3; ++s) B::unpack(tl.halo[s], hist[s]);
  }
  // The reload must follow the last read of the registers it overwrites;
  // without these fences the scheduler hoists it, old and new values overlap,
  // and the new tile needs register copies (and full waits) every step.
  __builtin_amdgcn_sched_barrier(0);
  // (the other waves get the next step's look-back rows from the wave before
  // them, through LDS: see the exchange)
  if (halo_from_memory) load_halo<T, CH, KL, CONV>(tl, next, voff);
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    P[ch] = 1.0f;
    H[ch] = 0.0f;
  }
#pragma unroll
  for (int i = 0; i < KL; ++i) {
    float xv[CH], gxv[CH], gav[CH], xc[CH];
    PairRow<CH> pp0;
    if constexpr (PACKED) {
      pp0 = pair_rows(prev_row, tl.x[i]);
      prev_row = tl.x[i];
    } else {
      B::unpack(tl.x[i], xv);
    }
    if (!PLAIN) B::unpack(tl.gx[i], gxv);
    B::unpack(tl.ga[i], gav);
    __builtin_amdgcn_sched_barrier(0);
    load_token<T, CH, KL, PLAIN>(tl, i, next, voff);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (PACKED) {
      conv_dot(pp2, pp0, k, xc);
      pp2 = pp1;
      pp1 = pp0;
      B::round(xc);  // the conv output is a module output: activation dtype
    } else if (CONV) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        xc[ch] = conv4_as<T>(xv[ch], hist[0][ch], hist[1][ch], hist[2][ch],
                             k.w0[ch], k.w1[ch], k.w2[ch], k.w3[ch], k.bias[ch]);
        hist[2][ch] = hist[1][ch];
        hist[1][ch] = hist[0][ch];
        hist[0][ch] = xv[ch];
      }
      B::round(xc);  // the conv output is a module output: activation dtype
    } else {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) xc[ch] = xv[ch];
    }
    gate_math<CH, FAST, PLAIN>(xc, gxv, gav, k.decay, false, a_[i], xn_[i]);
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      H[ch] = __builtin_fmaf(a_[i][ch], H[ch], xn_[i][ch]);
      P[ch] = P[ch] * a_[i][ch];
    }
  }
}

// Phase 1, slow path: a step with a document start.  Recomputes the wave's
// (a, xn) pairs from memory (the rows are still in cache), with the conv
// history cut at every start and a = 0, input scale 1 there.  It does not
// touch the prefetched tile.
template <typename T, int CH, int KL, bool CONV, bool FAST, bool PLAIN>
__device__ __forceinline__ void phase1_with_starts(
    const StepAddr<KL>& at, uint32_t voff, uint32_t starts,
    const ChanConst<CH>& k, float (&a_)[KL][CH], float (&xn_)[KL][CH],
    float (&P)[CH], float (&H)[CH]) {
  using B = Buf<T, CH>;
  constexpr bool PACKED = kPackedConv<T, CH, CONV>;
  float hist[3][CH];
  typename B::Raw rows[3] = {};  // PACKED: rows[s] = x[t-1-s], still packed
#pragma unroll
  for (int s = 0; s < 3; ++s)
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) hist[s][ch] = 0.0f;
  if (CONV && at.has_halo) {
#pragma unroll
    for (int s = 0; s < 3; ++s) {  // hist[s] = x[first-1-s]
      rows[s] =
          B::template load<0>(at.rhalo, voff, (uint32_t)(2 - s) * at.row_bytes);
      B::unpack(rows[s], hist[s]);
    }
    // a document start at first-1 hides x[first-2], x[first-3]; one at
    // first-2 hides x[first-3]
    if (starts & 4u) {
      rows[1] = rows[2] = typename B::Raw{};
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) hist[1][ch] = hist[2][ch] = 0.0f;
    }
    if (starts & 2u) {
      rows[2] = typename B::Raw{};
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) hist[2][ch] = 0.0f;
    }
  }
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    P[ch] = 1.0f;
    H[ch] = 0.0f;
  }
#pragma unroll
  for (int i = 0; i < KL; ++i) {
    const bool start = (starts >> (i + 3)) & 1u;
    const uint32_t so = at.soff(i);
    float xv[CH], gxv[CH], gav[CH], xc[CH];
    const typename B::Raw xraw = B::template load<0>(at.rx, voff, so);
    B::unpack(xraw, xv);
    if (!PLAIN) B::unpack(B::template load<0>(at.rgx, voff, so), gxv);
    B::unpack(B::template load<0>(at.rga, voff, so), gav);
    if constexpr (PACKED) {
      // the same two dot products per output as on the hot path
      if (start) rows[0] = rows[1] = rows[2] = typename B::Raw{};
      conv_dot(pair_rows(rows[2], rows[1]), pair_rows(rows[0], xraw), k, xc);
      rows[2] = rows[1];
      rows[1] = rows[0];
      rows[0] = xraw;
      B::round(xc);
    } else if (CONV) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        if (start) hist[0][ch] = hist[1][ch] = hist[2][ch] = 0.0f;
        xc[ch] = conv4_as<T>(xv[ch], hist[0][ch], hist[1][ch], hist[2][ch],
                             k.w0[ch], k.w1[ch], k.w2[ch], k.w3[ch], k.bias[ch]);
        hist[2][ch] = hist[1][ch];
        hist[1][ch] = hist[0][ch];
        hist[0][ch] = xv[ch];
      }
      B::round(xc);
    } else {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) xc[ch] = xv[ch];
    }
    gate_math<CH, FAST, PLAIN>(xc, gxv, gav, k.decay, start, a_[i], xn_[i]);
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      H[ch] = __builtin_fmaf(a_[i][ch], H[ch], xn_[i][ch]);
      P[ch] = P[ch] * a_[i][ch];
    }
  }
}

// Phase 2: replay the recurrence from the incoming state and write y.  Stores
// of tokens past the end of the sequence get a scalar offset outside the
// descriptor and are dropped by the range check.  The state after token T-1
// is written to h_last by the wave that holds that token.
template <typename T, int CH, int KL>
__device__ __forceinline__ void phase2(__amdgpu_buffer_rsrc_t ry, uint32_t voff,
                                       uint32_t row_bytes, int n_valid,
                                       float* h_last_lane,
                                       const float (&a_)[KL][CH],
                                       const float (&xn_)[KL][CH],
                                       float (&h)[CH]) {
  using B = Buf<T, CH>;
#pragma unroll
  for (int i = 0; i < KL; ++i) {
    float out[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      h[ch] = __builtin_fmaf(a_[i][ch], h[ch], xn_[i][ch]);
      out[ch] = h[ch];
    }
    B::template store<kStream>(
        ry, voff, i < n_valid ? (uint32_t)i * row_bytes : kOutOfRange, out);
    if (h_last_lane && i == n_valid - 1) {
      RG_RARE_BLOCK();
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) h_last_lane[ch] = h[ch];
    }
  }
}

// SPLIT: a row's sequence cut into chunks that run as workgroups of their own
// (blockIdx.y), for few rows and channel slabs: 0 = the whole row in one
// workgroup; 1 = summary of a chunk: its state from a zero start and the
// product of its a_t, nothing else written; 2 = the chunk again from its true
// incoming state (h_in, computed from the summaries), writing y.  The scan
// operator is associative, so this is the kernel's own cross-wave carry one
// level up.
enum ScanSplit { kWholeRow = 0, kChunkSummary = 1, kChunkReplay = 2 };

template <typename T, int CH, int KL, bool CONV, bool FAST, bool PLAIN,
          int SPLIT>
__global__ void __launch_bounds__(kMaxNW* kWave, (sizeof(T) == 2 ? 4 : 2))
lru_scan_kernel(ScanArgs p) {
  // LDS (sized at launch): per buffer and wave the lanes' (P.., Hloc..)
  // pairs, then the two carry rows
  extern __shared__ __align__(16) float lds_f[];
  typedef float AggRow[kWave][2 * CH];
  typedef float CarryRow[kWave][CH];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nw = blockDim.x >> 6;
  AggRow* const agg0 = reinterpret_cast<AggRow*>(lds_f);   // [2][nw]
  CarryRow* const carry_s =
      reinterpret_cast<CarryRow*>(lds_f + 2 * nw * kWave * 2 * CH);  // [2]
  // The three look-back rows of a wave's conv are the last three rows of the
  // wave before it: instead of reading them from memory a second time, every
  // wave leaves the last three of the rows it has prefetched for the next
  // step in LDS before the step's barrier and takes its neighbour's behind
  // it, [2][nw][3][64].  Wave 0, whose look-back rows belong to the step
  // before, keeps loading them.
  typedef typename Buf<T, CH>::Raw RawRow;
  RawRow* const halo_s = reinterpret_cast<RawRow*>(
      lds_f + 2 * nw * kWave * 2 * CH + 2 * kWave * CH);
  const bool share_halo = CONV && KL >= 3 && nw > 1;
  // tokens [t_lo, T_len) of the row are this workgroup's; everything below
  // treats T_len as the end of the sequence
  const int chunk = SPLIT == kWholeRow ? 0 : (int)blockIdx.y;
  const int t_lo = SPLIT == kWholeRow ? 0 : chunk * p.t_chunk;
  const int T_len =
      SPLIT == kWholeRow ? p.T : (t_lo + p.t_chunk < p.T ? t_lo + p.t_chunk : p.T);
  const bool last_chunk = T_len == p.T;
  const int64_t W = p.W;
  const int nslab = (p.W + kWave * CH - 1) / (kWave * CH);
  const int b = blockIdx.x / nslab;
  const int slab = blockIdx.x - b * nslab;
  const int c_raw = (slab * kWave + lane) * CH;
  const bool active = c_raw < p.W;  // W % CH == 0, so the whole vector is in
  const int c = active ? c_raw : 0;  // for the few plain-pointer accesses

  ChanConst<CH> k;
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    if (CONV) {
      const T* cw = (const T*)p.conv_w;
      k.w0[ch] = load_scalar(cw + c + ch);
      k.w1[ch] = load_scalar(cw + W + c + ch);
      k.w2[ch] = load_scalar(cw + 2 * W + c + ch);
      k.w3[ch] = load_scalar(cw + 3 * W + c + ch);
      k.bias[ch] = load_scalar((const T*)p.conv_b + c + ch);
      if (sizeof(T) == 2) {
        const uint16_t* cb = (const uint16_t*)p.conv_w;
        k.w10[ch] = (uint32_t)cb[c + ch] | ((uint32_t)cb[W + c + ch] << 16);
        k.w32[ch] = (uint32_t)cb[2 * W + c + ch] |
                    ((uint32_t)cb[3 * W + c + ch] << 16);
      } else {
        k.w10[ch] = k.w32[ch] = 0u;
      }
    } else {
      k.w0[ch] = k.w1[ch] = k.w2[ch] = k.w3[ch] = k.bias[ch] = 0.0f;
      k.w10[ch] = k.w32[ch] = 0u;
    }
    if (PLAIN) {
      k.decay[ch] = 0.0f;
    } else {
      const float sp =
          softplus_precise(load_scalar((const T*)p.a_param + c + ch));
      k.decay[ch] = FAST ? (-8.0f * kLog2e) * sp : sp;
    }
  }

  const int64_t row0 = (int64_t)b * p.T;
  const uint32_t row_bytes = (uint32_t)p.W * (uint32_t)sizeof(T);
  const uint32_t voff =
      active ? (uint32_t)c_raw * (uint32_t)sizeof(T) : kOutOfRange;
  const uint32_t span_bytes = (uint32_t)KL * row_bytes;
  // wave-uniform pointers to token 0 of this batch row
  const char* xrow = (const char*)p.x + row0 * row_bytes;
  const char* gxrow = (const char*)p.gx + row0 * row_bytes;
  const char* garow = (const char*)p.ga + row0 * row_bytes;
  char* yrow = (char*)p.y + row0 * row_bytes;

  // per-chunk rows of the workspace: [B][chunks][W] each
  const int64_t ws_row = ((int64_t)b * p.chunks + chunk) * W + c;
  float h[CH];
  float chunk_p[CH];  // kChunkSummary: product of every a_t seen so far
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    if (SPLIT == kChunkSummary) h[ch] = 0.0f;
    else if (SPLIT == kChunkReplay) {
      // state at the start of this chunk: h <- P[k] h + H[k] over the chunks
      // before it (the scan operator one level up)
      float hin = p.h0 ? p.h0[(int64_t)b * W + c + ch] : 0.0f;
      const int64_t ws0 = (int64_t)b * p.chunks * W + c + ch;
      for (int kc = 0; kc < chunk; ++kc)
        hin = __builtin_fmaf(p.ws_p[ws0 + (int64_t)kc * W], hin,
                             p.ws_h[ws0 + (int64_t)kc * W]);
      h[ch] = hin;
    }
    else h[ch] = p.h0 ? p.h0[(int64_t)b * W + c + ch] : 0.0f;
    chunk_p[ch] = 1.0f;
  }

  const int span = nw * KL;

  // Every wave runs every step with the same code, so that the prefetched
  // tile is never merged with a copy of itself at a branch join (that would
  // cost register copies and a full wait per step).  A wave whose tokens lie
  // past the end of the sequence works on a re-read of the last row, drops
  // its stores and contributes the identity pair.

  // prologue: the first step's rows
  Tile<T, CH, KL> tl;
  uint32_t starts;
  {
    const SegRaw seg =
        load_seg<KL, CONV>(p, row0, t_lo + wave * KL, T_len, lane);
    const StepAddr<KL> a0 =
        step_addr<KL>(xrow, gxrow, garow, t_lo + wave * KL, T_len, row_bytes);
    load_halo<T, CH, KL, CONV>(tl, a0, voff);
#pragma unroll
    for (int i = 0; i < KL; ++i) load_token<T, CH, KL, PLAIN>(tl, i, a0, voff);
    starts = doc_starts(seg);
  }

  for (int step = 0, tb = t_lo; tb < T_len; ++step, tb += span) {
    const int buf = step & 1;
    const int t0 = tb + wave * KL;
    const bool any = t0 < T_len;
    // tokens of this wave inside the sequence (<= 0: none)
    const int n_valid = T_len - t0 < KL ? T_len - t0 : KL;
    float a_[KL][CH], xn_[KL][CH], P[CH], H[CH];
    const StepAddr<KL> next =
        step_addr<KL>(xrow, gxrow, garow, t0 + span, T_len, row_bytes);
    // next step's document starts: loaded now, looked at after this step
    const SegRaw seg_next = load_seg<KL, CONV>(p, row0, t0 + span, T_len, lane);
    phase1<T, CH, KL, CONV, FAST, PLAIN>(tl, next, voff, k, a_, xn_, P, H,
                                         !share_halo || wave == 0);
    if (starts != 0u) {
      RG_RARE_BLOCK();
      const StepAddr<KL> cur =
          step_addr<KL>(xrow, gxrow, garow, t0, T_len, row_bytes);
      phase1_with_starts<T, CH, KL, CONV, FAST, PLAIN>(cur, voff, starts, k, a_,
                                                       xn_, P, H);
    }

    // exchange
    AggRow* const agg = agg0 + buf * nw;
    if (!any) {  // past the end of the sequence: the identity pair
      RG_RARE_BLOCK();
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        P[ch] = 1.0f;
        H[ch] = 0.0f;
      }
    }
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      agg[wave][lane][ch] = P[ch];
      agg[wave][lane][CH + ch] = H[ch];
    }
    if (share_halo) {  // tl.x holds the next step's rows by now
      RawRow* const dst = halo_s + ((buf * nw + wave) * 3) * kWave + lane;
#pragma unroll
      for (int s = 0; s < 3; ++s) dst[s * kWave] = tl.x[KL - 1 - s];
    }
    lds_barrier();  // LDS only: prefetched rows and earlier stores stay in flight
    if (share_halo && wave > 0) {
      const RawRow* const src =
          halo_s + ((buf * nw + wave - 1) * 3) * kWave + lane;
#pragma unroll
      for (int s = 0; s < 3; ++s) tl.halo[s] = src[s * kWave];  // x[first-1-s]
    }
    if (step > 0) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) h[ch] = carry_s[buf ^ 1][lane][ch];
    }
    for (int v = 0; v < wave; ++v) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) {
        h[ch] = __builtin_fmaf(agg[v][lane][ch], h[ch], agg[v][lane][CH + ch]);
        if (SPLIT == kChunkSummary) chunk_p[ch] *= agg[v][lane][ch];
      }
    }
    if (SPLIT == kChunkSummary) {  // complete in the last wave only
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) chunk_p[ch] *= P[ch];
    }

    {
      // (a summary writes no y: a descriptor of no bytes drops every store)
      const __amdgpu_buffer_rsrc_t ry = make_rsrc(
          yrow + (int64_t)(any ? t0 : T_len - 1) * row_bytes,
          SPLIT == kChunkSummary ? 0u : span_bytes);
      // this wave holds token T-1 iff its valid tokens end the sequence
      float* h_end = p.h_last ? p.h_last + (int64_t)b * W + c : nullptr;
      if (SPLIT == kChunkSummary) h_end = p.ws_h + ws_row;
      if (SPLIT == kChunkReplay && !last_chunk) h_end = nullptr;
      float* const h_last_lane =
          (h_end && active && any && t0 + n_valid == T_len) ? h_end : nullptr;
      if (SPLIT == kChunkSummary) {
        // no outputs to replay for: the wave's pair applied to its incoming
        // state is its final state (summaries are taken of whole steps only:
        // the last chunk of a row, which may end inside a step, has none; a
        // wave without tokens holds the identity pair)
#pragma unroll
        for (int ch = 0; ch < CH; ++ch)
          h[ch] = __builtin_fmaf(P[ch], h[ch], H[ch]);
        if (h_last_lane) {
#pragma unroll
          for (int ch = 0; ch < CH; ++ch) h_last_lane[ch] = h[ch];
        }
      } else if (any) {
        // (a wave without tokens hands the carry on unchanged)
        phase2<T, CH, KL>(ry, voff, row_bytes, n_valid, h_last_lane, a_, xn_,
                          h);
      }
    }
    if (wave == nw - 1) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) carry_s[buf][lane][ch] = h[ch];
    }
    starts = doc_starts(seg_next);
  }

  if (SPLIT == kChunkSummary) {
    if (wave == nw - 1 && active) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) p.ws_p[ws_row + ch] = chunk_p[ch];
    }
    return;
  }
  if (SPLIT == kChunkReplay && !last_chunk) return;

  // Masked conv state: rows T-3..T-1 of x, each zeroed if a document starts in
  // a later position of the row; rows before the sequence start are zero.
  if (CONV && p.cache_out && wave == 0 && active) {
    T* cache = (T*)p.cache_out + (int64_t)b * 3 * W + c;
    bool later_start = false;
#pragma unroll
    for (int kk = 2; kk >= 0; --kk) {
      const int t = T_len - 3 + kk;
      const bool copy = t >= 0 && !later_start;
      const T* src = (const T*)(xrow + (int64_t)(t >= 0 ? t : 0) * row_bytes) + c;
#pragma unroll
      for (int ch = 0; ch < CH; ++ch)
        store_scalar(cache + (int64_t)kk * W + ch,
                     copy ? load_scalar(src + ch) : 0.0f);
      if (t >= 0 && is_doc_start(p.segpos, p.seg_kind, row0 + t))
        later_start = true;
    }
  }
}

template <typename T, int CH, int KL, bool CONV, bool FAST, bool PLAIN,
          int SPLIT>
hipError_t launch_t(const ScanArgs& a, hipStream_t s) {
  const int nslab = (a.W + kWave * CH - 1) / (kWave * CH);
  const int64_t blocks = (int64_t)a.B * nslab;
  // (the last chunk's summary would feed no other chunk: not computed)
  const int chunks = SPLIT == kWholeRow
                         ? 1
                         : (SPLIT == kChunkSummary ? a.chunks - 1 : a.chunks);
  const int t_run = SPLIT == kWholeRow ? a.T : a.t_chunk;
  // Waves per workgroup: enough to cover the sequence, and 16 rather than 8
  // when the grid alone would leave most of the 256 CUs' wave slots empty.
  int max_nw = blocks * chunks * 8 >= 4096 ? 8 : kMaxNW;
  int nw = 1;
  while (nw < max_nw && nw * KL < t_run) nw *= 2;
  if (SPLIT != kWholeRow && (a.t_chunk % (nw * KL) != 0 || chunks > 65535))
    return hipErrorInvalidValue;
  // a wave's rows of one step must fit a descriptor's 32-bit offsets
  if (blocks > 0x7fffffff ||
      (int64_t)a.W * sizeof(T) * (KL + 3) >= (int64_t)kOutOfRange)
    return hipErrorInvalidValue;
  const size_t halo_rows =
      CONV && KL >= 3 && nw > 1
          ? (size_t)2 * nw * 3 * kWave * sizeof(typename Buf<T, CH>::Raw)
          : 0;
  const size_t lds =
      sizeof(float) * (2 * nw * kWave * 2 * CH + 2 * kWave * CH) + halo_rows;
  auto kern = lru_scan_kernel<T, CH, KL, CONV, FAST, PLAIN, SPLIT>;
  // the limit is raised once, to what the largest workgroup of this
  // instantiation needs
  constexpr size_t lds_max =
      sizeof(float) * (2 * kMaxNW * kWave * 2 * CH + 2 * kWave * CH) +
      (size_t)2 * kMaxNW * 3 * kWave * sizeof(typename Buf<T, CH>::Raw);
  if (lds_max > 48 * 1024) {
    static OncePerDevice once;  // one per instantiation of this launcher
    hipError_t e = set_max_dynamic_lds(once, (const void*)kern, lds_max);
    if (e != hipSuccess) return e;
  }
  kern<<<dim3((unsigned)blocks, (unsigned)chunks), dim3(nw * kWave), lds, s>>>(
      a);
  return hipGetLastError();
}

template <typename T, int CH, int KL, bool CONV, bool FAST, bool PLAIN>
hipError_t launch_split(const ScanArgs& a, hipStream_t s) {
  if (a.chunks <= 1)
    return launch_t<T, CH, KL, CONV, FAST, PLAIN, kWholeRow>(a, s);
  hipError_t e = launch_t<T, CH, KL, CONV, FAST, PLAIN, kChunkSummary>(a, s);
  if (e != hipSuccess) return e;
  return launch_t<T, CH, KL, CONV, FAST, PLAIN, kChunkReplay>(a, s);
}

template <typename T, int CH, int KL, bool FAST>
hipError_t launch_mode(const ScanArgs& a, hipStream_t s) {
  if (a.plain) return launch_split<T, CH, KL, false, FAST, true>(a, s);
  if (a.apply_conv) return launch_split<T, CH, KL, true, FAST, false>(a, s);
  return launch_split<T, CH, KL, false, FAST, false>(a, s);
}

}  // namespace

// Whether, and how, to cut the sequences of this shape into chunks.  One
// workgroup walks a row at about 2.5 us per 64-token step however few of them
// run (a row of 8192 tokens: 0.32 ms).  Cut into chunks the rows are read
// twice, but every CU works: the aim is one workgroup per CU (more would queue
// for a second round on the CUs that finish first), chunk lengths in multiples
// of `granule` tokens, the longest step of the kernel that will run (16 waves
// at 8 tokens each: 128; float32 with two channels per lane: 16 x 4 = 64).
// Worth it up to about 32 (row, 256-channel slab) pairs and from about five
// hundred tokens on; measured, bf16, T = 8192: 10 pairs 321 -> 75 us, 80 pairs
// no gain.
void scan_split_plan(int B, int T, int W, int granule, int* chunks,
                     int* t_chunk) {
  *chunks = 1;
  *t_chunk = T;
  const int64_t wide_blocks = (int64_t)B * ((W + 255) / 256);
  if (wide_blocks > 32 || T < 512) return;
  const int want = (int)(256 / wide_blocks);
  const int len = ((T + want - 1) / want + granule - 1) / granule * granule;
  const int n = (T + len - 1) / len;
  if (n < 2) return;
  *t_chunk = len;
  *chunks = n;
}

int scan_split_granule(int dtype, int W) {
  return dtype == 0 && W % 2 == 0 ? 64 : 128;
}

hipError_t launch_lru_scan(const ScanArgs& a, int dtype, hipStream_t s) {
  // Channels per lane: 8 bytes per lane where the width allows it (every row
  // then starts on a vector boundary; base pointers are checked by the
  // caller), with short steps; narrower vectors take longer steps.
  if (dtype == 0) {
    if (a.W % 2 == 0) return launch_mode<float, 2, 4, false>(a, s);
    return launch_mode<float, 1, 8, false>(a, s);
  }
  // 8-byte lanes halve the number of workgroups (B * ceil(W/256)); below
  // about 200 of them too many of the 256 CUs idle and 4-byte lanes win.
  const int64_t wide_blocks =
      (int64_t)a.B * ((a.W + 255) / 256) * (a.chunks > 1 ? a.chunks : 1);
  if (a.W % 4 == 0 && wide_blocks >= 200)
    return launch_mode<uint16_t, 4, 4, true>(a, s);
  if (a.W % 2 == 0) return launch_mode<uint16_t, 2, 8, true>(a, s);
  return launch_mode<uint16_t, 1, 8, true>(a, s);
}

}  // namespace rg
