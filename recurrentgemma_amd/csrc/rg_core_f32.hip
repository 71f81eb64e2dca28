// The recurrent core of a short float32 prefill in ONE launch (256-wide
// heads, few rows): width-4 conv -> both gate projections on the float32
// matrix instruction -> gate activations -> recurrence.
//
// The three-launch form (gate GEMM, then the scan in two passes over chunks of
// the sequence) spends most of a small call waiting for launches and for each
// kernel's first loads.  Here one workgroup of eight waves (two per SIMD) owns
// 16 channels of one head of one row for the whole sequence: 16 B x H
// workgroups.  Per segment of 512 tokens each wave takes 64 of them in tiles
// of 16, and a tile's 256 input channels in two passes of 128: rows loaded
// (two channels a lane), convolved and staged in LDS (every workgroup of a
// head convolves the same rows again: the conv is 4 multiply-adds per
// element), 64 v_mfma_f32_16x16x4_f32 per pass against the wave's resident
// weights (256 x 16 per gate: 128 accumulation registers) give the
// pre-activations of the 16 channels, the gate arithmetic leaves (a, a-scaled
// input) per token and channel in LDS; then the workgroup scans the segment as
// 32 chunks of 16 tokens per channel (chunk summaries, a scan over the
// summaries by lane shifts, replay) and stores y.
//
// True float32 products and sums (no reduced-precision operand formats): the
// float32 bar of 1e-5 stands (measured against the gate GEMM + scan pair:
// 2e-7 .. 5e-7 of the largest output, conv state identical).  Same conv4() tap
// chain as the other float32 kernels; exp2, reciprocal and square root of the
// gate arithmetic are the hardware's.
//
// Where the time goes (B1 T512 W2560, 160 workgroups, 35-37 us = 72 000
// cycles): fetching the weights 7 000, the eight tiles of a SIMD 61 000, the
// scan 4 000.  A tile costs 7 600 cycles, 4 100 of them its 128 matrix
// instructions at 32 cycles each: the float32 matrix instruction keeps the
// SIMD's vector unit busy while it runs (a second wave's multiply-adds do not
// get in between, measured), so matrix and vector work add up whatever the
// schedule, and the second wave per SIMD only hides latencies.
//
// Replaces the chain Conv1D.forward -> RGLRU.forward of
// recurrentgemma/torch/modules.py:632-643 (layers.py:447-529, 313-365,
// 140-191) for such shapes.
#include <type_traits>
#include <utility>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;      // head width
constexpr int kCh = 16;       // output channels per workgroup
constexpr int kTile = 16;     // tokens per matrix tile
constexpr int kSeg = 512;     // tokens per segment
constexpr int kWaves = 8;     // two per SIMD
constexpr int kThreads = kWaves * 64;
constexpr int kTilesPerWave = kSeg / kWaves / kTile;  // 4
constexpr int kHalf = kBW / 2;                        // input channels per pass
constexpr int kStageStride = kHalf + 4;               // floats per staged row
constexpr int kChunk = 16;                            // tokens per scan chunk
constexpr int kChunks = kSeg / kChunk;                // 32
constexpr int kWRow = kCh + 4;  // floats per row of the weights' way through LDS

// Where token t of a segment keeps its 16 channels in CoreF32Lds::a / xn: four
// tokens fill the 64 banks, and which quarter of them a token takes rotates
// with the token's group of 4 and group of 16, so that neither the gate
// stage (a wave writes tokens 4 g + q, g = 0..3, at once) nor the scan (a wave
// reads tokens 16 c + i of four chunks c at once) meets a bank twice.
__device__ __forceinline__ int gate_slot(int t) {
  return (t & ~3) + (((t & 3) + (t >> 2) + (t >> 4)) & 3);
}

struct CoreF32Lds {
  float stage[kWaves][kTile][kStageStride];  // conv output, half a tile's K
  float a[kSeg][kCh];                        // per token and channel: a_t
  float xn[kSeg][kCh];                       // ... and the scaled input
  float chunk_p[kChunks][kCh];               // product of a over a chunk
  float chunk_h[kChunks][kCh];               // its state from a zero start,
                                             // then the state it starts from
  float carry[kCh];                          // state at the segment's start
  float own[kWaves][kTile][kCh];             // conv output of the own channels
  f32x2 taps[2][5][64];                      // conv taps and bias, per lane
};

// The wave's weights (256 x 16 per gate, B operands of
// v_mfma_f32_16x16x4_f32) live in the accumulation registers a[0..127],
// written and read by inline assembly with the register number spelled out:
// a[4 i + q] holds the input gate's weight of k = 16 i + 4 g + q for lane
// (g, n), a[64 + 4 i + q] the recurrence gate's.  With two waves per SIMD a
// wave has 256 registers, and the other 128 are what the conv rows in flight,
// the accumulators and the gate arithmetic need.  (Left to the compiler, the
// accumulators go to the accumulation registers and every weight is moved to
// an ordinary register before its use.)
//
// The matrix instructions being inline assembly, the compiler does not count
// the wait states between one and a vector instruction that reads its
// result.  Two things keep that safe: a tile's last two matrix instructions
// and the wait for their results are ONE statement, and the accumulators of
// consecutive tiles are different variables (the gate arithmetic of a tile
// runs during the next tile, on the set that tile does not use), so that the
// compiler has no copy of an accumulator to make between two matrix
// instructions.
__device__ __forceinline__ float in_accumulation_register(float v) {
  float w;
  asm("v_accvgpr_write_b32 %0, %1" : "=a"(w) : "v"(v));
  return w;
}
__device__ __forceinline__ void mfma_weight(float a, float w, f32x4& acc) {
  asm volatile("v_mfma_f32_16x16x4_f32 %0, %1, %2, %0"
               : "+v"(acc)
               : "v"(a), "a"(w));
}
__device__ __forceinline__ void mfma_weight_last(float a, float w_x, float w_a,
                                                 f32x4& acc_x, f32x4& acc_a) {
  asm volatile(
      "v_mfma_f32_16x16x4_f32 %0, %2, %3, %0\n\t"
      "v_mfma_f32_16x16x4_f32 %1, %2, %4, %1\n\t"
      "s_nop 15\n\t"
      "s_nop 3"
      : "+v"(acc_x), "+v"(acc_a)
      : "v"(a), "a"(w_x), "a"(w_a));
}
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// GELU: y is written as y * gelu(gate_branch), the join of the recurrent
// block's two branches (recurrentgemma/torch/modules.py:627-628, 644).
template <bool HAS_CONV, bool GELU>
__global__ void __launch_bounds__(kThreads) core_f32_small_kernel(FusedArgs p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  CoreF32Lds& lds = *reinterpret_cast<CoreF32Lds*>(lds_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // 16 workgroups per (row, head).  Workgroups go to the eight XCDs in turn
  // (linear id modulo 8), each with an L2 of its own: the 16 workgroups of a
  // pair are dealt to ONE of them, so that the head's rows and weights, which
  // all 16 read, come through one L2 (pair p runs on XCD p % 8; the grid is
  // rounded up to whole rounds of eight pairs and the surplus exits).
  constexpr int slices = kBW / kCh;
  const int xcd = blockIdx.x & 7;
  const int in_xcd = blockIdx.x >> 3;
  const int pair = (in_xcd / slices) * 8 + xcd;
  if (pair >= p.B * p.H) return;
  const int s = in_xcd % slices;
  const int h = pair % p.H;
  const int b = pair / p.H;
  const int T = p.T;
  const int64_t W = p.W;
  const int c_head = h * kBW;         // first channel of the head
  const int c0 = c_head + s * kCh;    // first channel of this workgroup
  const int g = lane >> 4;            // matrix layout: lane = (g, n)
  const int n = lane & 15;
  // the half of the head's channels this workgroup's own 16 are in, and where
  // in a staged row of that half
  const int own_half = s >> 3;
  const int own_col = (s & 7) * kCh + n;

  // (the small per-channel loads first, so that they travel together with
  // the weights instead of after them)
  const float bias_x = ((const float*)p.b[0])[c0 + n];
  const float bias_a = ((const float*)p.b[1])[c0 + n];
  // log2 a_t = sigmoid(.) * (-8 log2(e) softplus(a_param))  (layers.py:343-349)
  const float decay2 =
      -8.0f * kLog2e * softplus_precise(((const float*)p.a_param)[c0 + n]);

  // conv taps of this lane's two input channels of either half (2 lane,
  // 2 lane + 1 of the half); without conv weights x is the conv output already
  constexpr bool has_conv = HAS_CONV;
  // (kept in LDS and read per pass: 20 registers that the matrix passes need)
  if (has_conv && wave < 2) {
    const int hh = wave;
    const float* w = (const float*)p.conv_w + c_head + kHalf * hh + 2 * lane;
#pragma unroll
    for (int k = 0; k < 4; ++k)
      lds.taps[hh][k][lane] = *reinterpret_cast<const f32x2*>(w + k * W);
    lds.taps[hh][4][lane] = *reinterpret_cast<const f32x2*>(
        (const float*)p.conv_b + c_head + kHalf * hh + 2 * lane);
  }

  // ---- weights of the wave.  The k of a matrix instruction are chosen so
  //      that a lane's A values of four instructions are four consecutive
  //      floats of its staged row: instruction (i, q) multiplies
  //      k = 16 i + 4 g' + q, g' = 0..3.
  //      The workgroup fetches its 256 x 16 weights of either gate once, 16
  //      bytes a thread and four times, into LDS (where the gates' results
  //      will live later; rows of 20 floats, so that the 64 lanes of a wave
  //      read 64 banks), and every wave fills its registers from there.
  float wx[64], wa[64];  // [4 i + q]: k = 16 i + 4 g + q
  {
    float* const wbuf = &lds.a[0][0];
    static_assert(sizeof(lds.a) + sizeof(lds.xn) >= 2 * kBW * kWRow * 4, "");
#pragma unroll
    for (int j = 0; j < 2 * kBW * kCh / 4 / kThreads; ++j) {
      const int idx = tid + kThreads * j;
      const int gate = idx / (kBW * kCh / 4);
      const int k = (idx >> 2) & (kBW - 1);
      const int part = idx & 3;
      const float* src = (const float*)p.w[gate] + (int64_t)h * kBW * kBW +
                         (int64_t)k * kBW + s * kCh + 4 * part;
      *reinterpret_cast<f32x4*>(&wbuf[(gate * kBW + k) * kWRow + 4 * part]) =
          *reinterpret_cast<const f32x4*>(src);
    }
    __syncthreads();
#pragma unroll
    for (int j0 = 0; j0 < 64; j0 += 16) {
      // (16 of each gate at a time, all requested before the first is used)
      float vx[16], va[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int k = 16 * ((j0 + j) >> 2) + 4 * g + (j & 3);
        vx[j] = wbuf[k * kWRow + n];
        va[j] = wbuf[(kBW + k) * kWRow + n];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        wx[j0 + j] = in_accumulation_register(vx[j]);
        wa[j0 + j] = in_accumulation_register(va[j]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const uint32_t row_bytes = 4u * (uint32_t)W;
  const uint32_t seq_bytes = (uint32_t)T * row_bytes;  // < 2^31 (launcher)
  const __amdgpu_buffer_rsrc_t rx =
      make_rsrc((const char*)p.x + (int64_t)b * seq_bytes, seq_bytes);
  const __amdgpu_buffer_rsrc_t rnone =
      make_rsrc((const char*)p.x + (int64_t)b * seq_bytes, 0);
  const bool seg_is64 = p.seg_kind == kSegI64;
  const uint32_t seg_esize = seg_is64 ? 8u : 4u;
  const __amdgpu_buffer_rsrc_t rseg =
      make_rsrc((const char*)p.segpos + (int64_t)b * T * seg_esize,
                (uint32_t)T * seg_esize);

  if (tid < kCh)
    lds.carry[tid] = p.h0 ? p.h0[(int64_t)b * W + c0 + tid] : 0.0f;
  __syncthreads();  // taps and carry written, every wave has read its weights
  const int nseg = (T + kSeg - 1) / kSeg;
  for (int seg = 0; seg < nseg; ++seg) {
    // ---- stage 1: this wave's 64 tokens of the segment, a tile at a time, a
    //      tile's 256 input channels in two passes of 128 ----
    const int wave_t0 = seg * kSeg + wave * (kSeg / kWaves);
    // Rows t0-3 .. t0+15 of one half of the head's channels, two per lane
    // (rows outside the sequence: zeros).  The
    // rows of a pass are requested when the pass before it has consumed its
    // own, and arrive while it multiplies.
    f32x2 xr[kTile + 3];
    uint32_t seg_lo = 1, seg_hi = 0;
    const uint32_t lane_col = 4u * (uint32_t)(c_head + 2 * lane);
    // (a row's offset is a scalar, which the descriptor does not check: rows
    // outside the sequence are read through a descriptor of no bytes instead;
    // no per-lane address arithmetic)
    auto request_rows = [&](int t0, int hh) {
#pragma unroll
      for (int r = has_conv ? 0 : 3; r < kTile + 3; ++r) {
        const uint32_t t = (uint32_t)(t0 - 3 + r);
        xr[r] = __builtin_bit_cast(
            f32x2, __builtin_amdgcn_raw_buffer_load_b64(
                       t < (uint32_t)T ? rx : rnone, lane_col + 4u * kHalf * hh,
                       t * row_bytes, 0));
      }
    };
    // positions of rows t0-2 .. t0+15 (lane j looks at row t0 - 2 + j)
    auto request_positions = [&](int t0) {
      const int t = t0 - 2 + lane;
      const bool in = lane < kTile + 2 && t >= 0 && t < T;
      const uint32_t off = in ? (uint32_t)t * seg_esize : kBufferOutOfRange;
      seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
      seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
          rseg, seg_is64 ? off + 4u : kBufferOutOfRange, 0, 0);
    };
    request_positions(wave_t0);
    request_rows(wave_t0, 0);
    // gate arithmetic (layers.py:343-365) of one of a lane's four tokens of a
    // finished tile -> (a, scaled input) in LDS.  It runs a tile late, between
    // the matrix instructions of the tile after.
    // Two sets of accumulators, used by the tiles in turn: while one collects
    // a tile, the gate arithmetic reads the other (for a wave's first tile it
    // works on zeros and writes into that tile's own slots, which the real
    // values overwrite a tile later: no branch between matrix instructions).
    f32x4 acc_x[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    f32x4 acc_a[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
    uint64_t pend_starts = 0;
    int pend_t0 = wave_t0;
    auto gate_element = [&](int q, const f32x4& pend_x, const f32x4& pend_a) {
      const int r = 4 * g + q;
      const int t = pend_t0 + r;
      // (the hardware's exp2, reciprocal and square root, about 1 ulp each,
      // where the other float32 kernels call expf, divide and call sqrtf: a
      // quarter of the instructions; an argument's rounding before exp2
      // costs |argument| x 6e-8 of relative error where the result is far
      // from 1 and nothing where it is near: two orders of magnitude inside
      // the 1e-5 bar)
      const float gate_x =
          __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * pend_x[q]));
      const float gate_a =
          __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * pend_a[q]));
      const float log2_a = gate_a * decay2;
      float a = __builtin_amdgcn_exp2f(log2_a);
      float mult = __builtin_amdgcn_sqrtf(
          1.0f - __builtin_amdgcn_exp2f(log2_a + log2_a));
      if ((pend_starts >> (r + 2)) & 1u) {  // document start: forget the state
        a = 0.0f;
        mult = 1.0f;
      }
      float xn = (lds.own[wave][r][n] * gate_x) * mult;
      if (t >= T) {  // past the end: identity
        a = 1.0f;
        xn = 0.0f;
      }
      const int slot = gate_slot(t - seg * kSeg);
      lds.a[slot][n] = a;
      lds.xn[slot][n] = xn;
    };
    auto one_tile = [&](int tile, auto parity) {
      constexpr int cur = decltype(parity)::value;
      const int t0 = wave_t0 + tile * kTile;  // first token of the tile
      // document starts among rows t0-2 .. t0+15 (rows before the sequence or
      // past its end: no start)
      uint64_t starts;
      {
        const int t = t0 - 2 + lane;
        const bool in = lane < kTile + 2 && t >= 0 && t < T;
        starts = __ballot(in && (seg_lo | seg_hi) == 0u);
      }
      // both gates' pre-activations of tokens t0 .. t0+15, channels c0 .. +15:
      // lane (g, n) ends up with channel n of tokens 4 g .. 4 g + 3
      acc_x[cur] = f32x4{bias_x, bias_x, bias_x, bias_x};
      acc_a[cur] = f32x4{bias_a, bias_a, bias_a, bias_a};
      // the conv output of the workgroup's own 16 channels, which the gate
      // arithmetic multiplies: from the staged half they are in to a place
      // that lasts until the next tile
      auto copy_own = [&]() {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          lds.own[wave][4 * g + q][n] = lds.stage[wave][4 * g + q][own_col];
      };
      static_for<0, 2>([&](auto hc) {
        constexpr int hh = decltype(hc)::value;
        // conv of this half's 128 channels -> LDS.  Tap k of row r reads row
        // r - k, which counts only if no document starts in rows r-k+1 .. r
        // (bit j of `starts` is row j - 2).
        if (hh == 1 && own_half == 0) copy_own();  // still the first half's
        auto row = [&](int r) -> f32x2 { return xr[r + 3]; };
        f32x2 cw[4], cb;
        if (has_conv) {
#pragma unroll
          for (int k = 0; k < 4; ++k) cw[k] = lds.taps[hh][k][lane];
          cb = lds.taps[hh][4][lane];
        }
        if (__builtin_expect(starts == 0, 1)) {
#pragma unroll
          for (int r = 0; r < kTile; ++r) {
            f32x2 o;
#pragma unroll
            for (int e = 0; e < 2; ++e)
              o[e] = has_conv ? conv4(row(r)[e], row(r - 1)[e], row(r - 2)[e],
                                      row(r - 3)[e], cw[0][e], cw[1][e],
                                      cw[2][e], cw[3][e], cb[e])
                              : row(r)[e];
            *reinterpret_cast<f32x2*>(&lds.stage[wave][r][2 * lane]) = o;
          }
        } else {
#pragma unroll
          for (int r = 0; r < kTile; ++r) {
            const uint32_t near = (uint32_t)(starts >> r) & 7u;  // rows r-2, r-1, r
            const bool cut1 = (near & 4u) != 0;          // start at r
            const bool cut2 = cut1 || (near & 2u) != 0;  // ... or at r-1
            const bool cut3 = cut2 || (near & 1u) != 0;  // ... or at r-2
            f32x2 o;
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const float x0 = row(r)[e];
              const float x1 = cut1 ? 0.0f : row(r - 1)[e];
              const float x2 = cut2 ? 0.0f : row(r - 2)[e];
              const float x3 = cut3 ? 0.0f : row(r - 3)[e];
              o[e] = has_conv ? conv4(x0, x1, x2, x3, cw[0][e], cw[1][e],
                                      cw[2][e], cw[3][e], cb[e])
                              : x0;
            }
            *reinterpret_cast<f32x2*>(&lds.stage[wave][r][2 * lane]) = o;
          }
        }
        // (the rows are consumed: ask for the next pass's now, not earlier:
        // their registers are the same)
        __builtin_amdgcn_sched_barrier(0);
        if (hh == 0) {
          request_rows(t0, 1);
        } else if (tile + 1 < kTilesPerWave) {
          request_rows(t0 + kTile, 0);
          request_positions(t0 + kTile);
        }
        __builtin_amdgcn_wave_barrier();
        // the conv output of the workgroup's own channels, for the gates
        // (in the second pass: the gate arithmetic of the tile before, which
        // sits in the first, has read its own by then)
        if (hh == 1 && own_half == 1) copy_own();
        // A lane's A values are read one group of four k-steps ahead and the
        // groups are kept apart (left to itself the compiler reads each
        // group's values right before their first use and waits for the LDS
        // once per group); the gate arithmetic of the tile before sits between
        // the groups of the first pass.
        f32x4 av = *reinterpret_cast<const f32x4*>(&lds.stage[wave][n][4 * g]);
        static_for<0, 8>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          f32x4 av_next = av;
          if (i + 1 < 8)
            av_next = *reinterpret_cast<const f32x4*>(
                &lds.stage[wave][n][16 * (i + 1) + 4 * g]);
          constexpr int base = 4 * (8 * hh + i);
#pragma unroll
          for (int q = 0; q < 3; ++q) {
            mfma_weight(av[q], wx[base + q], acc_x[cur]);
            mfma_weight(av[q], wa[base + q], acc_a[cur]);
          }
          if constexpr (hh == 1 && i == 7) {
            mfma_weight_last(av[3], wx[base + 3], wa[base + 3], acc_x[cur],
                             acc_a[cur]);
          } else {
            mfma_weight(av[3], wx[base + 3], acc_x[cur]);
            mfma_weight(av[3], wa[base + 3], acc_a[cur]);
          }
          if (hh == 0 && (i & 1) == 1)
            gate_element(i >> 1, acc_x[cur ^ 1], acc_a[cur ^ 1]);
          av = av_next;
          __builtin_amdgcn_sched_barrier(0);
        });
        __builtin_amdgcn_wave_barrier();
      });
      // this tile's gate arithmetic waits for the next tile's matrix stage
      pend_starts = starts;
      pend_t0 = t0;
    };
    static_assert(kTilesPerWave % 2 == 0, "tiles alternate between two sets");
#pragma unroll 1
    for (int tile = 0; tile < kTilesPerWave; tile += 2) {
      one_tile(tile, std::integral_constant<int, 0>{});
      one_tile(tile + 1, std::integral_constant<int, 1>{});
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      gate_element(q, acc_x[1], acc_a[1]);  // the last tile's
    __syncthreads();

    // ---- stage 2: the recurrence over the segment, 32 chunks per channel ----
    {
      const int ch = tid & (kCh - 1);
      const int chunk = tid >> 4;
      const int i0 = chunk * kChunk;
      {
        float pp = 1.0f, hh = 0.0f;
#pragma unroll
        for (int i = 0; i < kChunk; ++i) {
          const float a = lds.a[gate_slot(i0 + i)][ch];
          hh = __builtin_fmaf(a, hh, lds.xn[gate_slot(i0 + i)][ch]);
          pp *= a;
        }
        lds.chunk_p[chunk][ch] = pp;
        lds.chunk_h[chunk][ch] = hh;
      }
      __syncthreads();
      // The state every chunk starts from: a scan over the 32 chunk summaries
      // with the operator of recurrentgemma/jax/scan.py:161-187, by lane
      // shifts inside a wave (lane = 2 chunk + channel; a wave takes 2 of the
      // 16 channels), left where the chunk's own summary was.
      {
        const int sc = lane >> 1;               // chunk
        const int sch = 2 * wave + (lane & 1);  // channel
        float sp = lds.chunk_p[sc][sch], sh = lds.chunk_h[sc][sch];
#pragma unroll
        for (int d = 1; d < kChunks; d *= 2) {
          const float pp = __shfl_up(sp, 2 * d, 64);
          const float hp = __shfl_up(sh, 2 * d, 64);
          if (sc >= d) {
            sh = __builtin_fmaf(sp, hp, sh);
            sp *= pp;
          }
        }
        // (sp, sh): chunks 0 .. sc from a zero state; the state after chunk sc
        // is sp * carry + sh, and chunk sc starts from its neighbour's
        const float carry = lds.carry[sch];
        const float after = __builtin_fmaf(sp, carry, sh);
        const float before = __shfl_up(after, 2, 64);
        lds.chunk_h[sc][sch] = sc == 0 ? carry : before;
        if (sc == kChunks - 1) lds.carry[sch] = after;
      }
      __syncthreads();
      float hin = lds.chunk_h[chunk][ch];
      const int64_t y_at = ((int64_t)b * T + seg * kSeg + i0) * W + c0 + ch;
      float* y = (float*)p.y + y_at;
      const int left = T - (seg * kSeg + i0);
      float other[kChunk];  // GELU: the other branch at this thread's tokens
      if (GELU) {
        const float* gb = (const float*)p.gate_branch + y_at;
#pragma unroll
        for (int i = 0; i < kChunk; ++i)
          other[i] = i < left ? gb[(int64_t)i * W] : 0.0f;
      }
#pragma unroll
      for (int i = 0; i < kChunk; ++i) {
        hin = __builtin_fmaf(lds.a[gate_slot(i0 + i)][ch], hin,
                             lds.xn[gate_slot(i0 + i)][ch]);
        if (i < left)
          y[(int64_t)i * W] = GELU ? gelu_mul_f32(hin, other[i]) : hin;
      }
    }
    __syncthreads();  // a, xn and the chunk states are free again
  }

  if (p.h_last && tid < kCh) p.h_last[(int64_t)b * W + c0 + tid] = lds.carry[tid];

  // Masked conv state: rows T-3..T-1 of x, each zeroed if a document starts in
  // a later position of the row; rows before the sequence start are zero.
  if (p.cache_out && tid < kCh) {
    float* cache = (float*)p.cache_out + (int64_t)b * 3 * W + c0 + tid;
    bool later_start = false;
#pragma unroll
    for (int kk = 2; kk >= 0; --kk) {
      const int t = T - 3 + kk;
      float v = 0.0f;
      if (t >= 0 && !later_start)
        v = ((const float*)p.x)[((int64_t)b * T + t) * W + c0 + tid];
      cache[(int64_t)kk * W] = v;
      if (t >= 0 && is_doc_start(p.segpos, p.seg_kind, (int64_t)b * T + t))
        later_start = true;
    }
  }
}

}  // namespace

// Shapes this kernel is for: float32, 256-wide heads, at most 32 (row, head)
// pairs (16 workgroups each), rows that fit 31-bit byte offsets.
bool core_f32_small_serves(int B, int T, int W, int H) {
  return W % H == 0 && W / H == kBW && (int64_t)B * H <= 32 &&
         (int64_t)T * W * 4 < (int64_t)0x7fffffff;
}

template <bool HAS_CONV, bool GELU>
static hipError_t launch_core_f32_small_as(const FusedArgs& a, dim3 grid,
                                           hipStream_t s) {
  static OncePerDevice once;
  hipError_t e = set_max_dynamic_lds(
      once, (const void*)core_f32_small_kernel<HAS_CONV, GELU>,
      (int)sizeof(CoreF32Lds));
  if (e != hipSuccess) return e;
  core_f32_small_kernel<HAS_CONV, GELU>
      <<<grid, kThreads, sizeof(CoreF32Lds), s>>>(a);
  return hipGetLastError();
}

hipError_t launch_core_f32_small(const FusedArgs& a, hipStream_t s) {
  const int rounds = (a.B * a.H + 7) / 8;
  const dim3 grid((unsigned)(rounds * 8 * (kBW / kCh)));
  if (a.conv_w)
    return a.gate_branch ? launch_core_f32_small_as<true, true>(a, grid, s)
                         : launch_core_f32_small_as<true, false>(a, grid, s);
  return a.gate_branch ? launch_core_f32_small_as<false, true>(a, grid, s)
                       : launch_core_f32_small_as<false, false>(a, grid, s);
}

}  // namespace rg
