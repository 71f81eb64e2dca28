// The recurrent core of a short float32 prefill in ONE launch (256-wide
// heads, few rows): width-4 conv -> both gate projections on the float32
// matrix instruction -> gate activations -> recurrence.
//
// The three-launch form (gate GEMM, then the scan in two passes over chunks of
// the sequence) spends most of a small call waiting for launches and for each
// kernel's first loads.  Here one workgroup of four waves owns 16 channels of
// one head of one row for the whole sequence: 16 B x H workgroups.  Per
// segment of 512 tokens each wave takes 128 of them in tiles of 16: the
// head's 256 input channels of a tile are loaded, convolved and staged in LDS
// (every workgroup of a head convolves the same rows again: the conv is 4
// multiply-adds per element), 128 v_mfma_f32_16x16x4_f32 against the wave's
// resident weights (256 x 16 per gate: 128 registers) give the
// pre-activations of the 16 channels, the gate arithmetic leaves (a, a-scaled
// input) per token and channel in LDS; then the workgroup scans the segment as
// 16 chunks of 32 tokens per channel (local scan, fold of the chunks before,
// replay) and stores y.
//
// True float32 products and sums (no reduced-precision operand formats): the
// float32 bar of 1e-5 stands (measured against the gate GEMM + scan pair:
// 2e-7 .. 6e-7 of the largest output, conv state identical).  Same conv4() tap
// chain and expf as the other float32 kernels; the reciprocal and the square
// root of the gate arithmetic are the hardware's.
//
// Where the time goes (B1 T512 W2560, 160 workgroups, 42 us): a tile of 16
// tokens takes a wave about 10 000 cycles -- 128 matrix instructions at 32
// cycles, the conv 1 600, the gate arithmetic 1 500, operand reads, loads and
// bookkeeping 2 500 -- one after the other: a wave issues in order and the
// compiler's schedule does not put the vector work between the matrix
// instructions.  Eight waves of one tile each per 128-token segment (two per
// SIMD) were slower (256 registers: spills, and four times the barriers).
//
// Replaces the chain Conv1D.forward -> RGLRU.forward of
// recurrentgemma/torch/modules.py:632-643 (layers.py:447-529, 313-365,
// 140-191) for such shapes.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;      // head width
constexpr int kCh = 16;       // output channels per workgroup
constexpr int kTile = 16;     // tokens per matrix tile
constexpr int kSeg = 512;     // tokens per segment
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int kTilesPerWave = kSeg / kWaves / kTile;  // 8
constexpr int kStageStride = kBW + 4;                 // floats per staged row
constexpr int kChunk = 32;                            // tokens per scan chunk
constexpr int kChunks = kSeg / kChunk;                // 16

struct CoreF32Lds {
  float stage[kWaves][kTile][kStageStride];  // conv output of a wave's tile
  float a[kSeg][kCh];                        // per token and channel: a_t
  float xn[kSeg][kCh];                       // ... and the scaled input
  float chunk_p[kChunks][kCh];               // product of a over a chunk
  float chunk_h[kChunks][kCh];               // its state from a zero start
  float carry[kCh];                          // state at the segment's start
};

template <bool HAS_CONV>
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

  // ---- weights of the wave: B operand of v_mfma_f32_16x16x4_f32, lane (g, n)
  //      holds W[k][n] for the k of its group.  The k of a matrix instruction
  //      are chosen so that a lane's A values of four instructions are four
  //      consecutive floats of its staged row: instruction (i, q) multiplies
  //      k = 16 i + 4 g' + q, g' = 0..3.
  float bx[64], ba[64];
  {
    const float* wx = (const float*)p.w[0] + (int64_t)h * kBW * kBW + s * kCh + n;
    const float* wa = (const float*)p.w[1] + (int64_t)h * kBW * kBW + s * kCh + n;
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = 16 * i + 4 * g + q;
        bx[4 * i + q] = wx[(int64_t)k * kBW];
        ba[4 * i + q] = wa[(int64_t)k * kBW];
      }
  }
  const float bias_x = ((const float*)p.b[0])[c0 + n];
  const float bias_a = ((const float*)p.b[1])[c0 + n];
  const float decay = softplus_precise(((const float*)p.a_param)[c0 + n]);

  // conv taps of this lane's four input channels (4 lane .. 4 lane + 3 of the
  // head); without conv weights x is the conv output already
  constexpr bool has_conv = HAS_CONV;
  f32x4 cw0 = {0, 0, 0, 0}, cw1 = cw0, cw2 = cw0, cw3 = {1, 1, 1, 1}, cb = cw0;
  if (has_conv) {
    const float* cw = (const float*)p.conv_w + c_head + 4 * lane;
    cw0 = *reinterpret_cast<const f32x4*>(cw);
    cw1 = *reinterpret_cast<const f32x4*>(cw + W);
    cw2 = *reinterpret_cast<const f32x4*>(cw + 2 * W);
    cw3 = *reinterpret_cast<const f32x4*>(cw + 3 * W);
    cb = *reinterpret_cast<const f32x4*>((const float*)p.conv_b + c_head +
                                         4 * lane);
  }

  const uint32_t row_bytes = 4u * (uint32_t)W;
  const uint32_t seq_bytes = (uint32_t)T * row_bytes;  // < 2^31 (launcher)
  const __amdgpu_buffer_rsrc_t rx =
      make_rsrc((const char*)p.x + (int64_t)b * seq_bytes, seq_bytes);
  const bool seg_is64 = p.seg_kind == kSegI64;
  const uint32_t seg_esize = seg_is64 ? 8u : 4u;
  const __amdgpu_buffer_rsrc_t rseg =
      make_rsrc((const char*)p.segpos + (int64_t)b * T * seg_esize,
                (uint32_t)T * seg_esize);

  if (tid < kCh)
    lds.carry[tid] = p.h0 ? p.h0[(int64_t)b * W + c0 + tid] : 0.0f;

  const int nseg = (T + kSeg - 1) / kSeg;
  for (int seg = 0; seg < nseg; ++seg) {
    // ---- stage 1: this wave's 128 tokens of the segment, a tile at a time --
    const int wave_t0 = seg * kSeg + wave * (kSeg / kWaves);
    // Rows t0-3 .. t0+15 of the head's 256 channels, four per lane (rows
    // outside the sequence fall outside the descriptor: zeros), and the
    // positions of rows t0-2 .. t0+15 (lane j looks at row t0 - 2 + j).  The
    // loads of a tile are issued while the tile before it is multiplied.
    f32x4 xr[kTile + 3];
    uint32_t seg_lo = 1, seg_hi = 0;
    auto request_tile = [&](int t0, bool first) {
      {
        const int t = t0 - 2 + lane;
        const bool in = lane < kTile + 2 && t >= 0 && t < T;
        const uint32_t off = in ? (uint32_t)t * seg_esize : kBufferOutOfRange;
        seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
        seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
            rseg, seg_is64 ? off + 4u : kBufferOutOfRange, 0, 0);
      }
      // (the three rows before the tile: loaded for a wave's first tile, the
      // last three rows of the tile before otherwise)
#pragma unroll
      for (int r = 0; r < kTile + 3; ++r) {
        if (r < 3 && !first) {
          xr[r] = xr[r + kTile];
          continue;
        }
        const int t = t0 - 3 + r;
        const uint32_t off =
            t >= 0 ? (uint32_t)t * row_bytes + 4u * (uint32_t)(c_head + 4 * lane)
                   : kBufferOutOfRange;
        xr[r] = __builtin_bit_cast(
            f32x4, __builtin_amdgcn_raw_buffer_load_b128(rx, off, 0, 0));
      }
    };
    request_tile(wave_t0, true);
    // gate arithmetic (layers.py:343-365) of one of a lane's four tokens of a
    // finished tile -> (a, scaled input) in LDS.  It runs a tile late, between
    // the matrix instructions of the tile after.
    f32x4 pend_x = {0, 0, 0, 0}, pend_a = {0, 0, 0, 0};
    float pend_xc[4] = {0, 0, 0, 0};
    uint64_t pend_starts = 0;
    int pend_t0 = wave_t0;
    auto gate_element = [&](int q) {
      const int r = 4 * g + q;
      const int t = pend_t0 + r;
      // (expf as everywhere in float32; the reciprocal and the square root are
      // the hardware's, 1 ulp, where the other float32 kernels divide and
      // call sqrtf: 70 fewer instructions per element, and the difference is
      // two orders of magnitude inside the 1e-5 bar)
      const float gate_x = __builtin_amdgcn_rcpf(1.0f + expf(-pend_x[q]));
      const float gate_a = __builtin_amdgcn_rcpf(1.0f + expf(-pend_a[q]));
      const float log_a = (-8.0f * gate_a) * decay;
      float a = expf(log_a);
      float mult = __builtin_amdgcn_sqrtf(1.0f - expf(2.0f * log_a));
      if ((pend_starts >> (r + 2)) & 1u) {  // document start: forget the state
        a = 0.0f;
        mult = 1.0f;
      }
      float xn = (pend_xc[q] * gate_x) * mult;
      if (t >= T) {  // past the end: identity
        a = 1.0f;
        xn = 0.0f;
      }
      lds.a[t - seg * kSeg][n] = a;
      lds.xn[t - seg * kSeg][n] = xn;
    };
#pragma unroll 1
    for (int tile = 0; tile < kTilesPerWave; ++tile) {
      const int t0 = wave_t0 + tile * kTile;  // first token of the tile
      // document starts among rows t0-2 .. t0+15 (rows before the sequence or
      // past its end: no start)
      uint64_t starts;
      {
        const int t = t0 - 2 + lane;
        const bool in = lane < kTile + 2 && t >= 0 && t < T;
        starts = __ballot(in && (seg_lo | seg_hi) == 0u);
      }
      // conv -> LDS.  Tap k of row r reads row r - k, which counts only if no
      // document starts in rows r-k+1 .. r (bit j of `starts` is row j - 2).
      if (__builtin_expect(starts == 0, 1)) {
#pragma unroll
        for (int r = 0; r < kTile; ++r) {
          f32x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o[e] = has_conv ? conv4(xr[r + 3][e], xr[r + 2][e], xr[r + 1][e],
                                    xr[r][e], cw0[e], cw1[e], cw2[e], cw3[e],
                                    cb[e])
                            : xr[r + 3][e];
          *reinterpret_cast<f32x4*>(&lds.stage[wave][r][4 * lane]) = o;
        }
      } else {
#pragma unroll
        for (int r = 0; r < kTile; ++r) {
          const uint32_t near = (uint32_t)(starts >> r) & 7u;  // rows r-2, r-1, r
          const bool cut1 = (near & 4u) != 0;          // start at r
          const bool cut2 = cut1 || (near & 2u) != 0;  // ... or at r-1
          const bool cut3 = cut2 || (near & 1u) != 0;  // ... or at r-2
          f32x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float x0 = xr[r + 3][e];
            const float x1 = cut1 ? 0.0f : xr[r + 2][e];
            const float x2 = cut2 ? 0.0f : xr[r + 1][e];
            const float x3 = cut3 ? 0.0f : xr[r][e];
            o[e] = has_conv ? conv4(x0, x1, x2, x3, cw0[e], cw1[e], cw2[e],
                                    cw3[e], cb[e])
                            : x0;
          }
          *reinterpret_cast<f32x4*>(&lds.stage[wave][r][4 * lane]) = o;
        }
      }
      // (the rows are consumed: ask for the next tile's now)
      if (tile + 1 < kTilesPerWave) request_tile(t0 + kTile, false);
      __builtin_amdgcn_wave_barrier();
      // both gates' pre-activations of tokens t0 .. t0+15, channels c0 .. +15:
      // lane (g, n) ends up with channel n of tokens 4 g .. 4 g + 3.  A lane's
      // A values are read one group of four k-steps ahead and the groups are
      // kept apart (left to itself the compiler reads each group's values
      // right before their first use and waits for the LDS 16 times a tile);
      // the gate arithmetic of the tile before sits in four of the groups (for
      // the first tile it works on zeros and writes into the tile's own
      // slots, which its real values overwrite a tile later: no branch
      // between the matrix instructions).
      f32x4 acc_x = {bias_x, bias_x, bias_x, bias_x};
      f32x4 acc_a = {bias_a, bias_a, bias_a, bias_a};
      f32x4 av = *reinterpret_cast<const f32x4*>(&lds.stage[wave][n][4 * g]);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        f32x4 av_next = av;
        if (i + 1 < 16)
          av_next = *reinterpret_cast<const f32x4*>(
              &lds.stage[wave][n][16 * (i + 1) + 4 * g]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc_x = __builtin_amdgcn_mfma_f32_16x16x4f32(av[q], bx[4 * i + q],
                                                       acc_x, 0, 0, 0);
          acc_a = __builtin_amdgcn_mfma_f32_16x16x4f32(av[q], ba[4 * i + q],
                                                       acc_a, 0, 0, 0);
        }
        if ((i & 3) == 1) gate_element(i >> 2);
        av = av_next;
        __builtin_amdgcn_sched_barrier(0);
      }
      // this tile's gate arithmetic waits for the next tile's matrix stage
      pend_x = acc_x;
      pend_a = acc_a;
      pend_starts = starts;
      pend_t0 = t0;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        pend_xc[q] = lds.stage[wave][4 * g + q][s * kCh + n];
      __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) gate_element(q);  // the last tile's
    __syncthreads();

    // ---- stage 2: the recurrence over the segment, 16 chunks per channel ----
    {
      const int ch = tid & (kCh - 1);
      const int chunk = tid >> 4;
      const bool active = chunk < kChunks;
      const int i0 = chunk * kChunk;
      if (active) {
        float pp = 1.0f, hh = 0.0f;
#pragma unroll
        for (int i = 0; i < kChunk; ++i) {
          const float a = lds.a[i0 + i][ch];
          hh = __builtin_fmaf(a, hh, lds.xn[i0 + i][ch]);
          pp *= a;
        }
        lds.chunk_p[chunk][ch] = pp;
        lds.chunk_h[chunk][ch] = hh;
      }
      __syncthreads();
      float hin = 0.0f;
      if (active) {
        // state at the start of this chunk: fold the chunks before it (the
        // scan operator of recurrentgemma/jax/scan.py:161-187)
        hin = lds.carry[ch];
        for (int k = 0; k < chunk; ++k)
          hin = __builtin_fmaf(lds.chunk_p[k][ch], hin, lds.chunk_h[k][ch]);
        float* y = (float*)p.y + ((int64_t)b * T + seg * kSeg + i0) * W + c0 + ch;
        const int left = T - (seg * kSeg + i0);
#pragma unroll
        for (int i = 0; i < kChunk; ++i) {
          hin = __builtin_fmaf(lds.a[i0 + i][ch], hin, lds.xn[i0 + i][ch]);
          if (i < left) y[(int64_t)i * W] = hin;
        }
      }
      __syncthreads();  // every thread has read the carry and the summaries
      if (chunk == kChunks - 1) lds.carry[ch] = hin;
    }
    __syncthreads();
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

hipError_t launch_core_f32_small(const FusedArgs& a, hipStream_t s) {
  const int rounds = (a.B * a.H + 7) / 8;
  const dim3 grid((unsigned)(rounds * 8 * (kBW / kCh)));
  if (a.conv_w) {
    static OncePerDevice once;
    hipError_t e = set_max_dynamic_lds(
        once, (const void*)core_f32_small_kernel<true>, (int)sizeof(CoreF32Lds));
    if (e != hipSuccess) return e;
    core_f32_small_kernel<true><<<grid, kThreads, sizeof(CoreF32Lds), s>>>(a);
  } else {
    static OncePerDevice once;
    hipError_t e = set_max_dynamic_lds(
        once, (const void*)core_f32_small_kernel<false>, (int)sizeof(CoreF32Lds));
    if (e != hipSuccess) return e;
    core_f32_small_kernel<false><<<grid, kThreads, sizeof(CoreF32Lds), s>>>(a);
  }
  return hipGetLastError();
}

}  // namespace rg
