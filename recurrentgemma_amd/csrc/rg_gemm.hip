// Block-diagonal gate projections (BlockDiagonalLinear) for gfx950.
//
// Two kernels:
//  * gates_mfma_bf16_kernel: bf16, block width 256.  Weight-stationary: each of
//    the 8 waves of a workgroup keeps a 256(K) x 64(N) slice of the two gates'
//    weights ([W_x | W_a], N = 512) in registers as MFMA B fragments for the
//    whole kernel and the group walks over 64-row tiles of x, staged (and
//    optionally convolved) through double-buffered LDS.  fp32 accumulation on
//    v_mfma_f32_32x32x16_bf16, bias added in fp32, one rounding to bf16.
//  * bdl_generic_kernel: any dtype / block width, LDS-tiled FMA with fp32
//    accumulation (used for fp32 and for block widths other than 256).
#include "rg_common.h"
#include "rg_internal.h"

#include <type_traits>

namespace rg {
namespace {

// ===================================================== generic FMA kernel ==

constexpr int kGT = 64;  // output tile edge
constexpr int kGK = 16;  // K chunk

template <typename T, bool CONV>
__global__ void __launch_bounds__(256) bdl_generic_kernel(GemmArgs p) {
  __shared__ float As[kGK][kGT + 4];
  __shared__ float Bs[kGK][kGT + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int z = blockIdx.z;
  const int gate = z / p.H;
  const int h = z - gate * p.H;
  const int bw = p.bw;
  const int64_t m0 = (int64_t)blockIdx.x * kGT;
  const int n0 = blockIdx.y * kGT;
  const T* x = (const T*)p.x;
  const T* w = (const T*)p.w[gate] + (int64_t)h * bw * bw;
  const T* bias = (const T*)p.b[gate] + (int64_t)h * bw;
  T* out = (T*)p.out[gate];

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;

  for (int k0 = 0; k0 < bw; k0 += kGK) {
#pragma unroll
    for (int e = tid; e < kGT * kGK; e += 256) {
      const int r = e / kGK, kk = e % kGK;
      const int64_t m = m0 + r;
      float v = 0.0f;
      if (m < p.M && k0 + kk < bw) {
        const int c = h * bw + k0 + kk;
        if (CONV)
          v = conv_point<T>(x, p.segpos, p.seg_kind, (const T*)p.conv_w,
                            (const T*)p.conv_b, p.T, p.W, 4, m, c);
        else
          v = load_scalar(x + m * p.W + c);
      }
      As[kk][r] = v;
    }
#pragma unroll
    for (int e = tid; e < kGT * kGK; e += 256) {
      const int kk = e / kGT, n = e % kGT;
      float v = 0.0f;
      if (k0 + kk < bw && n0 + n < bw)
        v = load_scalar(w + (int64_t)(k0 + kk) * bw + n0 + n);
      Bs[kk][n] = v;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kGK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = Bs[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty * 4 + i;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < bw)
        store_scalar(out + m * p.W + h * bw + n,
                     acc[i][j] + load_scalar(bias + n));
    }
  }
}

// ======================================================= bf16 MFMA kernel ==

constexpr int kBW = 256;          // block width (K and per-gate N)
constexpr int kTM = 64;           // rows of x per tile
constexpr int kLdsStride = 264;   // bf16 elements per LDS row (256 + 8 pad)
constexpr int kRowsPerGroup = 16; // rows each thread converts per tile
constexpr size_t kStageLdsBytes = 2ull * kTM * kLdsStride * sizeof(uint16_t);
// Per-wave output staging: one 32 x 64 result block in bf16, rows padded to
// 144 bytes so that the 16-byte row reads stay aligned.
constexpr int kEpiStride = 144;
constexpr size_t kEpiBytesPerWave = 32ull * kEpiStride;
constexpr size_t kBiasLdsOffset = kStageLdsBytes + 8 * kEpiBytesPerWave;
constexpr size_t kMfmaLdsBytes = kBiasLdsOffset + 8 * 64 * sizeof(float);

union Frag {
  bf16x8 v;
  uint16_t u[8];
  f32x4 q;
};

// ONE: a single matrix (p.w[0], p.b[0], p.out[0]).  Waves 0-3 then do all of
// the matrix work; waves 4-7 only take their share of the x staging (the
// staging loops are laid out for 512 threads), issue no matrix instruction
// and store through an empty descriptor.
// NARROW: heads narrower than the tile (bw < 256); the waves whose columns
// and the k-steps whose rows are all padding issue no matrix instruction.
template <bool CONV, bool ONE = false, bool NARROW = false>
__global__ void __launch_bounds__(512) gates_mfma_bf16_kernel(GemmArgs p) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(lds_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = blockIdx.y;
  const int64_t M = p.M;
  const int64_t W = p.W;
  const int T_len = p.T;
  const int bw = p.bw;  // 8 .. 256, a multiple of 8 (the launcher checks)
  const int64_t ntiles = (M + kTM - 1) / kTM;

  // ---- this wave's weight slice, resident in registers -----------------
  const int gate = ONE ? 0 : wave >> 2;  // waves 0-3: input gate, 4-7: a gate
  // (wave-uniform; n0 and bw come further down)
  const bool active = (!ONE || wave < 4) &&
                      (!NARROW || (wave & 3) * 64 < p.bw);
  const int ksteps = NARROW ? (p.bw + 15) / 16 : 16;  // k-steps with a row < bw
  const int n0 = (wave & 3) * 64;     // first output column inside the gate
  // The weights are [k][n] with n contiguous, the MFMA B operand wants 8
  // consecutive k per lane: transpose through LDS, 128 k-rows of one gate at
  // a time (coalesced 16-byte global reads, 2-byte LDS reads).
  Frag bfrag[16][2];
#pragma unroll
  for (int g = 0; g < (ONE ? 1 : 2); ++g) {
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      // (a head narrower than the 256 x 256 tile -- bw a multiple of 8 --
      // is padded with zeros: rows and columns from bw on)
      const uint16_t* src =
          (const uint16_t*)p.w[g] + ((int64_t)h * bw + kh * 128) * bw;
      for (int e = tid; e < 128 * 32; e += 512) {
        const int r = e >> 5, q = e & 31;
        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (kh * 128 + r < bw && q * 8 < bw)
          v = *reinterpret_cast<const f32x4*>(src + (size_t)r * bw + q * 8);
        *reinterpret_cast<f32x4*>(lds + (size_t)r * kLdsStride + q * 8) = v;
      }
      __syncthreads();
      if (gate == g) {
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
#pragma unroll
          for (int nt = 0; nt < 2; ++nt) {
            const int n = n0 + nt * 32 + (lane & 31);
            const int kb = ks * 16 + 8 * (lane >> 5);
#pragma unroll
            for (int e = 0; e < 8; ++e)
              bfrag[kh * 8 + ks][nt].u[e] = lds[(size_t)(kb + e) * kLdsStride + n];
          }
      }
      __syncthreads();
    }
  }
  // The MFMAs compute the transposed block (weights as the A operand): lane l
  // then holds, for x row l%32, the channels 8*g + 4*(l/32) + 0..3 of each
  // 32-channel block, g = 0..3, i.e. four adjacent channels per register
  // quad.  The accumulators start from the bias, which each wave keeps in LDS
  // as 64 floats (one 16-byte read per quad).
  float* const bias_lds =
      reinterpret_cast<float*>(lds_raw + kBiasLdsOffset) + wave * 64;
  bias_lds[lane] =
      n0 + lane < bw
          ? bf16_bits_to_f32(((const uint16_t*)p.b[gate])[h * bw + n0 + lane])
          : 0.0f;
  const float* const bias_r = bias_lds + 4 * (lane >> 5);
  // Output addressing: a wave-uniform tile pointer plus this 32-bit lane
  // offset.  Lane l stores the 16-byte chunk l%8 of rows l/8, l/8+8, ... of
  // the wave's 32 x 64 block.
  const uint32_t out_row_bytes = 2u * (uint32_t)p.W;
  // (a chunk of columns from bw on belongs to the next head: never stored)
  const uint32_t out_lane_bytes =
      n0 + 8 * (lane & 7) < bw
          ? (uint32_t)(lane >> 3) * out_row_bytes + 2u * (h * bw + n0) +
                16u * (lane & 7)
          : kBufferOutOfRange;
  unsigned char* const epi =
      lds_raw + kStageLdsBytes + (size_t)wave * kEpiBytesPerWave;
  // write side: x row lane%32, channels 4*(lane/32) + 8*g (+ 32)
  unsigned char* const epi_w =
      epi + (lane & 31) * kEpiStride + 8 * (lane >> 5);
  unsigned char* const epi_r = epi + (lane >> 3) * kEpiStride + 16 * (lane & 7);
  char* const outbase = (char*)p.out[gate];

  // ---- x staging: thread -> (channel pair, group of 16 rows) -----------
  const int cp = tid & 127;
  const int rg = __builtin_amdgcn_readfirstlane(tid >> 7);
  const uint32_t c = h * bw + cp * 2;  // lane offset inside a row of x
  const bool c_valid = cp * 2 < bw;    // else: the tile's zero padding
  // (out of range by itself and together with an out-of-range scalar offset:
  // the sum of two kBufferOutOfRange would wrap around to a valid address)
  const uint32_t c_bytes = c_valid ? 2u * c : kBufferOutOfRange / 2;
  const uint16_t* const xbase = (const uint16_t*)p.x;
  const uint32_t x_row_bytes = 2u * (uint32_t)p.W;
  constexpr int kHalo = CONV ? 3 : 0;
  constexpr int kRaw = kRowsPerGroup + kHalo;
  uint32_t cwp[5] = {0, 0, 0, 0, 0};  // conv w[0..3] and bias, two bf16 each
  if (CONV && c_valid) {
    const uint16_t* cw = (const uint16_t*)p.conv_w + c;
    cwp[0] = *reinterpret_cast<const uint32_t*>(cw);
    cwp[1] = *reinterpret_cast<const uint32_t*>(cw + W);
    cwp[2] = *reinterpret_cast<const uint32_t*>(cw + 2 * W);
    cwp[3] = *reinterpret_cast<const uint32_t*>(cw + 3 * W);
    cwp[4] = *reinterpret_cast<const uint32_t*>((const uint16_t*)p.conv_b + c);
  }
  uint32_t raw[kRaw];
  // Document-start lookup of the tile being fetched: lane j of the wave looks
  // at row mbase+j (all lanes of a wave stage the same rows).  Two
  // unconditional 32-bit buffer loads (low and high half of an int64
  // position; for int32 positions the high half is sent out of range and
  // reads as zero), tested a tile later in stage_begin(): a position is a
  // start iff both halves are zero.  Lanes without a row read out of range
  // and are masked in the test.
  uint32_t seg_lo = 1, seg_hi = 0;
  const bool seg_is64 = p.seg_kind == kSegI64;
  const uint32_t seg_esize = seg_is64 ? 8u : 4u;
  const __amdgpu_buffer_rsrc_t rseg =
      make_rsrc(CONV ? p.segpos : nullptr, CONV ? (uint32_t)M * seg_esize : 0u);

  // Both fetch parts are safe for a tile index beyond the last tile (the
  // values are then never used).
  auto fetch_seg = [&](int64_t tile) {
    if (CONV) {
      const int64_t mbase = tile * kTM + rg * kRowsPerGroup - kHalo;
      const int64_t m = mbase + lane;
      const bool look = lane < kRaw && m >= 0 && m < M;
      const uint32_t off = look ? (uint32_t)m * seg_esize : kBufferOutOfRange;
      seg_lo = __builtin_amdgcn_raw_buffer_load_b32(rseg, off, 0, 0);
      seg_hi = __builtin_amdgcn_raw_buffer_load_b32(
          rseg, seg_is64 ? off + 4u : kBufferOutOfRange, 0, 0);
    }
  };
  struct RowFetch {
    __amdgpu_buffer_rsrc_t rx;
    int before;
  };
  // Descriptor over this thread group's rows that exist: rows past the end
  // of x fall outside it, rows before the start (first tile only) get an
  // out-of-range scalar offset.  Both read as zero and are never used: a
  // row before the start is always cut off by the sequence boundary.
  auto fetch_rows_begin = [&](int64_t tile) {
    const int64_t mbase = tile * kTM + rg * kRowsPerGroup - kHalo;
    RowFetch f;
    f.before = mbase < 0 ? (int)-mbase : 0;                     // 0..kHalo
    const int64_t first = mbase < 0 ? 0 : mbase;
    int64_t nrows = M - first;
    nrows = nrows < 0 ? 0 : (nrows > kRaw ? kRaw : nrows);
    f.rx = make_rsrc(xbase + (first < M ? first : 0) * W,
                     (uint32_t)nrows * x_row_bytes);
    return f;
  };
  auto fetch_row = [&](const RowFetch& f, int j) {
    const uint32_t soff = j < f.before
                              ? kBufferOutOfRange
                              : (uint32_t)(j - f.before) * x_row_bytes;
    raw[j] = __builtin_amdgcn_raw_buffer_load_b32(f.rx, c_bytes, soff, 0);
  };
  auto fetch_rows = [&](int64_t tile) {
    const RowFetch f = fetch_rows_begin(tile);
#pragma unroll
    for (int j = 0; j < kRaw; ++j) fetch_row(f, j);
  };

  // Conv of one tile, one row at a time so that the rows can be placed
  // between the matrix instructions of the previous tile.
  //   stage_begin: document-start mask of the tile's rows, history cleared
  //   stage_row(j): j < kHalo feeds the history; j >= kHalo writes LDS row
  //                 j - kHalo of this thread's group
  // The conv in the bf16 kernels' one arithmetic (conv4_dot of rg_common.h):
  // per channel the taps paired as (w0, w1), (w2, w3), the rows paired in
  // time, two dot products per output; nothing is unpacked between the MFMAs.
  uint32_t cw10[2] = {0, 0}, cw32[2] = {0, 0};
  float cb[2] = {0.0f, 0.0f};
  if (CONV) {
    pair_up(cwp[0], cwp[1], cw10[0], cw10[1]);
    pair_up(cwp[2], cwp[3], cw32[0], cw32[1]);
    cb[0] = __uint_as_float(cwp[4] << 16);
    cb[1] = __uint_as_float(cwp[4] & 0xffff0000u);
  }
  uint32_t cut = 0;
  // history of this thread's channel pair: the row before (still packed) and
  // the time pairs (x[t-1], x[t]) that ended one and two rows back, zero where
  // a start cuts
  uint32_t r1 = 0, pn1[2] = {0, 0}, pn2[2] = {0, 0};
  uint16_t* const stage_dst0 =
      lds + (size_t)(rg * kRowsPerGroup) * kLdsStride + cp * 2;

  auto stage_begin = [&](int64_t tile) {
    if (!CONV) return;
    const int64_t mbase = tile * kTM + rg * kRowsPerGroup - kHalo;
    // bit j: row mbase+j begins a sequence row (t == 0) or a document; the
    // conv must not look past it.  Lane j of the wave looks at row mbase+j
    // (all lanes of a wave stage the same rows): one load and one ballot.
    bool st = false;
    {
      const int64_t m = mbase + lane;
      const uint32_t t_base = (uint32_t)(((mbase % T_len) + T_len) % T_len);
      // pin the test here: the values were loaded a tile ago
      uint32_t lo = seg_lo, hi = seg_hi;
      asm volatile("" : "+v"(lo), "+v"(hi));
      // lanes whose row starts a sequence row (t == 0): one lane at most when
      // the sequence is longer than the rows looked at
      bool seq_start;
      if (T_len >= 64) {
        const uint32_t j0 = t_base == 0 ? 0u : (uint32_t)T_len - t_base;
        seq_start = (uint32_t)lane == j0;
      } else {
        seq_start = (t_base + (uint32_t)lane) % (uint32_t)T_len == 0u;
      }
      if (lane < kRaw && m >= 0 && m < M) st = seq_start || ((lo | hi) == 0u);
    }
    cut = (uint32_t)__ballot(st);
    r1 = pn1[0] = pn1[1] = pn2[0] = pn2[1] = 0u;
  };
  // CUTS = false is the straight-line form for a tile without any sequence or
  // document start among its rows (cut == 0).
  auto stage_row = [&](int j, int buf, auto cuts) {
    constexpr bool CUTS = decltype(cuts)::value;
    uint16_t* dst = stage_dst0 + (size_t)buf * kTM * kLdsStride;
    if (!CONV) {
      *reinterpret_cast<uint32_t*>(dst + (size_t)j * kLdsStride) = raw[j];
      return;
    }
    if (CUTS && ((cut >> j) & 1u)) {
      r1 = pn1[0] = pn1[1] = pn2[0] = pn2[1] = 0u;
    }
    uint32_t pn0[2];
    pair_up(r1, raw[j], pn0[0], pn0[1]);
    if (j >= kHalo) {
      float o[2];
      conv4_dot_x2(pn2, pn0, cw10, cw32, cb, o);
      *reinterpret_cast<uint32_t*>(dst + (size_t)(j - kHalo) * kLdsStride) =
          pack_bf16x2(o[0], o[1]);
    }
#pragma unroll
    for (int ch = 0; ch < 2; ++ch) {
      pn2[ch] = pn1[ch];
      pn1[ch] = pn0[ch];
    }
    r1 = raw[j];
  };
  using WithCuts = std::integral_constant<bool, true>;
  using NoCuts = std::integral_constant<bool, false>;

  // Software pipeline over this workgroup's tiles i0, i0+G, ...: while the
  // MFMAs of tile i run, the conv of tile i+G is written to the other LDS
  // buffer and the rows of tile i+2G are loaded.  Per tile, three regions;
  // inside A and B the work is cut into 16 chunks (one k-step each) whose
  // order is pinned with scheduling barriers:
  //   A  chunk: LDS read k+1 | 2 MFMA (rows 0-31)  | conv row k of next tile
  //   B  chunk: LDS read k+1 | 2 MFMA (rows 32-63) | a store of rows 0-31 (first
  //      four chunks) | load of row k (+16) of the tile after next
  //   C  stores of rows 32-63
  int64_t tile = blockIdx.x;
  if (tile < ntiles) {
    fetch_seg(tile);
    fetch_rows(tile);
    stage_begin(tile);
#pragma unroll
    for (int j = 0; j < kRaw; ++j) stage_row(j, 0, WithCuts{});
    fetch_seg(tile + gridDim.x);
    fetch_rows(tile + gridDim.x);
  }
  lds_barrier();

  int buf = 0;
  for (; tile < ntiles; tile += gridDim.x, buf ^= 1) {
    const int64_t next = tile + gridDim.x;
    const int64_t next2 = next + gridDim.x;

    const uint16_t* abase = lds + (size_t)buf * kTM * kLdsStride +
                            (size_t)(lane & 31) * kLdsStride + 8 * (lane >> 5);
    const int64_t row_first = tile * kTM;                       // uniform
    char* const tilep = outbase + row_first * W * 2;            // uniform
    const int rows_left =
        (int)((M - row_first) < kTM ? (M - row_first) : kTM);   // uniform, > 0
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(
        tilep, active ? (uint32_t)rows_left * out_row_bytes : 0u);

    // The block goes through this wave's LDS patch (row-major, bf16) so that
    // each lane stores 16 contiguous bytes (8 rows x 128 bytes per
    // instruction).
    auto acc_init = [&](f32x16& acc0, f32x16& acc1) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const f32x4 b0 = *reinterpret_cast<const f32x4*>(bias_r + 8 * g);
        const f32x4 b1 = *reinterpret_cast<const f32x4*>(bias_r + 32 + 8 * g);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc0[4 * g + q] = b0[q];
          acc1[4 * g + q] = b1[q];
        }
      }
    };
    auto result_to_lds = [&](const f32x16& acc0, const f32x16& acc1) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 v0, v1;
        v0[0] = pack_bf16x2(acc0[4 * g], acc0[4 * g + 1]);
        v0[1] = pack_bf16x2(acc0[4 * g + 2], acc0[4 * g + 3]);
        v1[0] = pack_bf16x2(acc1[4 * g], acc1[4 * g + 1]);
        v1[1] = pack_bf16x2(acc1[4 * g + 2], acc1[4 * g + 3]);
        *reinterpret_cast<u32x2*>(epi_w + 16 * g) = v0;
        *reinterpret_cast<u32x2*>(epi_w + 64 + 16 * g) = v1;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    };
    auto patch_read = [&](int q) {
      return *reinterpret_cast<const u32x4*>(epi_r + q * 8 * kEpiStride);
    };
    // rows past the end of the output fall outside the descriptor
    auto patch_store = [&](int mt, int q, u32x4 v) {
      buffer_store_16(v, ro, out_lane_bytes,
                      (uint32_t)(mt * 32 + q * 8) * out_row_bytes);
    };
    auto a_read = [&](int mt, int ks) {
      Frag a;
      a.q = *reinterpret_cast<const f32x4*>(
          abase + (size_t)mt * 32 * kLdsStride + ks * 16);
      return a;
    };

    {  // ---- region A
      stage_begin(next);
      f32x16 acc0, acc1;
      acc_init(acc0, acc1);
      Frag a[3];  // operand reads run two k-steps ahead
      if (cut == 0) {
#pragma unroll
        for (int j = 0; j < kHalo; ++j) stage_row(j, buf ^ 1, NoCuts{});
        a[0] = a_read(0, 0);
        a[1] = a_read(0, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) {
          if (ks < 14) a[(ks + 2) % 3] = a_read(0, ks + 2);
          if (active && (!NARROW || ks < ksteps)) {
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                bfrag[ks][0].v, a[ks % 3].v, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                bfrag[ks][1].v, a[ks % 3].v, acc1, 0, 0, 0);
          }
          stage_row(kHalo + ks, buf ^ 1, NoCuts{});
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        // a sequence or document starts among the rows of the next tile
        // (one tile in T/64, plus one per document): conv first, with the
        // history cuts, then the matrix instructions
#pragma unroll
        for (int j = 0; j < kRaw; ++j) stage_row(j, buf ^ 1, WithCuts{});
        a[0] = a_read(0, 0);
#pragma unroll
        for (int ks = 0; ks < 16; ++ks) {
          if (ks < 15) a[(ks + 1) % 3] = a_read(0, ks + 1);
          if (active && (!NARROW || ks < ksteps)) {
            acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                bfrag[ks][0].v, a[ks % 3].v, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                bfrag[ks][1].v, a[ks % 3].v, acc1, 0, 0, 0);
          }
        }
      }
      result_to_lds(acc0, acc1);
    }
    fetch_seg(next2);
    {  // ---- region B
      const RowFetch rf = fetch_rows_begin(next2);
      f32x16 acc0, acc1;
      acc_init(acc0, acc1);
      Frag a[3];
      a[0] = a_read(1, 0);
      a[1] = a_read(1, 1);
      u32x4 pv = patch_read(0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < 16; ++ks) {
        if (ks < 14) a[(ks + 2) % 3] = a_read(1, ks + 2);
        if (active && (!NARROW || ks < ksteps)) {
          acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              bfrag[ks][0].v, a[ks % 3].v, acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              bfrag[ks][1].v, a[ks % 3].v, acc1, 0, 0, 0);
        }
        if (ks < 4) {
          patch_store(0, ks, pv);
          if (ks < 3) pv = patch_read(ks + 1);
        }
        fetch_row(rf, ks);
        if (ks + 16 < kRaw) fetch_row(rf, ks + 16);
        __builtin_amdgcn_sched_barrier(0);
      }
      result_to_lds(acc0, acc1);
    }
    // ---- region C
#pragma unroll
    for (int q = 0; q < 4; ++q) patch_store(1, q, patch_read(q));
    // LDS-only barrier: the x rows fetched ahead and the stores of this tile
    // stay in flight across it
    lds_barrier();
  }
}


// ======================================================= fp32 MFMA kernel ==
//
// float32, block width 256, on v_mfma_f32_32x32x2_f32: true float32 products
// and sums (no reduced-precision operand formats), so the 1e-5 bar of the
// float32 path holds.  One workgroup of four waves per (32-row tile of x, a
// quarter of a head's 256 outputs, head and gate); a wave owns 32 output
// columns and one half of K and keeps its 128 x 32 weights in 64 registers for
// all the row tiles it walks; the two halves of K meet in LDS.  The row tile
// (optionally convolved on load) is staged through LDS.  Small work items on
// purpose: the shapes that come here in float32 are small, and 32 x 64 outputs
// per workgroup with K in halves make 64 matrix instructions per wave, which
// spread evenly over the SIMDs (config 1: 1280 workgroups, five to a CU).
//
// Operand layout of the instruction: lane l supplies A[row l % 32][k = l / 32]
// and B[k = l / 32][col l % 32] of a 32 x 2 by 2 x 32 product.  Which two k go
// together is free as long as A and B agree, so each lane reads four
// consecutive k of its row with one 16-byte LDS read (k = 8 j + 4 (l / 32) + i,
// i = 0..3) and holds the weights of the same k.
constexpr int kF32TM = 32;          // rows per tile
constexpr int kF32Stride = kBW + 4; // floats per LDS row (16 rows: 64 banks)
constexpr size_t kF32LdsBytes = (size_t)kF32TM * kF32Stride * sizeof(float);

template <bool CONV>
__global__ void __launch_bounds__(256, 3) gates_mfma_f32_kernel(GemmArgs p) {
  extern __shared__ __align__(16) unsigned char f32_lds[];
  float* const As = reinterpret_cast<float*>(f32_lds);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int z = blockIdx.z;
  const int gate = z / p.H;
  const int h = z - gate * p.H;
  const int col = lane & 31, g = lane >> 5;
  const int nb = wave & 1, kh = wave >> 1;  // column block, half of K
  const int n = blockIdx.y * 64 + nb * 32 + col;  // output column in head
  const float* x = (const float*)p.x;
  const float* w = (const float*)p.w[gate] + (int64_t)h * kBW * kBW;
  float* out = (float*)p.out[gate];
  const int64_t W = p.W;

  // this lane's weights: k = 128 kh + 8 j + 4 g + i at register 4 j + i
  float bw_[64];
  {
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(w, kBW * kBW * 4);
    const uint32_t woff = (uint32_t)((128 * kh + 4 * g) * kBW + n) * 4u;
#pragma unroll
    for (int j = 0; j < 16; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        bw_[4 * j + i] = __builtin_bit_cast(
            float, __builtin_amdgcn_raw_buffer_load_b32(
                       rw, woff, (uint32_t)((8 * j + i) * kBW * 4), 0));
  }
  const float bias = ((const float*)p.b[gate])[h * kBW + n];

  // staging: thread = channel of the head
  const int c = h * kBW + tid;
  float cw0 = 0, cw1 = 0, cw2 = 0, cw3 = 0, cb = 0;
  if (CONV) {
    const float* cw = (const float*)p.conv_w;
    cw0 = cw[c]; cw1 = cw[W + c]; cw2 = cw[2 * W + c]; cw3 = cw[3 * W + c];
    cb = ((const float*)p.conv_b)[c];
  }

  const int64_t ntiles = (p.M + kF32TM - 1) / kF32TM;
  for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    const int64_t m0 = tile * kF32TM;
    if (CONV) {
      // bit 2 + r of starts: a document or a sequence begins at row m0 + r
      // (every wave works the mask out for itself: it stays in scalar
      // registers)
      bool st = false;
      if (lane < kF32TM + 2) {
        const int64_t m = m0 + lane - 2;
        st = true;
        if (m >= 0 && m < p.M)
          st = (m % p.T == 0) || is_doc_start(p.segpos, p.seg_kind, m);
      }
      // Rows m0-3 .. m0+31 through a descriptor over just these rows (rows
      // before the first and after the last read as zero), all requested
      // before the first is used: one memory round trip per tile.
      const int64_t first = m0 >= 3 ? m0 - 3 : 0;
      const int64_t last = m0 + kF32TM < p.M ? m0 + kF32TM : p.M;
      const __amdgpu_buffer_rsrc_t rx = make_rsrc(
          x + first * W, (uint32_t)((last - first) * W * sizeof(float)));
      const uint32_t row_bytes = (uint32_t)W * 4u;
      const uint32_t voff = (uint32_t)c * 4u;
      const int skip = (int)(first - (m0 - 3));  // rows before row 0: 0..3
      float xv[kF32TM + 3];
#pragma unroll
      for (int r = 0; r < kF32TM + 3; ++r)
        xv[r] = r < skip ? 0.0f
                         : __builtin_bit_cast(
                               float, __builtin_amdgcn_raw_buffer_load_b32(
                                          rx, voff,
                                          (uint32_t)(r - skip) * row_bytes, 0));
      const uint64_t starts = __ballot(st);  // (after the row loads are out)
#pragma unroll
      for (int r = 0; r < kF32TM; ++r) {
        // taps older than the newest document start of rows m-2 .. m are cut
        const bool a1 = !((starts >> (2 + r)) & 1);
        const bool a2 = a1 && !((starts >> (1 + r)) & 1);
        const bool a3 = a2 && !((starts >> r) & 1);
        As[r * kF32Stride + tid] =
            conv4(xv[r + 3], a1 ? xv[r + 2] : 0.0f, a2 ? xv[r + 1] : 0.0f,
                  a3 ? xv[r] : 0.0f, cw0, cw1, cw2, cw3, cb);
      }
    } else {
#pragma unroll 8
      for (int r = 0; r < kF32TM; ++r) {
        const int64_t m = m0 + r;
        As[r * kF32Stride + tid] = m < p.M ? x[m * W + c] : 0.0f;
      }
    }
    __syncthreads();

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    const float* a_lane = As + col * kF32Stride + 128 * kh + 4 * g;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(a_lane + 8 * j);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], bw_[4 * j + i], acc, 0,
                                                   0, 0);
    }
    // the upper half of K hands its sums over through LDS (the staged tile is
    // done with): [register][column block][lane], lanes next to each other
    __syncthreads();
    float* const red = As + nb * 64 + lane;
    if (kh == 1) {
#pragma unroll
      for (int r = 0; r < 16; ++r) red[r * 128] = acc[r];
    }
    __syncthreads();
    if (kh == 0) {
      // result register r of lane l: row 8 (r / 4) + 4 (l / 32) + r % 4,
      // column l % 32
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t m = m0 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (m < p.M)
          out[m * W + h * kBW + n] = (acc[r] + red[r * 128]) + bias;
      }
    }
    __syncthreads();  // the tile is overwritten by the next round
  }
}

}  // namespace

hipError_t launch_gemm_generic(const GemmArgs& a, int dtype, hipStream_t s) {
  const int64_t mt = (a.M + kGT - 1) / kGT;
  const int ntl = (a.bw + kGT - 1) / kGT;
  if (mt > 0x7fffffff || (int64_t)a.H * a.ngates > 65535 || ntl > 65535)
    return hipErrorInvalidValue;
  dim3 grid((unsigned)mt, (unsigned)ntl, (unsigned)(a.H * a.ngates));
  if (dtype == 0) {
    if (a.apply_conv)
      bdl_generic_kernel<float, true><<<grid, 256, 0, s>>>(a);
    else
      bdl_generic_kernel<float, false><<<grid, 256, 0, s>>>(a);
  } else {
    if (a.apply_conv)
      bdl_generic_kernel<uint16_t, true><<<grid, 256, 0, s>>>(a);
    else
      bdl_generic_kernel<uint16_t, false><<<grid, 256, 0, s>>>(a);
  }
  return hipGetLastError();
}

hipError_t launch_gemm_mfma_f32(const GemmArgs& a, hipStream_t s) {
  // needs float32 and bw == 256 (checked by the caller); one or two gates
  const int64_t ntiles = (a.M + kF32TM - 1) / kF32TM;
  // enough workgroups for every CU five times over; beyond that a workgroup
  // walks several row tiles with its weights in place
  const int64_t per_tile = 4 * (int64_t)a.H * a.ngates;
  int64_t gx = (1280 + per_tile - 1) / per_tile;
  if (gx > ntiles) gx = ntiles;
  if (gx < 1) gx = 1;
  if ((int64_t)a.H * a.ngates > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)gx, 4, (unsigned)(a.H * a.ngates));
  hipError_t e;
  if (a.apply_conv) {
    static OncePerDevice once;
    e = set_max_dynamic_lds(once, (const void*)gates_mfma_f32_kernel<true>,
                            kF32LdsBytes);
    if (e != hipSuccess) return e;
    gates_mfma_f32_kernel<true><<<grid, 256, kF32LdsBytes, s>>>(a);
  } else {
    static OncePerDevice once;
    e = set_max_dynamic_lds(once, (const void*)gates_mfma_f32_kernel<false>,
                            kF32LdsBytes);
    if (e != hipSuccess) return e;
    gates_mfma_f32_kernel<false><<<grid, 256, kF32LdsBytes, s>>>(a);
  }
  return hipGetLastError();
}

hipError_t launch_gemm_mfma_bf16(const GemmArgs& a, hipStream_t s) {
  // bw <= 256 and a multiple of 8 (narrower heads are padded with zeros
  // inside the kernel: the caller picks it where that still pays); one matrix
  // or both gates
  if (a.bw < 8 || a.bw > kBW || a.bw % 8 != 0) return hipErrorInvalidValue;
  const int64_t ntiles = (a.M + kTM - 1) / kTM;
  int per_head = 256 / a.H;  // about one resident workgroup per CU
  if (per_head < 1) per_head = 1;
  if (per_head > ntiles) per_head = (int)ntiles;
  if (a.H > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)per_head, (unsigned)a.H);
  if (a.ngates == 1 && a.apply_conv) return hipErrorInvalidValue;
  auto launch = [&](auto kernel, OncePerDevice& once) {
    const hipError_t e =
        set_max_dynamic_lds(once, (const void*)kernel, kMfmaLdsBytes);
    if (e != hipSuccess) return e;
    kernel<<<grid, 512, kMfmaLdsBytes, s>>>(a);
    return hipGetLastError();
  };
  static OncePerDevice once[6];
  const bool narrow = a.bw < kBW;
  if (a.ngates == 1)
    return narrow ? launch(gates_mfma_bf16_kernel<false, true, true>, once[0])
                  : launch(gates_mfma_bf16_kernel<false, true, false>, once[1]);
  if (a.apply_conv)
    return narrow ? launch(gates_mfma_bf16_kernel<true, false, true>, once[2])
                  : launch(gates_mfma_bf16_kernel<true, false, false>, once[3]);
  return narrow ? launch(gates_mfma_bf16_kernel<false, false, true>, once[4])
                : launch(gates_mfma_bf16_kernel<false, false, false>, once[5]);
}

}  // namespace rg
