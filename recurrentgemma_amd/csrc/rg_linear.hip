// Linear layers of the residual stack for a handful of rows (one decode step
// of a batch of at most 64 sequences): out[M, N] = x[M, K] @ W^T + bias, bf16
// with fp32 accumulation.  These are torch.nn.Linear / Einsum calls in the
// reference (recurrentgemma/torch/modules.py:579-601 linear_y / linear_x /
// linear_out, :711-721 ffw_up / ffw_down, :334-352 the attention projections);
// with M <= 64 each is one pass over its weight matrix and nothing else, so the
// kernel is built around streaming W:
//  * W is repacked once (linear_pack_kernel) into the operand order of
//    v_mfma_f32_32x32x16_bf16: block (tile, k-step) of 1 KB holds, for lane
//    l = 32 g + r, the eight values W[32 tile + r, 16 kstep + 8 g .. +8], so a
//    wave reads its 32 weight rows as one contiguous stream, 1 KB per
//    instruction.  (Reading the row-major matrix directly touches 32 cache
//    lines per instruction and ran at a quarter of the speed.)
//  * A workgroup owns NT tiles of 32 weight rows; its waves split K in chunks
//    of 64 and add their partial sums through LDS at the end.  x (at most
//    64 x K, L2 resident) is staged by each wave for its own chunks: 64 rows
//    x 128 B coalesced from global, through a wave-private LDS tile, into the
//    B-operand fragments.
//  * Few weight rows (N / 32 tiles well below the number of CUs) and a long K:
//    the grid also splits K (gridDim.y), every workgroup writes its fp32
//    partial sums, and linear_finish_kernel adds them in a fixed order, so the
//    result does not depend on which workgroup ran first.
// Epilogues: bias; bias then residual add (two roundings, like the separate
// add of the reference); gelu(gate) * up for the paired rows of the MLP's
// stacked up-projection (modules.py:752-757).
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

union Frag {
  u32x4 u;
  bf16x8 v;
};

constexpr int kXStride = 72;  // elements per staged x row: 64 + 8 of padding
constexpr int kWaves = 8;

__host__ __device__ constexpr int wave_lds_bytes(int nt) {
  return nt * 8192 > 64 * kXStride * 2 ? nt * 8192 : 64 * kXStride * 2;
}

enum LinearMode { kStore = 0, kGeluPair = 1, kPartial = 2 };

__device__ __forceinline__ void unpack4(u32x2 b, float (&v)[4]) {
  v[0] = __uint_as_float(b[0] << 16);
  v[1] = __uint_as_float(b[0] & 0xffff0000u);
  v[2] = __uint_as_float(b[1] << 16);
  v[3] = __uint_as_float(b[1] & 0xffff0000u);
}

// Where column n of the result lives: the output is [G][M][gw] with gw = N / G
// (G = 1: plain [M, N]).
__device__ __forceinline__ size_t out_index(int m, int n, int M, int gw) {
  const int grp = n / gw;
  return ((size_t)grp * M + m) * gw + (n - grp * gw);
}

template <int NT, int MODE>
__global__ void __launch_bounds__(kWaves * 64)
linear_rows_kernel(LinearArgs p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int kWaveLds = wave_lds_bytes(NT);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 31, g = lane >> 5;
  const int M = p.M, K = p.K;
  const int chunks = K / 64;
  // this workgroup's slice of K, then this wave's
  const int per_wg = (chunks + (int)gridDim.y - 1) / (int)gridDim.y;
  const int wg0 = blockIdx.y * per_wg, wg1 = min(chunks, wg0 + per_wg);
  const int per = (max(wg1 - wg0, 0) + kWaves - 1) / kWaves;
  const int c0 = wg0 + wave * per;
  const int c1 = min(wg1, c0 + per);
  uint16_t* xs = reinterpret_cast<uint16_t*>(smem + (size_t)wave * kWaveLds);

  // x chunk = 64 rows x 128 B; load j covers rows 8 j + lane / 8 (rows >= M
  // repeat row M - 1; their results are never stored)
  const int xrow = lane >> 3, xseg = lane & 7;
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x);
  const uint16_t* xg[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
    xg[j] = x + (size_t)min(8 * j + xrow, M - 1) * K + 8 * xseg;
  const u32x4* wg[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
    wg[t] = reinterpret_cast<const u32x4*>(p.w_packed) +
            ((size_t)(blockIdx.x * NT + t) * (K / 16)) * 64 + lane;

  f32x16 acc[NT][2];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[t][m][i] = 0.0f;

  u32x4 xr[8];
  Frag wq[2][NT][4];
  // loads of the chunk after the last one read the last one again
  auto load_chunk = [&](int c, int slot) {
    const int cc = min(c, chunks - 1);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      xr[j] = *reinterpret_cast<const u32x4*>(xg[j] + (size_t)cc * 64);
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int k = 0; k < 4; ++k)
        wq[slot][t][k].u =
            __builtin_nontemporal_load(wg[t] + (size_t)(cc * 4 + k) * 64);
  };
  auto body = [&](int slot, int c) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      *reinterpret_cast<u32x4*>(xs + (8 * j + xrow) * kXStride + 8 * xseg) =
          xr[j];
    Frag xf[4][2];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int m = 0; m < 2; ++m)
        xf[k][m].u = *reinterpret_cast<const u32x4*>(
            xs + (32 * m + r) * kXStride + 16 * k + 8 * g);
    load_chunk(c + 1, slot ^ 1);
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int m = 0; m < 2; ++m)
          acc[t][m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              wq[slot][t][k].v, xf[k][m].v, acc[t][m], 0, 0, 0);
  };
  if (c0 < c1) {
    load_chunk(c0, 0);
    int c = c0;
    for (; c + 1 < c1; c += 2) {
      body(0, c);
      body(1, c + 1);
    }
    if (c < c1) body(0, c);
  }

  // the waves' partial sums meet in LDS (each wave's region is its own x tile)
  float* mine = reinterpret_cast<float*>(smem + (size_t)wave * kWaveLds);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        mine[((t * 2 + m) * 16 + i) * 64 + lane] = acc[t][m][i];
  lds_barrier();
  const float* red = reinterpret_cast<const float*>(smem);
  // sum of accumulator registers 4 q .. 4 q + 3 of (tile t, half m, lane l):
  // result rows 32 m + l % 32, weight rows 32 t + 8 q + 4 (l / 32) + 0..3
  auto gather = [&](int t, int m, int q, int l, float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = 0.0f;
    for (int wv = 0; wv < kWaves; ++wv) {
      const float* src = red + (size_t)wv * (kWaveLds / 4) +
                         ((t * 2 + m) * 16 + q * 4) * 64 + l;
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += src[i * 64];
    }
  };
  const uint16_t* bias = reinterpret_cast<const uint16_t*>(p.bias);
  uint16_t* out = reinterpret_cast<uint16_t*>(p.out);
  if (MODE == kGeluPair) {
    // tile 0 = 32 rows of the gate half, tile 1 = the same rows of the up half
    static_assert(MODE != kGeluPair || NT == 2, "pairs need two tiles");
    const int half = p.N / 2;
    for (int qd = threadIdx.x; qd < 2 * 4 * 64; qd += kWaves * 64) {
      const int l = qd & 63, q = (qd >> 6) & 3, m = qd >> 8;
      const int row = 32 * m + (l & 31);
      const int col = blockIdx.x * 32 + 8 * q + 4 * (l >> 5);
      if (row >= M) continue;
      float gate[4], up[4];
      gather(0, m, q, l, gate);
      gather(NT - 1, m, q, l, up);
      if (bias) {
        float bg[4], bu[4];
        unpack4(*reinterpret_cast<const u32x2*>(bias + col), bg);
        unpack4(*reinterpret_cast<const u32x2*>(bias + half + col), bu);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          gate[i] += bg[i];
          up[i] += bu[i];
        }
      }
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = gelu_mul_bf16(round_to_bf16(up[i]), round_to_bf16(gate[i]));
      const u32x2 ov = {pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
      *reinterpret_cast<u32x2*>(out + (size_t)row * half + col) = ov;
    }
    return;
  }
  for (int qd = threadIdx.x; qd < NT * 2 * 4 * 64; qd += kWaves * 64) {
    const int l = qd & 63, q = (qd >> 6) & 3, m = (qd >> 8) & 1, t = qd >> 9;
    const int row = 32 * m + (l & 31);
    const int col = (blockIdx.x * NT + t) * 32 + 8 * q + 4 * (l >> 5);
    if (row >= M) continue;
    float v[4];
    gather(t, m, q, l, v);
    if (MODE == kPartial) {
      const f32x4 o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<f32x4*>(p.partial +
                                ((size_t)blockIdx.y * M + row) * p.N + col) = o;
      continue;
    }
    if (bias) {
      float b[4];
      unpack4(*reinterpret_cast<const u32x2*>(bias + col), b);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] += b[i];
    }
    const size_t at = out_index(row, col, M, p.group_width);
    if (p.residual) {
      float res[4];
      unpack4(*reinterpret_cast<const u32x2*>(
                  reinterpret_cast<const uint16_t*>(p.residual) + at), res);
#pragma unroll
      for (int i = 0; i < 4; ++i) v[i] = round_to_bf16(v[i]) + res[i];
    }
    const u32x2 ov = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
    *reinterpret_cast<u32x2*>(out + at) = ov;
  }
}

// Sum of the K slices (in slice order), bias, optional residual; four columns
// per thread.
__global__ void __launch_bounds__(256)
linear_finish_kernel(LinearArgs p, int slices) {
  const int quads_per_row = p.N / 4;
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.M * quads_per_row) return;
  const int row = idx / quads_per_row, col = 4 * (idx - row * quads_per_row);
  float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int s = 0; s < slices; ++s) {
    const f32x4 part = *reinterpret_cast<const f32x4*>(
        p.partial + ((size_t)s * p.M + row) * p.N + col);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += part[i];
  }
  if (p.bias) {
    float b[4];
    unpack4(*reinterpret_cast<const u32x2*>(
                reinterpret_cast<const uint16_t*>(p.bias) + col), b);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] += b[i];
  }
  const size_t at = out_index(row, col, p.M, p.group_width);
  if (p.residual) {
    float res[4];
    unpack4(*reinterpret_cast<const u32x2*>(
                reinterpret_cast<const uint16_t*>(p.residual) + at), res);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = round_to_bf16(v[i]) + res[i];
  }
  const u32x2 ov = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
  *reinterpret_cast<u32x2*>(reinterpret_cast<uint16_t*>(p.out) + at) = ov;
}

// One 16-byte item of the packed matrix per thread.  Source layouts:
//   0: [N, K] (torch.nn.Linear.weight)
//   1: [G, K, N / G] (the reference's Einsum weight "cdD", layers.py:97-101;
//      weight row n = g (N / G) + j is w[g, :, j])
// pair: tile 2 b is rows 32 b .. of the first half of the rows, tile 2 b + 1
// the same rows of the second half.
__global__ void __launch_bounds__(256)
linear_pack_kernel(const uint16_t* __restrict__ w, u32x4* __restrict__ packed,
                   int N, int K, int layout, int groups, int pair) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int ksteps = K / 16;
  if (idx >= (int64_t)(N / 32) * ksteps * 64) return;
  const int lane = (int)(idx & 63);
  const int ks = (int)((idx >> 6) % ksteps);
  const int tile = (int)((idx >> 6) / ksteps);
  int row = tile * 32 + (lane & 31);
  if (pair) row = (tile & 1) * (N / 2) + (tile >> 1) * 32 + (lane & 31);
  const int k = ks * 16 + 8 * (lane >> 5);
  u32x4 v;
  if (layout == 0) {
    v = *reinterpret_cast<const u32x4*>(w + (size_t)row * K + k);
  } else {
    const int gw = N / groups;
    const int grp = row / gw, j = row - grp * gw;
    const uint16_t* src = w + ((size_t)grp * K + k) * gw + j;
    uint32_t e[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) e[i] = src[(size_t)i * gw];
    v = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16),
              e[6] | (e[7] << 16)};
  }
  packed[idx] = v;
}

template <int NT, int MODE>
hipError_t launch_rows(const LinearArgs& a, dim3 grid, hipStream_t s) {
  constexpr int lds = kWaves * wave_lds_bytes(NT);
  static OncePerDevice once;  // one per instantiation of this launcher
  hipError_t e = set_max_dynamic_lds(
      once, (const void*)linear_rows_kernel<NT, MODE>, lds);
  if (e != hipSuccess) return e;
  linear_rows_kernel<NT, MODE><<<grid, kWaves * 64, lds, s>>>(a);
  return hipGetLastError();
}

}  // namespace

// How many slices of K the grid takes: more than one only where the weight
// rows alone leave most CUs idle and K is long enough to share out.
int linear_rows_k_slices(int K, int N) {
  const int tiles = N / 32;
  if (tiles <= 96 && K >= 5120) return 3;
  return 1;
}

hipError_t launch_linear_pack(const void* w, void* packed, int N, int K,
                              int layout, int groups, int pair, hipStream_t s) {
  const int64_t items = (int64_t)(N / 32) * (K / 16) * 64;
  linear_pack_kernel<<<dim3((unsigned)((items + 255) / 256)), 256, 0, s>>>(
      (const uint16_t*)w, (u32x4*)packed, N, K, layout, groups, pair);
  return hipGetLastError();
}

hipError_t launch_linear_rows_partial(const LinearArgs& a, int slices,
                                      hipStream_t s) {
  return launch_rows<1, kPartial>(a, dim3(a.N / 32, slices), s);
}

hipError_t launch_linear_rows(const LinearArgs& a, int gelu_pair,
                              hipStream_t s) {
  const int tiles = a.N / 32;
  if (gelu_pair)
    return launch_rows<2, kGeluPair>(a, dim3(tiles / 2, 1), s);
  const int slices = linear_rows_k_slices(a.K, a.N);
  if (slices > 1) {
    hipError_t e = launch_rows<1, kPartial>(a, dim3(tiles, slices), s);
    if (e != hipSuccess) return e;
    const int quads = a.M * (a.N / 4);
    linear_finish_kernel<<<dim3((quads + 255) / 256), 256, 0, s>>>(a, slices);
    return hipGetLastError();
  }
  // two tiles per workgroup once that still leaves a workgroup for most CUs
  if (tiles % 2 == 0 && tiles / 2 >= 200)
    return launch_rows<2, kStore>(a, dim3(tiles / 2, 1), s);
  return launch_rows<1, kStore>(a, dim3(tiles, 1), s);
}

}  // namespace rg
