// Stand-alone Conv1D kernels (any temporal width): the module-level drop-in
// for Conv1D.forward.  The fused prefill path does the width-4 conv inside the
// gate GEMM and the scan kernel instead and does not come through here.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

// One thread per output element; consecutive threads take consecutive
// channels, so every tap is a coalesced row read (taps hit L2 after the first).
template <typename T>
__global__ void __launch_bounds__(256)
conv1d_prefill_kernel(const T* __restrict__ x, const void* __restrict__ segpos,
                      int seg_kind, const T* __restrict__ w,
                      const T* __restrict__ bias, T* __restrict__ out,
                      int T_len, int W, int K, int64_t total) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const int64_t m = idx / W;
    const int c = (int)(idx - m * W);
    store_scalar(out + idx,
                 conv_point<T>(x, segpos, seg_kind, w, bias, T_len, W, K, m, c));
  }
}

// The conv state the reference hands back after a prefill: the last K-1 input
// rows, each zeroed if a document starts in one of the (up to K-1) positions
// after it; rows before the start of the sequence are zero.
template <typename T>
__global__ void __launch_bounds__(256)
conv1d_cache_tail_kernel(const T* __restrict__ x,
                         const void* __restrict__ segpos, int seg_kind,
                         T* __restrict__ cache_out, int B, int T_len, int W,
                         int K) {
  const int64_t total = (int64_t)B * (K - 1) * W;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const int c = (int)(idx % W);
    const int64_t bk = idx / W;
    const int k = (int)(bk % (K - 1));
    const int64_t b = bk / (K - 1);
    const int t = T_len - (K - 1) + k;
    float v = 0.0f;
    if (t >= 0) {
      bool alive = true;
      for (int j = 1; j <= K - 1 && t + j <= T_len - 1; ++j)
        if (is_doc_start(segpos, seg_kind, b * T_len + t + j)) alive = false;
      if (alive) v = load_scalar(x + (b * T_len + t) * W + c);
    }
    store_scalar(cache_out + idx, v);
  }
}

// Backward pass of the prefill conv.  With keep_s[t] = "no document starts
// among tokens t-s+1 .. t" (what conv_point applies tap by tap):
//   out[t] = bias + sum_s w[K-1-s] x[t-s] keep_s[t]
//   dx[u]      = sum_s w[K-1-s] dout[u+s] keep_s[u+s]        (u + s < T)
//   dw[K-1-s] += x[t-s] keep_s[t] dout[t],   dbias += dout[t]
// A thread owns one channel and a run of `rows` consecutive flattened rows
// (b, t): it writes dx for them and leaves its sums of dw and dbias in
// `partial` [row chunks][K + 1][W] (float32), which the caller adds up.  The
// neighbouring rows it re-reads come from cache.  `rows` is 32 while that
// leaves at most 512 chunks and grows up to 256 beyond (conv1d_backward_rows):
// a plane of partial sums is (K + 1) W floats written and read again, 16 %
// of the pass's own traffic at 32 rows of bf16 and 2 % at 256.
constexpr int kConvBwdRows = 32;
constexpr int kConvBwdMaxRows = 256;
constexpr int kConvBwdChunks = 512;

template <typename T>
__global__ void __launch_bounds__(256)
conv1d_backward_kernel(const T* __restrict__ dout, const T* __restrict__ x,
                       const void* __restrict__ segpos, int seg_kind,
                       const T* __restrict__ w, T* __restrict__ dx,
                       float* __restrict__ partial, int T_len, int W, int K,
                       int64_t M, int rows) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int64_t m0 = (int64_t)blockIdx.x * rows;
  const int64_t m1 = m0 + rows < M ? m0 + rows : M;
  constexpr int kMaxK = 16;  // widths above are refused by the caller
  float wk[kMaxK], dw[kMaxK], db = 0.0f;
#pragma unroll
  for (int s = 0; s < kMaxK; ++s) {
    wk[s] = s < K ? load_scalar(w + (int64_t)(K - 1 - s) * W + c) : 0.0f;
    dw[s] = 0.0f;
  }
  for (int64_t m = m0; m < m1; ++m) {
    const int t = (int)(m % T_len);
    const float g = load_scalar(dout + m * W + c);
    db += g;
    float acc = 0.0f;
    bool back = true, ahead = true;
#pragma unroll
    for (int s = 0; s < kMaxK; ++s) {
      if (s < K) {
        // tap s of token t looks back at x[t-s]
        if (s > 0 && s <= t && is_doc_start(segpos, seg_kind, m - s + 1))
          back = false;
        if (s <= t && back)
          dw[s] = __builtin_fmaf(load_scalar(x + (m - s) * W + c), g, dw[s]);
        // token t is x[t'-s] of token t' = t + s
        if (s > 0 && t + s < T_len && is_doc_start(segpos, seg_kind, m + s))
          ahead = false;
        if (t + s < T_len && ahead)
          acc = __builtin_fmaf(wk[s], load_scalar(dout + (m + s) * W + c), acc);
      }
    }
    store_scalar(dx + m * W + c, acc);
  }
  float* out = partial + (int64_t)blockIdx.x * (K + 1) * W + c;
#pragma unroll
  for (int s = 0; s < kMaxK; ++s)
    if (s < K) out[(int64_t)(K - 1 - s) * W] = dw[s];
  out[(int64_t)K * W] = db;
}

// ---- temporal width 4, 16 bytes per lane: the usual case, streaming ---------
// A wave takes 32 consecutive flattened rows (b, t) of 64 x 16 bytes of
// channels; a lane walks its rows in time order with the three rows before the
// current one in registers (loaded once as a halo), so every row of x is read
// once (plus 3 in 32 for the halo) and every output row written once, as
// 16-byte accesses.  A document start -- or the first token of a sequence row --
// zeroes the history registers: later tokens then see zeros exactly where the
// definition drops a tap.  Rows are requested eight at a time before the first
// is used.
constexpr int kConvRun = 32;    // rows per wave of the forward kernels
constexpr int kConvBatch = 8;   // rows requested together

template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  __device__ static void unpack(u32x4 r, float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(r[i]);
  }
  __device__ static u32x4 pack(const float (&v)[4]) {
    return u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]),
                 __float_as_uint(v[2]), __float_as_uint(v[3])};
  }
};
template <>
struct Vec16<uint16_t> {
  static constexpr int N = 8;
  __device__ static void unpack(u32x4 r, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(r[i] << 16);
      v[2 * i + 1] = __uint_as_float(r[i] & 0xffff0000u);
    }
  }
  __device__ static u32x4 pack(const float (&v)[8]) {
    return u32x4{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                 pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
  }
};

// Which of the rows around a run (fewer than `span` of them, from `base` on)
// is the first token of a sequence row: at most one when the sequences are at
// least `span` tokens long, found once per wave instead of a 64-bit remainder
// per row.
struct SeqStarts {
  int64_t first;  // first row >= base that begins a sequence row
  int T_len;
  bool one;       // the sequences are long enough for `first` to be the only one
  __device__ SeqStarts(int64_t base, int T, int span) : T_len(T), one(T >= span) {
    const int64_t r = base % T;
    first = r == 0 ? base : base + (T - r);
  }
  __device__ bool at(int64_t m) const {
    return one ? m == first : m % T_len == 0;
  }
};

// row m starts a history: first token of a sequence row, or of a document
__device__ __forceinline__ bool conv_row_starts(const void* segpos, int seg_kind,
                                                const SeqStarts& seq, int64_t m) {
  return seq.at(m) || is_doc_start(segpos, seg_kind, m);
}

// RUN rows per wave: the longer, the fewer halo rows are read twice (3 per
// run) and the fewer workgroups are dispatched.
template <typename T, int RUN>
__global__ void __launch_bounds__(1024)
conv1d_prefill_k4_kernel(const T* __restrict__ x, const void* __restrict__ segpos,
                         int seg_kind, const T* __restrict__ w,
                         const T* __restrict__ bias, T* __restrict__ out,
                         int T_len, int W, int64_t M) {
  using V = Vec16<T>;
  constexpr int N = V::N;
  // the waves of a workgroup lie side by side along a row (up to 16 of them:
  // 16 KB of a row), so that what they request together is contiguous
  const int c = ((int)blockIdx.y * (int)blockDim.x + (int)threadIdx.x) * N;
  if (c >= W) return;  // W % N == 0 (launcher): a lane is inside or outside
  const int64_t m0 = (int64_t)blockIdx.x * RUN;
  const int64_t m1 = m0 + RUN < M ? m0 + RUN : M;
  const SeqStarts seq(m0 >= 3 ? m0 - 3 : 0, T_len, RUN + 3);
  auto row = [&](const T* base, int64_t m) {
    return *reinterpret_cast<const u32x4*>(base + m * W + c);
  };
  if constexpr (sizeof(T) == 2) {
    // bf16: the kernels' one width-4 arithmetic (conv4_dot of rg_common.h) on
    // rows that stay packed: per channel the time pairs (x[t-1], x[t]), two
    // dot products per output
    float bb[N];
    V::unpack(*reinterpret_cast<const u32x4*>(bias + c), bb);
    uint32_t w10[N], w32[N];
    {
      const u32x4 t0 = row(w, 0), t1 = row(w, 1), t2 = row(w, 2), t3 = row(w, 3);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        pair_up(t0[q], t1[q], w10[2 * q], w10[2 * q + 1]);
        pair_up(t2[q], t3[q], w32[2 * q], w32[2 * q + 1]);
      }
    }
    // history: the row before (packed) and the pairs that ended one and two
    // rows back; zero where a start cuts
    u32x4 r1 = {0, 0, 0, 0};
    uint32_t pn1[N], pn2[N];
#pragma unroll
    for (int e = 0; e < N; ++e) pn1[e] = pn2[e] = 0u;
    auto cut = [&]() {
      r1 = u32x4{0, 0, 0, 0};
#pragma unroll
      for (int e = 0; e < N; ++e) pn1[e] = pn2[e] = 0u;
    };
    auto push = [&](const u32x4& cur, uint32_t (&pn0)[N]) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        pair_up(r1[q], cur[q], pn0[2 * q], pn0[2 * q + 1]);
    };
    auto shift = [&](const u32x4& cur, const uint32_t (&pn0)[N]) {
#pragma unroll
      for (int e = 0; e < N; ++e) {
        pn2[e] = pn1[e];
        pn1[e] = pn0[e];
      }
      r1 = cur;
    };
    for (int64_t j = m0 - 3; j < m0; ++j) {
      if (j < 0) continue;
      if (conv_row_starts(segpos, seg_kind, seq, j)) cut();
      const u32x4 cur = row(x, j);
      uint32_t pn0[N];
      push(cur, pn0);
      shift(cur, pn0);
    }
    for (int64_t mb = m0; mb < m1; mb += kConvBatch) {
      u32x4 raw[kConvBatch];
      bool st[kConvBatch];
#pragma unroll
      for (int u = 0; u < kConvBatch; ++u) {
        const int64_t m = mb + u < m1 ? mb + u : m1 - 1;
        raw[u] = row(x, m);
        st[u] = conv_row_starts(segpos, seg_kind, seq, m);
      }
#pragma unroll
      for (int u = 0; u < kConvBatch; ++u) {
        if (mb + u < m1) {
          if (st[u]) cut();
          uint32_t pn0[N];
          push(raw[u], pn0);
          float o[N];
#pragma unroll
          for (int q = 0; q < N; q += 4) {
            const uint32_t po[4] = {pn2[q], pn2[q + 1], pn2[q + 2], pn2[q + 3]};
            const uint32_t pw[4] = {pn0[q], pn0[q + 1], pn0[q + 2], pn0[q + 3]};
            const uint32_t wa[4] = {w10[q], w10[q + 1], w10[q + 2], w10[q + 3]};
            const uint32_t wb[4] = {w32[q], w32[q + 1], w32[q + 2], w32[q + 3]};
            const float bq[4] = {bb[q], bb[q + 1], bb[q + 2], bb[q + 3]};
            float oq[4];
            conv4_dot_x4(po, pw, wa, wb, bq, oq);
#pragma unroll
            for (int e = 0; e < 4; ++e) o[q + e] = oq[e];
          }
          shift(raw[u], pn0);
          *reinterpret_cast<u32x4*>(out + (mb + u) * W + c) = V::pack(o);
        }
      }
    }
    return;
  }
  float w0[N], w1[N], w2[N], w3[N], bb[N];
  V::unpack(row(w, 0), w0);
  V::unpack(row(w, 1), w1);
  V::unpack(row(w, 2), w2);
  V::unpack(row(w, 3), w3);
  V::unpack(*reinterpret_cast<const u32x4*>(bias + c), bb);
  // history: h1 = x[m-1], h2 = x[m-2], h3 = x[m-3], zero where a start cuts
  float h1[N], h2[N], h3[N];
#pragma unroll
  for (int e = 0; e < N; ++e) h1[e] = h2[e] = h3[e] = 0.0f;
  for (int64_t j = m0 - 3; j < m0; ++j) {
    if (j < 0) continue;
    if (conv_row_starts(segpos, seg_kind, seq, j)) {
#pragma unroll
      for (int e = 0; e < N; ++e) h1[e] = h2[e] = 0.0f;
    }
#pragma unroll
    for (int e = 0; e < N; ++e) {
      h3[e] = h2[e];
      h2[e] = h1[e];
    }
    V::unpack(row(x, j), h1);
  }
  for (int64_t mb = m0; mb < m1; mb += kConvBatch) {
    u32x4 raw[kConvBatch];
    bool st[kConvBatch];
#pragma unroll
    for (int u = 0; u < kConvBatch; ++u) {
      const int64_t m = mb + u < m1 ? mb + u : m1 - 1;
      raw[u] = row(x, m);
      st[u] = conv_row_starts(segpos, seg_kind, seq, m);
    }
#pragma unroll
    for (int u = 0; u < kConvBatch; ++u) {
      if (mb + u < m1) {
        if (st[u]) {
#pragma unroll
          for (int e = 0; e < N; ++e) h1[e] = h2[e] = h3[e] = 0.0f;
        }
        float cur[N], o[N];
        V::unpack(raw[u], cur);
#pragma unroll
        for (int e = 0; e < N; ++e) {
          o[e] = conv4(cur[e], h1[e], h2[e], h3[e], w0[e], w1[e], w2[e], w3[e],
                       bb[e]);
          h3[e] = h2[e];
          h2[e] = h1[e];
          h1[e] = cur[e];
        }
        *reinterpret_cast<u32x4*>(out + (mb + u) * W + c) = V::pack(o);
      }
    }
  }
}

// The backward pass in the same shape: the window of x slides as above (for
// dw), a window of dout[m .. m+3] slides ahead of it (for dx), with the starts
// of rows m+1 .. m+3 deciding which of them a tap may use.  Sums for dw and
// dbias go to the chunk's plane of `partial` like the general kernel's.
template <typename T>
__global__ void __launch_bounds__(64)
conv1d_backward_k4_kernel(const T* __restrict__ dout, const T* __restrict__ x,
                          const void* __restrict__ segpos, int seg_kind,
                          const T* __restrict__ w, T* __restrict__ dx,
                          float* __restrict__ partial, int T_len, int W,
                          int64_t M, int rows) {
  using V = Vec16<T>;
  constexpr int N = V::N;
  const int c = ((int)blockIdx.y * 64 + (int)threadIdx.x) * N;
  if (c >= W) return;
  const int64_t m0 = (int64_t)blockIdx.x * rows;
  const int64_t m1 = m0 + rows < M ? m0 + rows : M;
  const SeqStarts seq(m0 >= 3 ? m0 - 3 : 0, T_len, rows + 6);
  auto row = [&](const T* base, int64_t m) {
    return *reinterpret_cast<const u32x4*>(base + m * W + c);
  };
  // a row behind the last one counts as a start (nothing beyond it is used)
  auto starts = [&](int64_t m) {
    return m >= M || conv_row_starts(segpos, seg_kind, seq, m);
  };
  float w0[N], w1[N], w2[N], w3[N];
  V::unpack(row(w, 0), w0);
  V::unpack(row(w, 1), w1);
  V::unpack(row(w, 2), w2);
  V::unpack(row(w, 3), w3);
  float h1[N], h2[N], h3[N], d0[N], d1[N], d2[N], d3[N], db[N];
#pragma unroll
  for (int e = 0; e < N; ++e)
    h1[e] = h2[e] = h3[e] = d0[e] = d1[e] = d2[e] = d3[e] = db[e] = 0.0f;
  for (int64_t j = m0 - 3; j < m0; ++j) {
    if (j < 0) continue;
    if (conv_row_starts(segpos, seg_kind, seq, j)) {
#pragma unroll
      for (int e = 0; e < N; ++e) h1[e] = h2[e] = 0.0f;
    }
#pragma unroll
    for (int e = 0; e < N; ++e) {
      h3[e] = h2[e];
      h2[e] = h1[e];
    }
    V::unpack(row(x, j), h1);
  }
  // g0 = dout[m], g1 .. g3 the rows after it; f1 .. f3: those rows start
  float g0[N], g1[N], g2[N], g3[N];
  bool f1, f2, f3;
  auto dout_row = [&](int64_t m, float (&v)[N]) {
    if (m < M) {
      V::unpack(row(dout, m), v);
    } else {
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = 0.0f;
    }
  };
  dout_row(m0, g0);
  dout_row(m0 + 1, g1);
  dout_row(m0 + 2, g2);
  f1 = starts(m0 + 1);
  f2 = starts(m0 + 2);
  for (int64_t mb = m0; mb < m1; mb += kConvBatch) {
    u32x4 xr[kConvBatch], gr[kConvBatch];
    bool st[kConvBatch], fa[kConvBatch];
#pragma unroll
    for (int u = 0; u < kConvBatch; ++u) {
      const int64_t m = mb + u < m1 ? mb + u : m1 - 1;
      xr[u] = row(x, m);
      gr[u] = row(dout, m + 3 < M ? m + 3 : M - 1);
      st[u] = conv_row_starts(segpos, seg_kind, seq, m);
      fa[u] = starts(m + 3);
    }
#pragma unroll
    for (int u = 0; u < kConvBatch; ++u) {
      const int64_t m = mb + u;
      if (m < m1) {
        if (m + 3 < M) {
          V::unpack(gr[u], g3);
        } else {
#pragma unroll
          for (int e = 0; e < N; ++e) g3[e] = 0.0f;
        }
        f3 = fa[u];
        if (st[u]) {
#pragma unroll
          for (int e = 0; e < N; ++e) h1[e] = h2[e] = h3[e] = 0.0f;
        }
        float cur[N], o[N];
        V::unpack(xr[u], cur);
        const bool ok1 = !f1, ok2 = ok1 && !f2, ok3 = ok2 && !f3;
#pragma unroll
        for (int e = 0; e < N; ++e) {
          float acc = w3[e] * g0[e];
          acc = __builtin_fmaf(w2[e], ok1 ? g1[e] : 0.0f, acc);
          acc = __builtin_fmaf(w1[e], ok2 ? g2[e] : 0.0f, acc);
          acc = __builtin_fmaf(w0[e], ok3 ? g3[e] : 0.0f, acc);
          o[e] = acc;
          d3[e] = __builtin_fmaf(cur[e], g0[e], d3[e]);  // w[3] meets x[t]
          d2[e] = __builtin_fmaf(h1[e], g0[e], d2[e]);
          d1[e] = __builtin_fmaf(h2[e], g0[e], d1[e]);
          d0[e] = __builtin_fmaf(h3[e], g0[e], d0[e]);
          db[e] += g0[e];
          h3[e] = h2[e];
          h2[e] = h1[e];
          h1[e] = cur[e];
          g0[e] = g1[e];
          g1[e] = g2[e];
          g2[e] = g3[e];
        }
        f1 = f2;
        f2 = f3;
        *reinterpret_cast<u32x4*>(dx + m * W + c) = V::pack(o);
      }
    }
  }
  float* outp = partial + (int64_t)blockIdx.x * 5 * W + c;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    outp[e] = d0[e];
    outp[(int64_t)W + e] = d1[e];
    outp[2 * (int64_t)W + e] = d2[e];
    outp[3 * (int64_t)W + e] = d3[e];
    outp[4 * (int64_t)W + e] = db[e];
  }
}

// Decode step: one thread per (batch row, channel).  All state rows are read
// into registers before anything is written, so cache_out may alias cache_in.
template <typename T>
__global__ void __launch_bounds__(256)
conv1d_step_kernel(const T* __restrict__ x, const T* cache_in,
                   const T* __restrict__ w, const T* __restrict__ bias,
                   T* __restrict__ out, T* cache_out, int B, int W, int K) {
  const int64_t total = (int64_t)B * W;
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const int c = (int)(idx % W);
    const int64_t b = idx / W;
    float st[16];  // K - 1 <= 15 state rows, oldest first
#pragma unroll
    for (int k = 0; k < 15; ++k)
      st[k] = (k < K - 1) ? load_scalar(cache_in + (b * (K - 1) + k) * W + c)
                          : 0.0f;
    const float xv = load_scalar(x + idx);
    float acc;
    if (sizeof(T) == 2 && K == 4) {
      // the bf16 kernels' width-4 arithmetic (conv4_dot of rg_common.h)
      acc = conv4_bf16(xv, st[2], st[1], st[0], load_scalar(w + c),
                       load_scalar(w + (int64_t)W + c),
                       load_scalar(w + 2 * (int64_t)W + c),
                       load_scalar(w + 3 * (int64_t)W + c),
                       load_scalar(bias + c));
    } else {
      acc = load_scalar(bias + c);
      acc = __builtin_fmaf(xv, load_scalar(w + (int64_t)(K - 1) * W + c), acc);
#pragma unroll
      for (int k = 14; k >= 0; --k)  // newest state row first
        if (k < K - 1)
          acc = __builtin_fmaf(st[k], load_scalar(w + (int64_t)k * W + c), acc);
    }
    store_scalar(out + idx, acc);
    if (cache_out) {
#pragma unroll
      for (int k = 0; k < 15; ++k)
        if (k < K - 2) store_scalar(cache_out + (b * (K - 1) + k) * W + c,
                                    st[k + 1]);
      store_scalar(cache_out + (b * (K - 1) + (K - 2)) * W + c, xv);
    }
  }
}

inline int grid_for(int64_t total, int block) {
  int64_t g = (total + block - 1) / block;
  const int64_t cap = 256 * 64;  // grid-stride loop beyond this
  return (int)(g < 1 ? 1 : (g > cap ? cap : g));
}

// whether the 16-byte kernels serve this shape
template <typename T>
bool conv_k4_fits(int K, int W, int64_t M) {
  constexpr int N = 16 / (int)sizeof(T);
  return K == 4 && W % N == 0 && (M + kConvRun - 1) / kConvRun <= 0x7fffffff &&
         (W / N + 63) / 64 <= 65535;
}

template <typename T>
hipError_t conv_prefill_t(const ConvArgs& a, hipStream_t s) {
  const int64_t total = (int64_t)a.B * a.T * a.W;
  const int64_t M = (int64_t)a.B * a.T;
  if (conv_k4_fits<T>(a.K, a.W, M)) {
    constexpr int N = 16 / (int)sizeof(T);
    const unsigned slabs = (unsigned)((a.W / N + 63) / 64);
    const unsigned waves = slabs < 16 ? slabs : 16;  // per workgroup
    const unsigned across = (slabs + waves - 1) / waves;
    // long runs where that still leaves eight waves for every SIMD
    constexpr int kLongRun = 128;
    if ((M / kLongRun) * slabs >= 8192) {
      const dim3 grid((unsigned)((M + kLongRun - 1) / kLongRun), across);
      conv1d_prefill_k4_kernel<T, kLongRun><<<grid, waves * 64, 0, s>>>(
          (const T*)a.x, a.segpos, a.seg_kind, (const T*)a.w,
          (const T*)a.bias, (T*)a.out, a.T, a.W, M);
    } else {
      const dim3 grid((unsigned)((M + kConvRun - 1) / kConvRun), across);
      conv1d_prefill_k4_kernel<T, kConvRun><<<grid, waves * 64, 0, s>>>(
          (const T*)a.x, a.segpos, a.seg_kind, (const T*)a.w,
          (const T*)a.bias, (T*)a.out, a.T, a.W, M);
    }
  } else {
    conv1d_prefill_kernel<T><<<grid_for(total, 256), 256, 0, s>>>(
        (const T*)a.x, a.segpos, a.seg_kind, (const T*)a.w,
        (const T*)a.bias, (T*)a.out, a.T, a.W, a.K, total);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !a.cache_out) return e;
  const int64_t ctotal = (int64_t)a.B * (a.K - 1) * a.W;
  conv1d_cache_tail_kernel<T><<<grid_for(ctotal, 256), 256, 0, s>>>(
      (const T*)a.x, a.segpos, a.seg_kind, (T*)a.cache_out, a.B, a.T, a.W,
      a.K);
  return hipGetLastError();
}

template <typename T>
hipError_t conv_step_t(const ConvStepArgs& a, hipStream_t s) {
  const int64_t total = (int64_t)a.B * a.W;
  conv1d_step_kernel<T><<<grid_for(total, 256), 256, 0, s>>>(
      (const T*)a.x, (const T*)a.cache_in, (const T*)a.w, (const T*)a.bias,
      (T*)a.out, (T*)a.cache_out, a.B, a.W, a.K);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_conv1d_prefill(const ConvArgs& a, int dtype, hipStream_t s) {
  return dtype == 0 ? conv_prefill_t<float>(a, s)
                    : conv_prefill_t<uint16_t>(a, s);
}

hipError_t launch_conv1d_step(const ConvStepArgs& a, int dtype,
                              hipStream_t s) {
  return dtype == 0 ? conv_step_t<float>(a, s) : conv_step_t<uint16_t>(a, s);
}

// Rows per chunk of the backward pass (see kConvBwdRows above).
static int conv1d_backward_rows(int64_t M) {
  int rows = kConvBwdRows;
  while (rows < kConvBwdMaxRows && (M + rows - 1) / rows > kConvBwdChunks)
    rows *= 2;
  return rows;
}

int conv1d_backward_chunks(int B, int T) {
  const int64_t M = (int64_t)B * T;
  const int rows = conv1d_backward_rows(M);
  return (int)((M + rows - 1) / rows);
}

hipError_t launch_conv1d_backward(const ConvBwdArgs& a, int dtype,
                                  hipStream_t s) {
  const int64_t M = (int64_t)a.B * a.T;
  const int64_t chunks = conv1d_backward_chunks(a.B, a.T);
  const int rows = conv1d_backward_rows(M);
  const int64_t cblocks = ((int64_t)a.W + 255) / 256;
  if (chunks <= 0 || chunks > 0x7fffffff || cblocks > 65535 || a.K < 2 ||
      a.K > 16)
    return hipErrorInvalidValue;
  if (dtype == 0 ? conv_k4_fits<float>(a.K, a.W, M)
                 : conv_k4_fits<uint16_t>(a.K, a.W, M)) {
    if (dtype == 0)
      conv1d_backward_k4_kernel<float>
          <<<dim3((unsigned)chunks, (unsigned)((a.W / 4 + 63) / 64)), 64, 0, s>>>(
              (const float*)a.dout, (const float*)a.x, a.segpos, a.seg_kind,
              (const float*)a.w, (float*)a.dx, a.partial, a.T, a.W, M, rows);
    else
      conv1d_backward_k4_kernel<uint16_t>
          <<<dim3((unsigned)chunks, (unsigned)((a.W / 8 + 63) / 64)), 64, 0, s>>>(
              (const uint16_t*)a.dout, (const uint16_t*)a.x, a.segpos,
              a.seg_kind, (const uint16_t*)a.w, (uint16_t*)a.dx, a.partial, a.T,
              a.W, M, rows);
    return hipGetLastError();
  }
  const dim3 grid((unsigned)chunks, (unsigned)cblocks);
  if (dtype == 0)
    conv1d_backward_kernel<float><<<grid, 256, 0, s>>>(
        (const float*)a.dout, (const float*)a.x, a.segpos, a.seg_kind,
        (const float*)a.w, (float*)a.dx, a.partial, a.T, a.W, a.K, M, rows);
  else
    conv1d_backward_kernel<uint16_t><<<grid, 256, 0, s>>>(
        (const uint16_t*)a.dout, (const uint16_t*)a.x, a.segpos, a.seg_kind,
        (const uint16_t*)a.w, (uint16_t*)a.dx, a.partial, a.T, a.W, a.K, M,
        rows);
  return hipGetLastError();
}

}  // namespace rg
