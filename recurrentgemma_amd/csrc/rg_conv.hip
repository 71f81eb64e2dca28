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
// A thread owns one channel and a run of kConvBwdRows consecutive flattened
// rows (b, t): it writes dx for them and leaves its sums of dw and dbias in
// `partial` [row chunks][K + 1][W] (float32), which the caller adds up.  The
// neighbouring rows it re-reads come from cache.
constexpr int kConvBwdRows = 32;

template <typename T>
__global__ void __launch_bounds__(256)
conv1d_backward_kernel(const T* __restrict__ dout, const T* __restrict__ x,
                       const void* __restrict__ segpos, int seg_kind,
                       const T* __restrict__ w, T* __restrict__ dx,
                       float* __restrict__ partial, int T_len, int W, int K,
                       int64_t M) {
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int64_t m0 = (int64_t)blockIdx.x * kConvBwdRows;
  const int64_t m1 = m0 + kConvBwdRows < M ? m0 + kConvBwdRows : M;
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
    float acc = load_scalar(bias + c);
    acc = __builtin_fmaf(xv, load_scalar(w + (int64_t)(K - 1) * W + c), acc);
#pragma unroll
    for (int k = 14; k >= 0; --k)  // newest state row first
      if (k < K - 1)
        acc = __builtin_fmaf(st[k], load_scalar(w + (int64_t)k * W + c), acc);
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

template <typename T>
hipError_t conv_prefill_t(const ConvArgs& a, hipStream_t s) {
  const int64_t total = (int64_t)a.B * a.T * a.W;
  conv1d_prefill_kernel<T><<<grid_for(total, 256), 256, 0, s>>>(
      (const T*)a.x, a.segpos, a.seg_kind, (const T*)a.w,
      (const T*)a.bias, (T*)a.out, a.T, a.W, a.K, total);
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

int conv1d_backward_chunks(int B, int T) {
  return (int)(((int64_t)B * T + kConvBwdRows - 1) / kConvBwdRows);
}

hipError_t launch_conv1d_backward(const ConvBwdArgs& a, int dtype,
                                  hipStream_t s) {
  const int64_t M = (int64_t)a.B * a.T;
  const int64_t chunks = conv1d_backward_chunks(a.B, a.T);
  const int64_t cblocks = ((int64_t)a.W + 255) / 256;
  if (chunks <= 0 || chunks > 0x7fffffff || cblocks > 65535 || a.K < 2 ||
      a.K > 16)
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)chunks, (unsigned)cblocks);
  if (dtype == 0)
    conv1d_backward_kernel<float><<<grid, 256, 0, s>>>(
        (const float*)a.dout, (const float*)a.x, a.segpos, a.seg_kind,
        (const float*)a.w, (float*)a.dx, a.partial, a.T, a.W, a.K, M);
  else
    conv1d_backward_kernel<uint16_t><<<grid, 256, 0, s>>>(
        (const uint16_t*)a.dout, (const uint16_t*)a.x, a.segpos, a.seg_kind,
        (const uint16_t*)a.w, (uint16_t*)a.dx, a.partial, a.T, a.W, a.K, M);
  return hipGetLastError();
}

}  // namespace rg
