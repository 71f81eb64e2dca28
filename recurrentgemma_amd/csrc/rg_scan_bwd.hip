// Backward pass of the linear recurrence  h_t = a'_t h_{t-1} + x_t  (a' = a
// with zeros at resets), y_t = h_t:
//   g_t  = dy_t + a'_{t+1} g_{t+1}      (g_T taken as dh_last, coefficient one)
//   dx_t = g_t
//   da_t = g_t h_{t-1}  (0 at resets),  h_{-1} = h0
//   dh0  = a'_0 g_0
// i.e. the same recurrence run from the end of the sequence with the
// coefficients shifted by one step, and the product with the outputs shifted
// the other way, in one kernel: what autograd does with the loop of
// recurrentgemma/torch/layers.py:181-189, and what the reference's own
// backward is (recurrentgemma/jax/pallas.py:792-846: the forward kernel on dy
// in reverse, then da = dx * y_shifted).
//
// Lanes are channels, a workgroup takes (row, slab of 64 CH channels), its
// waves split the sequence into contiguous chunks.  Pass 1: every wave reduces
// its chunk to the pair (product of its coefficients, g at its first token
// from a zero incoming value); the pairs meet in LDS and each wave folds the
// chunks behind its own onto dh_last (the scan operator of
// recurrentgemma/jax/scan.py:161-187, from the end); pass 2: the chunk again
// from its true incoming value, writing dx and da (dy and a are read a second
// time, mostly from cache).
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBwdWaves = 16;
constexpr int kBwdRows = 8;  // rows requested before the first is used

template <typename T, int CH>
__global__ void __launch_bounds__(kBwdWaves * 64)
linear_scan_backward_kernel(ScanBwdArgs p) {
  using A = Act<T, CH>;
  __shared__ float s_p[kBwdWaves][64 * CH];
  __shared__ float s_h[kBwdWaves][64 * CH];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nslab = (p.W + 64 * CH - 1) / (64 * CH);
  const int b = blockIdx.x / nslab;
  const int slab = blockIdx.x - b * nslab;
  const int c_raw = (slab * 64 + lane) * CH;
  const bool active = c_raw < p.W;  // W % CH == 0: the whole vector is inside
  const int c = active ? c_raw : 0;
  const int T_len = p.T;
  const int64_t W = p.W;
  const int per = (T_len + kBwdWaves - 1) / kBwdWaves;
  const int t0 = wave * per < T_len ? wave * per : T_len;
  const int t1 = t0 + per < T_len ? t0 + per : T_len;

  const T* dy = (const T*)p.dy + (int64_t)b * T_len * W + c;
  const T* a = (const T*)p.a + (int64_t)b * T_len * W + c;
  const T* y = (const T*)p.y + (int64_t)b * T_len * W + c;
  T* dx = (T*)p.dx + (int64_t)b * T_len * W + c;
  T* da = (T*)p.da + (int64_t)b * T_len * W + c;
  const uint8_t* reset = (const uint8_t*)p.reset + (int64_t)b * T_len;

  // Step t multiplies g_{t+1} by a'_{t+1} (one behind the last token).  The
  // loads of a batch of rows are all issued before any value is looked at
  // (rows below the chunk are clamped into it and skipped afterwards; the
  // reset byte is applied as a select, not a branch): one memory round trip
  // per batch.
  auto coef_row = [&](int t) { return t + 1 < T_len ? t + 1 : T_len - 1; };
  auto finish_coef = [&](int t, uint8_t r, float (&coef)[CH]) {
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
      coef[ch] = t + 1 < T_len ? (r ? 0.0f : coef[ch]) : 1.0f;
  };

  // ---- pass 1: this chunk as (P, H): g at t0 = H + P * (g at t1) ----------
  float P[CH], H[CH];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    P[ch] = 1.0f;
    H[ch] = 0.0f;
  }
  for (int tb = t1; tb > t0; tb -= kBwdRows) {
    float dyv[kBwdRows][CH], coef[kBwdRows][CH];
    uint8_t rn[kBwdRows];
#pragma unroll
    for (int u = 0; u < kBwdRows; ++u) {
      const int t = tb - 1 - u > t0 ? tb - 1 - u : t0;
      A::load(dy + (int64_t)t * W, dyv[u]);
      A::load(a + (int64_t)coef_row(t) * W, coef[u]);
      rn[u] = reset[coef_row(t)];
    }
#pragma unroll
    for (int u = 0; u < kBwdRows; ++u) {
      const int t = tb - 1 - u;
      if (t >= t0) {
        finish_coef(t, rn[u], coef[u]);
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
          H[ch] = __builtin_fmaf(coef[u][ch], H[ch], dyv[u][ch]);
          P[ch] = coef[u][ch] * P[ch];
        }
      }
    }
  }
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    s_p[wave][lane * CH + ch] = P[ch];
    s_h[wave][lane * CH + ch] = H[ch];
  }
  __syncthreads();

  // ---- value coming into this chunk from the tokens behind it -------------
  float g[CH];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch)
    g[ch] = p.dh_last ? p.dh_last[(int64_t)b * W + c + ch] : 0.0f;
  for (int k = kBwdWaves - 1; k > wave; --k) {
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
      g[ch] = __builtin_fmaf(s_p[k][lane * CH + ch], g[ch],
                             s_h[k][lane * CH + ch]);
  }

  // ---- pass 2: replay, dx and da ---------------------------------------------
  float h_first[CH];  // h_{-1} in the activation dtype
#pragma unroll
  for (int ch = 0; ch < CH; ++ch)
    h_first[ch] =
        p.h0 ? A::round(p.h0[(int64_t)b * W + c + ch]) : 0.0f;
  for (int tb = t1; tb > t0; tb -= kBwdRows) {
    float dyv[kBwdRows][CH], coef[kBwdRows][CH], hp[kBwdRows][CH];
    uint8_t rn[kBwdRows], rs[kBwdRows];
#pragma unroll
    for (int u = 0; u < kBwdRows; ++u) {
      const int t = tb - 1 - u > t0 ? tb - 1 - u : t0;
      A::load(dy + (int64_t)t * W, dyv[u]);
      A::load(a + (int64_t)coef_row(t) * W, coef[u]);
      A::load(y + (int64_t)(t > 0 ? t - 1 : 0) * W, hp[u]);
      rn[u] = reset[coef_row(t)];
      rs[u] = reset[t];
    }
#pragma unroll
    for (int u = 0; u < kBwdRows; ++u) {
      const int t = tb - 1 - u;
      if (t >= t0) {
        finish_coef(t, rn[u], coef[u]);
        float gx[CH], ga[CH];
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
          g[ch] = __builtin_fmaf(coef[u][ch], g[ch], dyv[u][ch]);
          gx[ch] = A::round(g[ch]);
          const float hprev = t > 0 ? hp[u][ch] : h_first[ch];
          ga[ch] = rs[u] ? 0.0f : gx[ch] * hprev;
        }
        if (active) {
          A::store(dx + (int64_t)t * W, gx);
          A::store(da + (int64_t)t * W, ga);
        }
      }
    }
  }
  // dh0 = a'_0 g_0: the wave that holds token 0
  if (p.dh0 && t0 == 0 && t1 > 0 && active) {
    float a0[CH];
    A::load(a, a0);
    const bool r0 = reset[0] != 0;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
      p.dh0[(int64_t)b * W + c + ch] = r0 ? 0.0f : a0[ch] * g[ch];
  }
}

template <typename T, int CH>
hipError_t launch_as(const ScanBwdArgs& a, hipStream_t s) {
  const int nslab = (a.W + 64 * CH - 1) / (64 * CH);
  const int64_t blocks = (int64_t)a.B * nslab;
  if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
  linear_scan_backward_kernel<T, CH>
      <<<dim3((unsigned)blocks), kBwdWaves * 64, 0, s>>>(a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_linear_scan_backward(const ScanBwdArgs& a, int dtype,
                                       hipStream_t s) {
  if (dtype == 0)
    return a.W % 2 == 0 ? launch_as<float, 2>(a, s) : launch_as<float, 1>(a, s);
  return a.W % 2 == 0 ? launch_as<uint16_t, 2>(a, s)
                      : launch_as<uint16_t, 1>(a, s);
}

}  // namespace rg
