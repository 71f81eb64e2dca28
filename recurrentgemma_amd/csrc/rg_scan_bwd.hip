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

// The same pass with the RG-LRU's gating inside it: the backward of
// RGLRU.forward (recurrentgemma/torch/layers.py:335-360) from the gate
// pre-activations on, in one kernel.  Forward, per element (sp = softplus of
// the channel's a_param, r = document start):
//   gx = sigmoid(px), ga = sigmoid(pa), log_a = -8 ga sp, a = exp(log_a),
//   a2 = exp(2 log_a), m = r ? 1 : sqrt(1 - a2), xn = x gx m,
//   h_t = (r ? 0 : a) h_{t-1} + xn
// Backward, with g_t the gradient arriving at xn_t (the reversed recurrence
// above) and da_t = g_t h_{t-1}:
//   d_gated = g m,  d_m = g x gx,  d_(1 - a2) = d_m / sqrt(max(4 (1 - a2), 1e-6))
//                                  (SqrtBoundDerivative.backward, layers.py:225-230)
//   d_log_a = da a - 2 a2 d_(1 - a2)          (0 at document starts)
//   d_pa = -8 sp d_log_a ga (1 - ga),  d_a_param += -8 ga d_log_a sigmoid(a_param)
//   d_px = d_gated x gx (1 - gx),  dx = d_gated gx
// The coefficients a' are recomputed from pa with the forward kernels' own
// arithmetic (FAST: hardware exp2 / rcp as on their bf16 path; else expf), so
// nothing but y is kept from the forward pass.  The coefficient of step t is
// a' of token t+1, which pass 2 has just computed for that token's own gate
// gradients: it is carried in registers, not loaded again.
// Rows of the five streams requested before the first is used: eight where
// the registers allow (128 per wave at 16 waves), four for float32 with two
// channels per lane.
template <typename T, int CH>
constexpr int gate_bwd_rows() {
  return sizeof(T) == 4 && CH == 2 ? 4 : 8;
}

template <typename T, int CH, bool FAST>
__global__ void __launch_bounds__(kBwdWaves * 64)
rglru_backward_kernel(RglruBwdArgs p) {
  using A = Act<T, CH>;
  __shared__ float s_p[kBwdWaves][64 * CH];
  __shared__ float s_h[kBwdWaves][64 * CH];
  __shared__ float s_l[kBwdWaves][64 * CH];

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

  const int64_t row0 = (int64_t)b * T_len * W + c;
  const T* dy = (const T*)p.dy + row0;
  const T* xin = (const T*)p.x + row0;
  const T* pgx = (const T*)p.gx + row0;
  const T* pga = (const T*)p.ga + row0;
  const T* y = (const T*)p.y + row0;
  T* dx = (T*)p.dx + row0;
  T* dgx = (T*)p.dgx + row0;
  T* dga = (T*)p.dga + row0;
  const uint8_t* reset = (const uint8_t*)p.reset + (int64_t)b * T_len;

  float sp[CH], sig_lam[CH], decay2[CH];
  {
    float lam[CH];
    A::load((const T*)p.a_param + c, lam);
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      sp[ch] = softplus_precise(lam[ch]);
      sig_lam[ch] = sigmoid_precise(lam[ch]);
      decay2[ch] = (-8.0f * kLog2e) * sp[ch];
    }
  }
  auto sigmoid_of = [](float v) {
    return FAST ? sigmoid_fast(v) : sigmoid_precise(v);
  };
  // a (not yet zeroed at a document start) from sigmoid(pa)
  auto a_from_gate = [&](float gate_a, int ch) {
    return FAST ? __builtin_amdgcn_exp2f(gate_a * decay2[ch])
                : expf((-8.0f * gate_a) * sp[ch]);
  };
  auto coef_row = [&](int t) { return t + 1 < T_len ? t + 1 : T_len - 1; };

  // ---- pass 1: this chunk as (P, H): g at t0 = H + P * (g at t1) ----------
  float P[CH], H[CH];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    P[ch] = 1.0f;
    H[ch] = 0.0f;
  }
  for (int tb = t1; tb > t0; tb -= kBwdRows) {
    float dyv[kBwdRows][CH], pav[kBwdRows][CH];
    uint8_t rn[kBwdRows];
#pragma unroll
    for (int u = 0; u < kBwdRows; ++u) {
      const int t = tb - 1 - u > t0 ? tb - 1 - u : t0;
      A::load(dy + (int64_t)t * W, dyv[u]);
      A::load(pga + (int64_t)coef_row(t) * W, pav[u]);
      rn[u] = reset[coef_row(t)];
    }
#pragma unroll
    for (int u = 0; u < kBwdRows; ++u) {
      const int t = tb - 1 - u;
      if (t >= t0) {
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
          const float a = a_from_gate(sigmoid_of(pav[u][ch]), ch);
          const float coef = t + 1 < T_len ? (rn[u] ? 0.0f : a) : 1.0f;
          H[ch] = __builtin_fmaf(coef, H[ch], dyv[u][ch]);
          P[ch] = coef * P[ch];
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

  // ---- pass 2: replay with the gate gradients -----------------------------
  float h_first[CH], a_next[CH], lam_acc[CH];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) {
    h_first[ch] = p.h0 ? A::round(p.h0[(int64_t)b * W + c + ch]) : 0.0f;
    a_next[ch] = 1.0f;  // behind the last token: dh_last comes in as it is
    lam_acc[ch] = 0.0f;
  }
  if (t1 < T_len && t1 > t0) {
    float pav[CH];
    A::load(pga + (int64_t)t1 * W, pav);
    const bool r = reset[t1] != 0;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
      a_next[ch] = r ? 0.0f : a_from_gate(sigmoid_of(pav[ch]), ch);
  }
  constexpr int kGateBwdRows = gate_bwd_rows<T, CH>();
  for (int tb = t1; tb > t0; tb -= kGateBwdRows) {
    float dyv[kGateBwdRows][CH], hp[kGateBwdRows][CH], xv[kGateBwdRows][CH];
    float pxv[kGateBwdRows][CH], pav[kGateBwdRows][CH];
    uint8_t rs[kGateBwdRows];
#pragma unroll
    for (int u = 0; u < kGateBwdRows; ++u) {
      const int t = tb - 1 - u > t0 ? tb - 1 - u : t0;
      A::load(dy + (int64_t)t * W, dyv[u]);
      A::load(y + (int64_t)(t > 0 ? t - 1 : 0) * W, hp[u]);
      A::load(xin + (int64_t)t * W, xv[u]);
      A::load(pgx + (int64_t)t * W, pxv[u]);
      A::load(pga + (int64_t)t * W, pav[u]);
      rs[u] = reset[t];
    }
#pragma unroll
    for (int u = 0; u < kGateBwdRows; ++u) {
      const int t = tb - 1 - u;
      if (t >= t0) {
        const bool start = rs[u] != 0;
        float o_dx[CH], o_dgx[CH], o_dga[CH];
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
          g[ch] = __builtin_fmaf(a_next[ch], g[ch], dyv[u][ch]);
          const float gr = A::round(g[ch]);  // the gradient of xn as a tensor
          const float hprev = t > 0 ? hp[u][ch] : h_first[ch];
          const float gate_x = sigmoid_of(pxv[u][ch]);
          const float gate_a = sigmoid_of(pav[u][ch]);
          const float a = a_from_gate(gate_a, ch);
          const float a2 = FAST ? a * a : expf(2.0f * ((-8.0f * gate_a) * sp[ch]));
          const float om = 1.0f - a2;
          const float m =
              start ? 1.0f : (FAST ? __builtin_amdgcn_sqrtf(om) : sqrtf(om));
          const float d_gated = gr * m;
          const float d_m = gr * (xv[u][ch] * gate_x);
          const float clipped = fmaxf(4.0f * om, 1e-6f);
          const float d_om = FAST ? d_m * __builtin_amdgcn_rsqf(clipped)
                                  : d_m / sqrtf(clipped);
          const float d_log_a =
              start ? 0.0f : (gr * hprev) * a - 2.0f * a2 * d_om;
          o_dx[ch] = d_gated * gate_x;
          o_dgx[ch] = (d_gated * xv[u][ch]) * (gate_x * (1.0f - gate_x));
          o_dga[ch] = (-8.0f * sp[ch]) * d_log_a * (gate_a * (1.0f - gate_a));
          lam_acc[ch] = __builtin_fmaf(-8.0f * gate_a, d_log_a, lam_acc[ch]);
          a_next[ch] = start ? 0.0f : a;
        }
        if (active) {
          A::store(dx + (int64_t)t * W, o_dx);
          A::store(dgx + (int64_t)t * W, o_dgx);
          A::store(dga + (int64_t)t * W, o_dga);
        }
      }
    }
  }
  // dh0 = a'_0 g_0: the wave that holds token 0 (a_next is a'_0 by now)
  if (p.dh0 && t0 == 0 && t1 > 0 && active) {
#pragma unroll
    for (int ch = 0; ch < CH; ++ch)
      p.dh0[(int64_t)b * W + c + ch] = a_next[ch] * g[ch];
  }
  // gradient of a_param: this row's share, summed over the waves' chunks
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) s_l[wave][lane * CH + ch] = lam_acc[ch];
  __syncthreads();
  if (wave == 0 && active) {
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      float sum = 0.0f;
      for (int k = 0; k < kBwdWaves; ++k) sum += s_l[k][lane * CH + ch];
      p.dlam[(int64_t)b * W + c + ch] = sum * sig_lam[ch];
    }
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

template <typename T, int CH, bool FAST>
hipError_t launch_gates_as(const RglruBwdArgs& a, hipStream_t s) {
  const int nslab = (a.W + 64 * CH - 1) / (64 * CH);
  const int64_t blocks = (int64_t)a.B * nslab;
  if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
  rglru_backward_kernel<T, CH, FAST>
      <<<dim3((unsigned)blocks), kBwdWaves * 64, 0, s>>>(a);
  return hipGetLastError();
}

}  // namespace

// Two channels per lane halve the memory instructions, one channel per lane
// doubles the workgroups: the latter until there is one per CU.
static bool two_channels_per_lane(int B, int W) {
  return W % 2 == 0 && (int64_t)B * ((W + 127) / 128) >= 256;
}

hipError_t launch_rglru_backward(const RglruBwdArgs& a, int dtype,
                                 hipStream_t s) {
  const bool two = two_channels_per_lane(a.B, a.W);
  if (dtype == 0)
    return two ? launch_gates_as<float, 2, false>(a, s)
               : launch_gates_as<float, 1, false>(a, s);
  return two ? launch_gates_as<uint16_t, 2, true>(a, s)
             : launch_gates_as<uint16_t, 1, true>(a, s);
}

hipError_t launch_linear_scan_backward(const ScanBwdArgs& a, int dtype,
                                       hipStream_t s) {
  const bool two = two_channels_per_lane(a.B, a.W);
  if (dtype == 0) return two ? launch_as<float, 2>(a, s) : launch_as<float, 1>(a, s);
  return two ? launch_as<uint16_t, 2>(a, s) : launch_as<uint16_t, 1>(a, s);
}

}  // namespace rg
