// Fused Conv1D(width 4) + RG-LRU gating + linear recurrence for gfx950.
//
// Work decomposition.  Lanes map to channels (CH adjacent channels per lane),
// so every global access of a wave is one contiguous row segment.  A workgroup
// owns one batch row and one slab of 64*CH channels and walks the sequence in
// steps of nw*kL tokens (nw = waves in the group).  Inside a step, wave v
// takes the kL consecutive tokens [v*kL, (v+1)*kL):
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
// The carry into the next step is the last wave's final h.  Tokens past the
// end of the sequence are the operator's identity (1, 0).  A document start
// (segment_pos == 0) sets a = 0 and the input scale to 1, and zeroes the conv
// history, which is exactly the reference's masking rule.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kL = 16;     // tokens per wave per step
constexpr int kMaxNW = 8;  // waves per workgroup

template <int CH>
struct ChanConst {
  float w0[CH], w1[CH], w2[CH], w3[CH], bias[CH];
  float decay[CH];  // FAST: -8 softplus(L) log2(e);  precise: softplus(L)
};

// Phase 1 for one wave.  CHECK=false is the straight-line case: all kL tokens
// inside the sequence and no document start among them.
template <typename T, int CH, bool CONV, bool FAST, bool PLAIN, bool CHECK>
__device__ __forceinline__ void phase1(
    const char* __restrict__ xrow, const char* __restrict__ gxrow,
    const char* __restrict__ garow, uint32_t lane_bytes, int64_t row_bytes,
    int t0, int T_len, uint32_t starts,
    const ChanConst<CH>& k, float (&hist)[3][CH], float (&a_)[kL][CH],
    float (&xn_)[kL][CH], float (&P)[CH], float (&H)[CH]) {
  using A = Act<T, CH>;
  // All loads of the wave's kL tokens are issued before any arithmetic so that
  // 3*kL row segments per wave are in flight; the (a, xn) results then take
  // over the registers of the raw inputs.
  typename A::Raw xr[kL], gxr[kL], gar[kL];
#pragma unroll
  for (int i = 0; i < kL; ++i) {
    const int t = t0 + i;
    // wave-uniform row address + 32-bit lane offset
    const int64_t off =
        (int64_t)(CHECK ? (t < T_len ? t : T_len - 1) : t) * row_bytes;
    xr[i] = A::load_raw((const T*)(xrow + off + lane_bytes));
    if (!PLAIN) gxr[i] = A::load_raw((const T*)(gxrow + off + lane_bytes));
    gar[i] = A::load_raw((const T*)(garow + off + lane_bytes));
  }
#pragma unroll
  for (int i = 0; i < kL; ++i) {
    const int t = t0 + i;
    const bool valid = !CHECK || (t < T_len);
    const bool start = CHECK && ((starts >> (i + 3)) & 1u);
    float xv[CH], gxv[CH], gav[CH];
    A::unpack(xr[i], xv);
    if (!PLAIN) A::unpack(gxr[i], gxv);
    A::unpack(gar[i], gav);
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      float xc;
      if (CONV) {
        if (start) hist[0][ch] = hist[1][ch] = hist[2][ch] = 0.0f;
        xc = A::round(conv4(xv[ch], hist[0][ch], hist[1][ch], hist[2][ch],
                            k.w0[ch], k.w1[ch], k.w2[ch], k.w3[ch],
                            k.bias[ch]));
        hist[2][ch] = hist[1][ch];
        hist[1][ch] = hist[0][ch];
        hist[0][ch] = xv[ch];
      } else {
        xc = xv[ch];
      }
      float a, mult, gate_x;
      if (PLAIN) {
        a = gav[ch];
        mult = 1.0f;
        gate_x = 1.0f;
      } else if (FAST) {
        gate_x = sigmoid_fast(gxv[ch]);
        const float gate_a = sigmoid_fast(gav[ch]);
        a = __builtin_amdgcn_exp2f(gate_a * k.decay[ch]);
        mult = __builtin_amdgcn_sqrtf(__builtin_fmaf(-a, a, 1.0f));
      } else {
        gate_x = sigmoid_precise(gxv[ch]);
        const float gate_a = sigmoid_precise(gav[ch]);
        const float log_a = (-8.0f * gate_a) * k.decay[ch];
        a = expf(log_a);
        mult = sqrtf(1.0f - expf(2.0f * log_a));
      }
      if (start) {
        a = 0.0f;
        mult = 1.0f;
      }
      float xn = PLAIN ? xc : (xc * gate_x) * mult;
      if (!valid) {
        a = 1.0f;
        xn = 0.0f;
      }
      a_[i][ch] = a;
      xn_[i][ch] = xn;
      H[ch] = __builtin_fmaf(a, H[ch], xn);
      P[ch] = P[ch] * a;
    }
  }
}

template <typename T, int CH, bool CONV, bool FAST, bool PLAIN>
__global__ void __launch_bounds__(kMaxNW* kWave, (sizeof(T) == 2 ? 4 : 2))
lru_scan_kernel(ScanArgs p) {
  using A = Act<T, CH>;
  __shared__ float agg[2][kMaxNW][kWave][2 * CH];  // (P.., Hloc..) per lane
  __shared__ float carry_s[2][kWave][CH];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nw = blockDim.x >> 6;
  const int T_len = p.T;
  const int64_t W = p.W;
  const int nslab = (p.W + kWave * CH - 1) / (kWave * CH);
  const int b = blockIdx.x / nslab;
  const int slab = blockIdx.x - b * nslab;
  const int c_raw = (slab * kWave + lane) * CH;
  const bool active = c_raw < p.W;  // W % CH == 0, so the whole vector is in
  const int c = active ? c_raw : 0;

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
    } else {
      k.w0[ch] = k.w1[ch] = k.w2[ch] = k.w3[ch] = k.bias[ch] = 0.0f;
    }
    if (PLAIN) {
      k.decay[ch] = 0.0f;
    } else {
      const float sp =
          softplus_precise(load_scalar((const T*)p.a_param + c + ch));
      k.decay[ch] = FAST ? (-8.0f * kLog2e) * sp : sp;
    }
  }

  const int64_t row0 = (int64_t)b * T_len;
  const int64_t row_bytes = W * (int64_t)sizeof(T);
  const uint32_t lane_bytes = (uint32_t)c * (uint32_t)sizeof(T);
  // wave-uniform pointers to token 0 of this batch row
  const char* xrow = (const char*)p.x + row0 * row_bytes;
  const char* gxrow = (const char*)p.gx + row0 * row_bytes;
  const char* garow = (const char*)p.ga + row0 * row_bytes;
  char* yrow = (char*)p.y + row0 * row_bytes;

  float h_first[CH];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch)
    h_first[ch] = p.h0 ? p.h0[(int64_t)b * W + c + ch] : 0.0f;

  const int span = nw * kL;
  float h[CH];
#pragma unroll
  for (int ch = 0; ch < CH; ++ch) h[ch] = h_first[ch];

  for (int step = 0, tb = 0; tb < T_len; ++step, tb += span) {
    const int buf = step & 1;
    const int t0 = tb + wave * kL;
    const bool any = t0 < T_len;
    float a_[kL][CH], xn_[kL][CH], P[CH], H[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      P[ch] = 1.0f;
      H[ch] = 0.0f;
    }
    if (any) {
      // bit j <-> token t0-3+j starts a document (only tokens inside the row;
      // the three look-back tokens matter only for the conv history).
      // Lane j looks at token t0-3+j: one coalesced load and one ballot for
      // the whole wave instead of kL+3 dependent loads.
      bool st = false;
      {
        const int t = t0 - 3 + lane;
        if (lane < kL + 3 && (CONV || lane >= 3) && t >= 0 && t < T_len)
          st = is_doc_start(p.segpos, p.seg_kind, row0 + t);
      }
      const uint32_t starts = (uint32_t)__ballot(st);
      float hist[3][CH];
      if (CONV) {
#pragma unroll
        for (int s = 1; s <= 3; ++s) {
          const int t = t0 - s;
          float v[CH];
          A::load((const T*)(xrow + (int64_t)(t < 0 ? 0 : t) * row_bytes +
                             lane_bytes), v);
#pragma unroll
          for (int ch = 0; ch < CH; ++ch) hist[s - 1][ch] = t < 0 ? 0.0f : v[ch];
        }
        // a document start at t0-1 hides x[t0-2], x[t0-3]; one at t0-2 hides
        // x[t0-3].
        if (starts & 4u) {
#pragma unroll
          for (int ch = 0; ch < CH; ++ch) hist[1][ch] = hist[2][ch] = 0.0f;
        }
        if (starts & 2u) {
#pragma unroll
          for (int ch = 0; ch < CH; ++ch) hist[2][ch] = 0.0f;
        }
      } else {
#pragma unroll
        for (int ch = 0; ch < CH; ++ch)
          hist[0][ch] = hist[1][ch] = hist[2][ch] = 0.0f;
      }
      const bool plain = (t0 + kL <= T_len) && ((starts >> 3) == 0u);
      if (plain)
        phase1<T, CH, CONV, FAST, PLAIN, false>(xrow, gxrow, garow, lane_bytes,
                                                row_bytes, t0, T_len, starts, k,
                                                hist, a_, xn_, P, H);
      else
        phase1<T, CH, CONV, FAST, PLAIN, true>(xrow, gxrow, garow, lane_bytes,
                                               row_bytes, t0, T_len, starts, k,
                                               hist, a_, xn_, P, H);
    }

    // exchange
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
      agg[buf][wave][lane][ch] = P[ch];
      agg[buf][wave][lane][CH + ch] = H[ch];
    }
    __syncthreads();
    if (step > 0) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) h[ch] = carry_s[buf ^ 1][lane][ch];
    }
    for (int v = 0; v < wave; ++v) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch)
        h[ch] = __builtin_fmaf(agg[buf][v][lane][ch], h[ch],
                               agg[buf][v][lane][CH + ch]);
    }

    // phase 2
    if (any) {
#pragma unroll
      for (int i = 0; i < kL; ++i) {
        float out[CH];
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
          h[ch] = __builtin_fmaf(a_[i][ch], h[ch], xn_[i][ch]);
          out[ch] = h[ch];
        }
        if (t0 + i < T_len && active)
          A::store((T*)(yrow + (int64_t)(t0 + i) * row_bytes + lane_bytes), out);
      }
    }
    if (wave == nw - 1) {
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) carry_s[buf][lane][ch] = h[ch];
    }
  }

  // The last wave's h after the final step is h_{T-1}.
  if (wave == nw - 1 && p.h_last && active) {
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) p.h_last[(int64_t)b * W + c + ch] = h[ch];
  }

  // Masked conv state: rows T-3..T-1 of x, each zeroed if a document starts in
  // a later position of the row; rows before the sequence start are zero.
  if (CONV && p.cache_out && wave == 0 && active) {
    T* cache = (T*)p.cache_out + (int64_t)b * 3 * W + c;
    bool later_start = false;
#pragma unroll
    for (int kk = 2; kk >= 0; --kk) {
      const int t = T_len - 3 + kk;
      float v[CH];
#pragma unroll
      for (int ch = 0; ch < CH; ++ch) v[ch] = 0.0f;
      if (t >= 0) {
        if (!later_start)
          A::load((const T*)(xrow + (int64_t)t * row_bytes + lane_bytes), v);
        if (is_doc_start(p.segpos, p.seg_kind, row0 + t))
          later_start = true;
      }
      A::store(cache + (int64_t)kk * W, v);
    }
  }
}

template <typename T, int CH, bool CONV, bool FAST, bool PLAIN>
hipError_t launch_t(const ScanArgs& a, hipStream_t s) {
  const int nslab = (a.W + kWave * CH - 1) / (kWave * CH);
  int nw = 1;
  while (nw < kMaxNW && nw * kL < a.T) nw *= 2;
  const int64_t blocks = (int64_t)a.B * nslab;
  if (blocks > 0x7fffffff) return hipErrorInvalidValue;
  lru_scan_kernel<T, CH, CONV, FAST, PLAIN>
      <<<dim3((unsigned)blocks), dim3(nw * kWave), 0, s>>>(a);
  return hipGetLastError();
}

template <typename T, bool FAST>
hipError_t launch_dt(const ScanArgs& a, hipStream_t s) {
  // Two channels per lane need the channel count even (every row then starts
  // on a vector boundary; base pointers are checked by the caller).
  const bool vec2 = (a.W % 2) == 0;
  if (a.plain)
    return vec2 ? launch_t<T, 2, false, FAST, true>(a, s)
                : launch_t<T, 1, false, FAST, true>(a, s);
  if (a.apply_conv)
    return vec2 ? launch_t<T, 2, true, FAST, false>(a, s)
                : launch_t<T, 1, true, FAST, false>(a, s);
  return vec2 ? launch_t<T, 2, false, FAST, false>(a, s)
              : launch_t<T, 1, false, FAST, false>(a, s);
}

}  // namespace

hipError_t launch_lru_scan(const ScanArgs& a, int dtype, hipStream_t s) {
  return dtype == 0 ? launch_dt<float, false>(a, s)
                    : launch_dt<uint16_t, true>(a, s);
}

}  // namespace rg
