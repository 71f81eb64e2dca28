/* Body of the plain-C oracle, included once per precision by rglru_ref.c with
 * REAL (float|double), SUFFIX(name) and the math macros defined.
 *
 * TEST INFRASTRUCTURE ONLY: linked/loaded by tests, the smoke check and the
 * benchmark's CPU-baseline leg; never by the shipped library.
 *
 * Scalar restatement of the reference's torch path.  All tensors are dense,
 * row-major, channel fastest.  Arithmetic is done in REAL with separate
 * multiply and add (compile with -ffp-contract=off) in the reference's order.
 */

/* Conv1D.forward, prefill branch (cache is None):
 * recurrentgemma/torch/layers.py:447-529, mask :575-607.
 * out[b,t,c] = sum over taps s=0..min(K-1,t) of w[K-1-s,c] * x[b,t-s,c] * keep,
 * keep = 0 if any of segment_pos[b,t-s+1..t] is 0; accumulated s=0,1,2,... then
 * + bias.  cache_out (nullable) [B,K-1,W] is the masked tail the reference
 * returns: x[b,t,c] * prod_{j=1..min(K-1,T-1-t)} (segment_pos[b,t+j] != 0),
 * zero-padded on the left when T < K-1 (layers.py:526-527,624-636). */
void SUFFIX(ref_conv1d_prefill)(const REAL* x, const int64_t* segpos,
                                const REAL* w, const REAL* bias, int B, int T,
                                int W, int K, REAL* out, REAL* cache_out) {
  for (int b = 0; b < B; ++b) {
    const int64_t* sp = segpos + (size_t)b * T;
    for (int t = 0; t < T; ++t) {
      for (int c = 0; c < W; ++c) {
        REAL acc = (REAL)0;
        int alive = 1;
        for (int s = 0; s < K && s <= t; ++s) {
          if (s > 0 && sp[t - s + 1] == 0) alive = 0;
          REAL v = alive ? x[((size_t)b * T + (t - s)) * W + c] : (REAL)0;
          REAL term = v * w[(size_t)(K - 1 - s) * W + c];
          acc = acc + term;
        }
        out[((size_t)b * T + t) * W + c] = acc + bias[c];
      }
    }
    if (cache_out) {
      for (int k = 0; k < K - 1; ++k) {
        int t = T - (K - 1) + k;
        for (int c = 0; c < W; ++c) {
          REAL v = (REAL)0;
          if (t >= 0) {
            int alive = 1;
            for (int j = 1; j <= K - 1 && t + j <= T - 1; ++j)
              if (sp[t + j] == 0) alive = 0;
            v = alive ? x[((size_t)b * T + t) * W + c] : (REAL)0;
          }
          cache_out[((size_t)b * (K - 1) + k) * W + c] = v;
        }
      }
    }
  }
}

/* Conv1D.forward, decode branch (cache given, one token):
 * recurrentgemma/torch/layers.py:469-474,491-529.  No masking.  Taps are
 * accumulated newest first (shift 0 is the current token). */
void SUFFIX(ref_conv1d_step)(const REAL* x, const REAL* cache, const REAL* w,
                             const REAL* bias, int B, int W, int K, REAL* out,
                             REAL* cache_out) {
  for (int b = 0; b < B; ++b) {
    for (int c = 0; c < W; ++c) {
      REAL acc = (REAL)0;
      for (int s = 0; s < K; ++s) {
        int pos = K - 1 - s; /* index into concat(cache, x) */
        REAL v = (pos == K - 1) ? x[(size_t)b * W + c]
                                : cache[((size_t)b * (K - 1) + pos) * W + c];
        acc = acc + v * w[(size_t)pos * W + c];
      }
      out[(size_t)b * W + c] = acc + bias[c];
    }
    if (cache_out) {
      for (int k = 0; k < K - 1; ++k)
        for (int c = 0; c < W; ++c)
          cache_out[((size_t)b * (K - 1) + k) * W + c] =
              (k + 1 == K - 1) ? x[(size_t)b * W + c]
                               : cache[((size_t)b * (K - 1) + k + 1) * W + c];
    }
  }
}

/* BlockDiagonalLinear.forward: recurrentgemma/torch/layers.py:127-137.
 * x [M, H*bw], w [H, bw(in), bw(out)], b [H, bw] -> y [M, H*bw]. */
void SUFFIX(ref_block_diag_linear)(const REAL* x, const REAL* w, const REAL* b,
                                   int M, int H, int bw, REAL* y) {
  for (int m = 0; m < M; ++m)
    for (int h = 0; h < H; ++h)
      for (int j = 0; j < bw; ++j) {
        REAL acc = (REAL)0;
        for (int i = 0; i < bw; ++i)
          acc += x[(size_t)m * H * bw + h * bw + i] *
                 w[((size_t)h * bw + i) * bw + j];
        y[(size_t)m * H * bw + h * bw + j] = acc + b[(size_t)h * bw + j];
      }
}

/* RGLRU.forward + rnn_scan: recurrentgemma/torch/layers.py:313-365,140-191.
 * x is the conv output [B,T,W]; h0 nullable [B,W]; y [B,T,W]; h_last [B,W].
 * Gate pre-activations gx_pre/ga_pre [B,T,W] are given (from
 * ref_block_diag_linear) so that this function is the elementwise + scan part.
 * The T == 1 / h0 == NULL special case of rnn_scan (layers.py:172-173) gives
 * the same numbers as the general recurrence from h = 0, so it is not
 * special-cased here. */
void SUFFIX(ref_rglru_scan)(const REAL* x, const REAL* gx_pre,
                            const REAL* ga_pre, const int64_t* segpos,
                            const REAL* a_param, const REAL* h0, int B, int T,
                            int W, REAL* y, REAL* h_last) {
  for (int b = 0; b < B; ++b)
    for (int c = 0; c < W; ++c) {
      REAL ap = a_param[c];
      /* softplus with torch's threshold of 20 */
      REAL sp = ap > (REAL)20 ? ap : R_LOG1P(R_EXP(ap));
      REAL h = h0 ? h0[(size_t)b * W + c] : (REAL)0;
      for (int t = 0; t < T; ++t) {
        size_t i = ((size_t)b * T + t) * W + c;
        int reset = segpos[(size_t)b * T + t] == 0;
        REAL gate_x = (REAL)1 / ((REAL)1 + R_EXP(-gx_pre[i]));
        REAL gate_a = (REAL)1 / ((REAL)1 + R_EXP(-ga_pre[i]));
        REAL log_a = (REAL)-8 * gate_a * sp;
        REAL a = R_EXP(log_a);
        REAL a_sq = R_EXP((REAL)2 * log_a);
        REAL gated = x[i] * gate_x;
        REAL mult = reset ? (REAL)1 : R_SQRT((REAL)1 - a_sq);
        REAL xn = gated * mult;
        if (reset) a = (REAL)0;
        h = a * h + xn;
        y[i] = h;
      }
      if (h_last) h_last[(size_t)b * W + c] = h;
    }
}
