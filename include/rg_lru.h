/* rg_lru.h -- C ABI of the MI355X (gfx950) Conv1D + RG-LRU recurrent-block core.
 *
 * The reference (google-deepmind/recurrentgemma, torch path) has no FFI: its
 * boundary for this path is the Python module surface of
 * recurrentgemma/torch/layers.py (Conv1D, BlockDiagonalLinear, RGLRU, rnn_scan).
 * Each entry point below names the reference function it stands in for.
 *
 * Conventions
 *  - All pointers are DEVICE pointers to dense row-major tensors, channel
 *    fastest: activations [B,T,W], segment positions [B,T], RG-LRU state [B,W]
 *    (always float32), conv state [B,K-1,W].
 *  - `dtype` is the activation/parameter element type (RG_DTYPE_*): the
 *    reference requires parameters and activations to share one dtype.
 *  - `stream` is a hipStream_t passed as void*.  Calls only enqueue work on it:
 *    no synchronisation, no allocation, no use of any other stream.
 *  - The library never keeps a pointer after a call returns and never frees or
 *    allocates caller-visible memory.
 *  - Return value: RG_OK or a negative RG_ERR_* code; rg_last_error() then
 *    gives a thread-local, human-readable reason.  No C++ exception crosses
 *    this boundary.  Arguments are validated before anything is launched.
 *  - Inputs are never modified (the reference's Conv1D multiplies its input by
 *    the document mask in place, layers.py:497-508; that side effect is NOT
 *    reproduced, the masked conv state it leads to is).
 */
#ifndef RG_LRU_H_
#define RG_LRU_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RG_ABI_VERSION 1

enum {
  RG_OK = 0,
  RG_ERR_BAD_ARG = -1,     /* null pointer, non-positive size, misalignment  */
  RG_ERR_UNSUPPORTED = -2, /* shape or dtype this build has no kernel for     */
  RG_ERR_LAUNCH = -3,      /* hipLaunch / runtime error                       */
  RG_ERR_WORKSPACE = -4    /* workspace missing or too small                  */
};

enum { RG_DTYPE_F32 = 0, RG_DTYPE_BF16 = 1 };

#define RG_MAX_CONV_WIDTH 16

/* Library identification. */
int rg_abi_version(void);
const char* rg_last_error(void);

/* Conv1D.forward, prefill branch (cache is None):
 * recurrentgemma/torch/layers.py:447-529 (mask :575-607, cache :526-527).
 *   out[b,t,c] = bias[c] + sum_{s=0..min(K-1,t)} w[K-1-s,c] * x[b,t-s,c] * keep
 *   keep = 0 iff some segpos[b,t-s+1..t] == 0.
 * cache_out (nullable, [B,K-1,W]) receives the reference's masked tail
 *   x[b,t,c] * prod_{j=1..min(K-1,T-1-t)} (segpos[b,t+j] != 0), t = T-K+1..T-1,
 * zero-filled on the left when T < K-1.  2 <= K <= RG_MAX_CONV_WIDTH. */
int rg_conv1d_prefill(const void* x, const void* segpos, int segpos_is_i64,
                      const void* w, const void* bias, void* out,
                      void* cache_out, int B, int T, int W, int K, int dtype,
                      void* stream);

/* Backward pass of rg_conv1d_prefill (Conv1D.forward without a cache under
 * autograd, recurrentgemma/torch/layers.py:477-520): from dout [B,T,W], the
 * gradient of the conv output, dx [B,T,W] (`dtype`) and, in `partial`
 * (float32 [chunks][temporal_width + 1][W], chunks =
 * rg_conv1d_backward_workspace_bytes / ((temporal_width + 1) * W * 4)), per
 * chunk of rows the sums that add up to the gradient of w (planes 0 ..
 * temporal_width-1, laid out like w) and of b (last plane); the caller sums
 * over the chunks (chunks of 32 rows of [B*T] while that leaves at most 512 of
 * them, of 64, 128 or 256 rows beyond).  Taps cut by a document start carry no
 * gradient, as in the forward pass.  2 <= temporal_width <= RG_MAX_CONV_WIDTH. */
size_t rg_conv1d_backward_workspace_bytes(int B, int T, int W,
                                          int temporal_width);
int rg_conv1d_backward(const void* dout, const void* x, const void* segpos,
                       int segpos_is_i64, const void* w, void* dx,
                       void* partial, size_t partial_bytes, int B, int T, int W,
                       int temporal_width, int dtype, void* stream);

/* Conv1D.forward, decode branch (cache given, exactly one token):
 * recurrentgemma/torch/layers.py:469-474,491-529,531-550.  No document mask.
 *   out[b,c] = bias[c] + sum_k w[k,c] * concat(cache_in, x)[b,k,c]
 *   cache_out = concat(cache_in, x)[:,1:]      (may alias cache_in)
 * x,out [B,1,W]; cache_in/out [B,K-1,W] in the activation dtype. */
int rg_conv1d_step(const void* x, const void* cache_in, const void* w,
                   const void* bias, void* out, void* cache_out, int B, int W,
                   int K, int dtype, void* stream);

/* BlockDiagonalLinear.forward: recurrentgemma/torch/layers.py:127-137.
 *   y[m, h*bw + j] = b[h,j] + sum_i x[m, h*bw + i] * w[h,i,j]
 * x,y [M, H*bw]; w [H,bw,bw] laid out [head, in, out]; b [H,bw]. */
int rg_block_diag_linear(const void* x, const void* w, const void* b, void* y,
                         int64_t M, int H, int bw, int dtype, void* stream);

/* Weight and bias gradients of the two gate projections of RGLRU.forward
 * (what autograd forms for recurrentgemma/torch/layers.py:134-136, called at
 * :338-339 on the same x) from the gradients of their outputs:
 *   dw_g[h,i,j] = sum_m x[m, h*256 + i] * dy_g[m, h*256 + j]
 *   db_g[h,j]   = sum_m dy_g[m, h*256 + j]            g = input gate, a gate
 * x, dgx, dga [M, W] (M = B*T rows); dwx, dwa [H,256,256] laid out like the
 * weights; dbx, dba [H,256] (both nullable, together).  bf16, W == 256 * H
 * (RG_ERR_UNSUPPORTED otherwise: the caller keeps its own batched product);
 * sums in float32 over row ranges whose partial results meet in `workspace`
 * (rg_gates_weight_grads_workspace_bytes, 16-byte aligned) in a fixed order,
 * one rounding: the same bits on every run. */
size_t rg_gates_weight_grads_workspace_bytes(int64_t M, int W, int H);
int rg_gates_weight_grads(const void* x, const void* dgx, const void* dga,
                          void* dwx, void* dwa, void* dbx, void* dba,
                          void* workspace, size_t workspace_bytes, int64_t M,
                          int W, int H, int dtype, void* stream);

/* The two gate projections of RGLRU.forward (layers.py:338-339, before the
 * sigmoid) in one pass over x:
 *   gx_pre = input_gate(xc), ga_pre = a_gate(xc), both [B,T,W] in `dtype`.
 * apply_conv == 0: xc = x (x is already the conv output).
 * apply_conv != 0: xc = Conv1D(x) computed on load with the width-4 kernel
 *   conv_w [4,W], conv_b [W] and the segpos mask (prefill semantics of
 *   rg_conv1d_prefill, rounded to `dtype` like the reference's module output);
 *   segpos must then be given.
 * bw = W / H.  On the matrix cores: bf16 with 128 <= bw <= 256 (bw a multiple
 * of 8; weights held in registers, x tiles staged through LDS, narrower heads
 * padded to the 256-wide tile inside the kernel) and float32 with bw == 256
 * (true float32 products, v_mfma_f32_32x32x2_f32).  Any other combination runs
 * on a plain FMA kernel with fp32 accumulation. */
int rg_gates_gemm(const void* x, int apply_conv, const void* segpos,
                  int segpos_is_i64, const void* conv_w, const void* conv_b,
                  const void* w_x, const void* b_x, const void* w_a,
                  const void* b_a, void* gx_pre, void* ga_pre, int B, int T,
                  int W, int H, int dtype, void* stream);

/* RGLRU.forward after the gate projections + rnn_scan, optionally with the
 * width-4 Conv1D fused in front: recurrentgemma/torch/layers.py:335-365 and
 * :140-191 (+ :447-529 when apply_conv).
 *   xc      = apply_conv ? Conv1D(x) : x
 *   r       = segpos == 0
 *   gx, ga  = sigmoid(gx_pre), sigmoid(ga_pre)
 *   a       = r ? 0 : exp(-8 * ga * softplus(a_param))
 *   xn      = xc * gx * (r ? 1 : sqrt(1 - a^2))
 *   h_t     = a_t * h_{t-1} + xn_t     (float32 state, h_{-1} = h0 or 0)
 *   y_t     = h_t rounded to `dtype`
 * h0 (nullable) and h_last (nullable) are float32 [B,W]; h_last may alias h0.
 * conv_cache_out (nullable, only with apply_conv) is the [B,3,W] masked tail
 * described at rg_conv1d_prefill.  The recurrence over T runs as a chunked
 * parallel scan (per-wave local scans of (a, xn) pairs, carries combined
 * across the waves of a workgroup). */
int rg_lru_scan_fused(const void* x, int apply_conv, const void* conv_w,
                      const void* conv_b, const void* gx_pre,
                      const void* ga_pre, const void* a_param,
                      const void* segpos, int segpos_is_i64, const void* h0,
                      void* y, void* h_last, void* conv_cache_out, int B, int T,
                      int W, int dtype, void* stream);

/* rnn_scan: recurrentgemma/torch/layers.py:140-191.
 *   h_t = (reset_t ? 0 : a_t) * h_{t-1} + x_t,  y_t = h_t rounded to `dtype`
 * x, a, y [B,T,W] in `dtype`; reset [B,T] bytes (non-zero = reset, the memory
 * of a torch.bool tensor); h0 (nullable) / h_last (nullable) float32 [B,W].
 * Same chunked scan kernel as rg_lru_scan_fused without the gating. */
int rg_linear_scan(const void* x, const void* a, const void* reset,
                   const void* h0, void* y, void* h_last, int B, int T, int W,
                   int dtype, void* stream);

/* Backward pass of rnn_scan (what autograd computes through the loop of
 * recurrentgemma/torch/layers.py:181-189; the reference's own formulation is
 * recurrentgemma/jax/pallas.py:792-846: the recurrence on dy from the end of
 * the sequence, then da = dx * y shifted by one step).  With a' = a zeroed at
 * resets:
 *   g_t = dy_t + a'_{t+1} g_{t+1}  (the term behind the last token is dh_last)
 *   dx_t = g_t,  da_t = g_t * h_{t-1} (0 at resets; h_{-1} = h0),  dh0 = a'_0 g_0
 * dy, a, y, dx, da [B,T,W] in `dtype` (y: the forward output), reset [B,T]
 * bytes, h0 / dh_last / dh0 (all nullable) float32 [B,W].  The recurrence runs
 * in float32; dx is g rounded to `dtype`, da the product of the rounded g and
 * y rounded again.  dx may alias dy; no other aliasing. */
int rg_linear_scan_backward(const void* dy, const void* a, const void* reset,
                            const void* y, const void* h0, const void* dh_last,
                            void* dx, void* da, void* dh0, int B, int T, int W,
                            int dtype, void* stream);

/* Backward pass of RGLRU.forward from the gate pre-activations on
 * (recurrentgemma/torch/layers.py:335-360 under autograd, with
 * SqrtBoundDerivative.backward :225-230 and the reversed recurrence of
 * recurrentgemma/jax/pallas.py:792-846) in one kernel.  Inputs as
 * rg_lru_scan_fused without the conv takes them: x [B,T,W] (the conv output),
 * gx_pre / ga_pre [B,T,W], a_param [W], all `dtype`; reset [B,T] bytes
 * (segment_pos == 0); y the forward output; h0 / dh_last nullable float32
 * [B,W]; dy the gradient of y.  Outputs: dx, dgx_pre, dga_pre [B,T,W] in
 * `dtype`; d_a_param_rows float32 [B,W], each row's share of a_param's
 * gradient (the caller sums over B); dh0 (nullable) float32 [B,W].  The gates
 * and coefficients are recomputed from the pre-activations with the forward
 * kernels' arithmetic; everything runs in float32 and is rounded once per
 * output.  No output may alias an input or another output. */
int rg_rglru_backward(const void* dy, const void* x, const void* gx_pre,
                      const void* ga_pre, const void* a_param,
                      const void* reset, const void* y, const void* h0,
                      const void* dh_last, void* dx, void* dgx_pre,
                      void* dga_pre, void* d_a_param_rows, void* dh0, int B,
                      int T, int W, int dtype, void* stream);

/* The two scans above for few rows and channels: one workgroup per (row, slab
 * of 256 or 128 channels) leaves most of the GPU idle when B * W / 256 is
 * small (a single prompt: 10 to 16 workgroups).  These variants cut every
 * sequence into chunks that run as workgroups of their own: a first pass
 * reduces each chunk to (product of its a_t, its state from a zero start), a
 * second pass chains those into its chunk's incoming state, runs the chunk
 * from there and writes y -- the scan operator is associative
 * (recurrentgemma/jax/scan.py:161-187), this is the kernel's own cross-wave
 * carry one level up.  Twice the reads, none of the idling.
 * rg_scan_split_workspace_bytes is 0 for shapes
 * that gain nothing (then the calls behave exactly like the plain ones and
 * workspace may be null); otherwise workspace (16-byte aligned, that many
 * bytes) is required.  Same arguments and results otherwise (fp32 1e-5, the
 * float32 state is combined in a different order). */
size_t rg_scan_split_workspace_bytes(int B, int T, int W);
int rg_lru_scan_fused_split(const void* x, int apply_conv, const void* conv_w,
                            const void* conv_b, const void* gx_pre,
                            const void* ga_pre, const void* a_param,
                            const void* segpos, int segpos_is_i64,
                            const void* h0, void* y, void* h_last,
                            void* conv_cache_out, void* workspace,
                            size_t workspace_bytes, int B, int T, int W,
                            int dtype, void* stream);
int rg_linear_scan_split(const void* x, const void* a, const void* reset,
                         const void* h0, void* y, void* h_last, void* workspace,
                         size_t workspace_bytes, int B, int T, int W, int dtype,
                         void* stream);

/* Prefill of the conv -> RG-LRU core in ONE launch, as RecurrentBlock.forward
 * chains the two modules without a cache (recurrentgemma/torch/modules.py:
 * 632-643: Conv1D.forward layers.py:447-529, then RGLRU.forward :313-365 with
 * rnn_scan :140-191).  x, y [B,T,W]; segpos [B,T]; conv_w [4,W], conv_b [W];
 * w_x, w_a [H,W/H,W/H], b_x, b_a [H,W/H]; a_param [W]; h0 (nullable) and
 * h_last (nullable) float32 [B,W]; conv_cache_out (nullable) [B,3,W], the
 * masked tail described at rg_conv1d_prefill.  Same arithmetic as
 * rg_gates_gemm(apply_conv) followed by rg_lru_scan_fused(apply_conv), but the
 * conv output and the gate pre-activations stay on chip, the latter in
 * float32 (the two-call form rounds them to bf16 on their way through memory,
 * so the two agree to a bf16 unit or two, not bit for bit): one workgroup of
 * four waves, one per SIMD, per (b, head) walks the sequence in 64-token tiles
 * (x -> LDS by the memory pipe, conv -> LDS, bf16 MFMA on weights resident in
 * accumulation registers, gates, in-register recurrence).  w_packed (nullable) is the
 * output of rg_pack_gate_weights for the same w_x / w_a (see below): with it
 * the kernel skips its own re-layout of the weights.  Returns RG_ERR_UNSUPPORTED
 * unless dtype is bf16, W/H == 256 and T*W*2 < 2^31; callers then use the
 * two-call form. */
int rg_recurrent_prefill(const void* x, const void* segpos, int segpos_is_i64,
                         const void* conv_w, const void* conv_b,
                         const void* w_x, const void* b_x, const void* w_a,
                         const void* b_a, const void* w_packed,
                         const void* a_param, const void* h0, void* y,
                         void* h_last, void* conv_cache_out, int B, int T,
                         int W, int H, int dtype, void* stream);

/* rg_recurrent_prefill for few (row, head) pairs: one workgroup per pair
 * leaves most of the GPU idle below 256 pairs, so the sequences are cut into
 * chunks of whole 64-token tiles that run as workgroups of their own, in two
 * launches.  The first runs chunk 0 for real (from h0, writing y) beside
 * chunks 1 .. n-2 from a zero state, of which only (prod a_t, h_end) per
 * channel is kept; the second runs chunks 1 .. n-1, each from the state it
 * chains out of the summaries before it (h_in[k+1] = P[k] h_in[k] + H[k]: the
 * scan operator of recurrentgemma/jax/scan.py:161-187, the algebra of
 * multi_shard_correction, jax/pallas.py:73-195, across workgroups instead of
 * devices), and writes y.  `workspace` (16-byte aligned) must hold
 * rg_recurrent_prefill_split_workspace_bytes(B, T, W, H) bytes; that is 0 for
 * shapes that are not cut, where the call is rg_recurrent_prefill itself.
 * Results equal rg_recurrent_prefill's up to the float32 association of the
 * recurrence across chunk boundaries. */
size_t rg_recurrent_prefill_split_workspace_bytes(int B, int T, int W, int H);
int rg_recurrent_prefill_split(const void* x, const void* segpos,
                               int segpos_is_i64, const void* conv_w,
                               const void* conv_b, const void* w_x,
                               const void* b_x, const void* w_a,
                               const void* b_a, const void* w_packed,
                               const void* a_param, const void* h0, void* y,
                               void* h_last, void* conv_cache_out,
                               void* workspace, size_t workspace_bytes, int B,
                               int T, int W, int H, int dtype, void* stream);

/* The recurrent block between its linear layers in one kernel
 * (RecurrentBlock.forward, recurrentgemma/torch/modules.py:627-644):
 *   out = rglru(conv1d(x)) * gelu_tanh(gate_branch)
 * x is the output of linear_x, gate_branch the output of linear_y before its
 * activation, both [B,T,W]; out feeds linear_out.  rg_recurrent_prefill_split
 * (whole rows or rows in chunks: same workspace rule, workspace may be null
 * when rg_recurrent_prefill_split_workspace_bytes is 0) with the join of the
 * two branches applied where y is stored: same values, bit for bit, as that
 * call followed by rg_gelu_mul(y, gate_branch) (gelu rounded to `dtype` like
 * the tensor it is in the reference, then the product rounded), without the
 * pass over y in between.  out may alias gate_branch (every element is read
 * before it is written, by the same lane); neither may alias x.  h_last and
 * conv_cache_out as in rg_recurrent_prefill.  RG_ERR_UNSUPPORTED for the
 * shapes rg_recurrent_prefill refuses: callers then use the separate calls. */
int rg_recurrent_prefill_gelu_mul(
    const void* x, const void* gate_branch, const void* segpos,
    int segpos_is_i64, const void* conv_w, const void* conv_b, const void* w_x,
    const void* b_x, const void* w_a, const void* b_a, const void* w_packed,
    const void* a_param, const void* h0, void* out, void* h_last,
    void* conv_cache_out, void* workspace, size_t workspace_bytes, int B, int T,
    int W, int H, int dtype, void* stream);

/* conv_1d -> rg_lru of a prefill as RecurrentBlock.forward chains them
 * (recurrentgemma/torch/modules.py:632-643), for every shape and both dtypes,
 * with the choice of kernels made here: the single prefill kernel
 * (rg_recurrent_prefill_split; bf16, 256-wide heads, enough (row, head) pairs
 * or rows long enough to be cut into chunks, but not more than 256 pairs of
 * fewer than 64 tokens); for float32 with 256-wide heads and at most 32
 * (row, head) pairs one launch that does the same in float32 (needs no
 * workspace; no entry point of its own); else rg_gates_gemm with the conv
 * applied on load followed by rg_lru_scan_fused_split, the pre-activations of
 * both gates living in the workspace.  gate_branch (nullable, [B,T,W]): the
 * block's linear_y output; `out` is then rglru(conv1d(x)) * gelu_tanh(
 * gate_branch) (modules.py:627-628, 644: inside the single kernels, bf16 and
 * float32, as in rg_recurrent_prefill_gelu_mul; after the two-kernel form
 * rg_gelu_mul over `out` as a last launch), else the plain RG-LRU output.  `workspace` (16-byte aligned)
 * must hold rg_recurrent_core_workspace_bytes(B, T, W, H, dtype) bytes (0 for
 * whole rows in the single kernel: workspace may then be null).  Same values
 * as the calls it is made of; h0 / h_last / conv_cache_out / w_packed as in
 * rg_recurrent_prefill (w_packed is only read by the single kernel).
 * conv_w == conv_b == NULL (conv_cache_out then NULL too): x is the conv
 * output already, and the call is RGLRU.forward on its own
 * (recurrentgemma/torch/layers.py:313-365); rg_recurrent_prefill and its
 * variants take the same. */
size_t rg_recurrent_core_workspace_bytes(int B, int T, int W, int H, int dtype);
int rg_recurrent_core(const void* x, const void* gate_branch,
                      const void* segpos, int segpos_is_i64,
                      const void* conv_w, const void* conv_b, const void* w_x,
                      const void* b_x, const void* w_a, const void* b_a,
                      const void* w_packed, const void* a_param,
                      const void* h0, void* out, void* h_last,
                      void* conv_cache_out, void* workspace,
                      size_t workspace_bytes, int B, int T, int W, int H,
                      int dtype, void* stream);

/* One decode step of the conv -> RG-LRU core, as RecurrentBlock.forward chains
 * them with a cache (recurrentgemma/torch/modules.py:632-643 with
 * layers.py:469-474 and :170-177): x [B,1,W], segpos [B,1],
 * conv_cache_in/out [B,3,W] (`dtype`), h_in/h_out [B,W] float32 (outputs may
 * alias inputs), y [B,1,W].  `workspace` must hold at least
 * rg_recurrent_step_workspace_bytes(B, W, dtype) bytes of device memory. */
size_t rg_recurrent_step_workspace_bytes(int B, int W, int dtype);
int rg_recurrent_step(const void* x, const void* segpos, int segpos_is_i64,
                      const void* conv_cache_in, void* conv_cache_out,
                      const void* h_in, void* h_out, const void* conv_w,
                      const void* conv_b, const void* w_x, const void* b_x,
                      const void* w_a, const void* b_a, const void* a_param,
                      void* y, void* workspace, size_t workspace_bytes, int B,
                      int W, int H, int dtype, void* stream);

/* rg_recurrent_step without a workspace argument and without any allocation.
 * It has no counterpart in the reference: it is for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The three launches of rg_recurrent_step
 * (conv step, gate projections, scan step) exchange the conv output and the
 * two gate pre-activations through a buffer of RG_STEP_STATIC_SCRATCH_BYTES
 * that is part of the library's code object: every GPU the library runs on
 * holds one copy until the process ends.  Shapes whose
 * rg_recurrent_step_workspace_bytes(B, W, dtype) exceeds that size are
 * rejected with RG_ERR_WORKSPACE.  Every call on a GPU uses that GPU's one
 * buffer: calls that overlap on one GPU (two streams, two threads) race;
 * calls in stream order do not, and nothing is carried from one call to the
 * next.  The buffer's address is looked up on the first call on each device
 * (hipGetSymbolAddress); make that call outside a graph capture.  All other
 * arguments and results are those of rg_recurrent_step. */
#define RG_STEP_STATIC_SCRATCH_BYTES (8u << 20)
int rg_recurrent_step_static(const void* x, const void* segpos,
                             int segpos_is_i64, const void* conv_cache_in,
                             void* conv_cache_out, const void* h_in,
                             void* h_out, const void* conv_w,
                             const void* conv_b, const void* w_x,
                             const void* b_x, const void* w_a, const void* b_a,
                             const void* a_param, void* y, int B, int W, int H,
                             int dtype, void* stream);

/* The join of RecurrentBlock.forward's two branches in one pass:
 * out = a * gelu(g) with the tanh approximation, for recurrentgemma/torch/
 * modules.py:627-628 (`y = gelu(linear_y(x))`, gelu at :289-291) and :644
 * (`x = x * y`): `a` is the RG-LRU output, `g` the linear_y output, n elements
 * each in `dtype`.  bf16: gelu evaluated in float32 and rounded to bf16 (it is
 * a tensor of its own in the reference), then the product rounded once.  out
 * may alias a or g. */
int rg_gelu_mul(const void* a, const void* g, void* out, int64_t n, int dtype,
                void* stream);

/* The backward pass of rg_gelu_mul, for autograd through
 * recurrentgemma/torch/modules.py:627-628 and :644 (the reference leaves it to
 * torch's gelu and multiply nodes), one pass:
 *   d_a = dout * gelu(g),   d_g = dout * a * gelu'(g)
 * with gelu the tanh approximation of modules.py:289-291.  dout, a, g, d_a,
 * d_g: n elements each in `dtype`, 16-byte aligned.  bf16: gelu(g) and
 * dout * a are rounded to bf16 before they are used (the tensors they are in
 * the reference's graph), the derivative is evaluated in float32, each output
 * rounded once.  The outputs alias neither each other nor an input. */
int rg_gelu_mul_backward(const void* dout, const void* a, const void* g,
                         void* d_a, void* d_g, int64_t n, int dtype,
                         void* stream);

/* RMSNorm of the residual stack around the recurrent block, one pass:
 * out[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * (scale + 1) for
 * recurrentgemma/torch/layers.py:65-73 (RMSNorm.forward; eps 1e-6 there).
 * x, out [rows, width], scale [width], all in `dtype`.  bf16 reproduces the
 * reference's chain of bf16 tensors: x^2, their mean (float32 sum), var + eps,
 * the rsqrt, x * rsqrt and scale + 1 are each rounded to bf16.  out may alias
 * x. */
int rg_rms_norm(const void* x, const void* scale, void* out, int64_t rows,
                int width, float eps, int dtype, void* stream);

/* The residual sum of a block and the norm that follows it in one pass
 * (recurrentgemma/torch/modules.py:893-896 `residual = x + raw_x;
 * x = self.channel_pre_norm(residual)`): sum_out = x + addend (rounded to
 * `dtype`), out = rg_rms_norm(sum_out).  sum_out may alias x or addend; out
 * must be a different buffer. */
int rg_add_rms_norm(const void* x, const void* addend, const void* scale,
                    void* sum_out, void* out, int64_t rows, int width,
                    float eps, int dtype, void* stream);

/* ---- the local-attention block around its matrix products ----------------
 * Not part of the recurrent path: the steps of the attention block that the
 * reference spells as dozens of elementwise tensor ops per block and decoded
 * token, one kernel each.  Projections, scores and the weighted sum of the
 * values remain batched GEMMs of the caller. */

/* Rotary embedding on the first half of the head dimension
 * (recurrentgemma/torch/modules.py:52-83 `_apply_rope`): x, out
 * [rows, heads, head_dim] in `dtype`, positions [rows] int32/int64, inv_freq
 * [head_dim / 4] float32 = 1 / max_wavelength^(2 i / (head_dim / 2)).  Element
 * i < head_dim/4 pairs with element i + head_dim/4; sin, cos and every product
 * are rounded to `dtype` like the reference's tensors. */
int rg_rope(const void* x, const void* positions, int positions_is_i64,
            const float* inv_freq, void* out, int64_t rows, int heads,
            int head_dim, int dtype, void* stream);
/* The same for queries and keys in one launch (modules.py:431-432 applies it
 * to both with the same positions): q [rows, q_heads, head_dim],
 * k [rows, k_heads, head_dim]. */
int rg_rope_pair(const void* q, const void* k, const void* positions,
                 int positions_is_i64, const float* inv_freq, void* q_out,
                 void* k_out, int64_t rows, int q_heads, int k_heads,
                 int head_dim, int dtype, void* stream);

/* Prompt-pass attention of LocalAttentionBlock.forward without a cache
 * (recurrentgemma/torch/modules.py:404-476; mask :86-127): for every query t
 * the softmax over the keys first_key[t] .. t of scale * q_t . k_j, times the
 * values -- multi-query (H heads of queries, one head of keys and values),
 * bf16, head_dim 256, one kernel (RG_ERR_UNSUPPORTED otherwise: callers keep
 * their batched products).  q, out [B,T,H,256]; k [B,T,256] (both after the
 * rotary embedding); v_t [B,256,T_pad]: the values transposed, T_pad a
 * multiple of 64, zeros from column T on; first_key [B,T] int32,
 * non-decreasing along T: max(first token of the query's document,
 * t - window), which is the reference's mask for a prompt.  Scores and the
 * softmax are float32, the probabilities enter the second product as bf16
 * like the reference's; out is rounded once. */
int rg_attention_prefill(const void* q, const void* k, const void* v_t,
                         const void* first_key, void* out, int B, int T,
                         int T_pad, int H, int head_dim, float scale, int dtype,
                         void* stream);

/* Masked softmax of one decoded token against the ring cache and itself
 * (modules.py:152-183 `_compute_cache_mask`, :462-470): scores
 * [B, heads, window] = q . k of the ring slots, unscaled, in `dtype`; q
 * [B, heads, head_dim] and k_new [B, head_dim] after rg_rope; num_tokens [B]
 * int32, tokens seen before this one; probs [B, heads, window + 1], last
 * column = the new token.  Scores are scaled and rounded to `dtype`, the
 * softmax is taken in float32 over the ring slots that were ever written and
 * the new token, probabilities are rounded to `dtype`. */
int rg_attention_decode_probs(const void* scores, const void* q,
                              const void* k_new, const int32_t* num_tokens,
                              void* probs, int B, int heads, int head_dim,
                              int window, float scale, int dtype,
                              void* stream);

/* out = from_ring + probs[..., window] * v_new (modules.py:471-474), then, if
 * update_cache, the ring update of modules.py:186-216 (`n_fill == 1`): k_new,
 * v_new into slot num_tokens % window of ring_keys / ring_values
 * [B, window, head_dim], num_tokens += 1.  from_ring, out [B, heads, head_dim]
 * (out may alias from_ring). */
int rg_attention_decode_finish(const void* from_ring, const void* probs,
                               const void* k_new, const void* v_new, void* out,
                               void* ring_keys, void* ring_values,
                               int32_t* num_tokens, int B, int heads,
                               int head_dim, int window, int update_cache,
                               int dtype, void* stream);

/* One decoded token per row of the local-attention block against its ring
 * cache, from the projections to the block's output before proj_final
 * (recurrentgemma/torch/modules.py:431-476; cache :152-216): rotary embedding
 * of the queries and the new key (:52-83), scores against the ring, mask (slot
 * j is visible iff it was ever written), softmax with the new token's own
 * score, weighted sum of the values, the new token's share; with update_cache
 * the rotated key and the value go into slot num_tokens % window and
 * num_tokens is incremented, in place.  Two launches that read the ring once
 * (rg_rope + two batched products + rg_attention_decode_probs + _finish
 * otherwise).  bf16, head_dim 256, heads <= 16, window <= 16384.
 * q [B, heads*256] rows ldq elements apart, k_new / v_new [B, 256] rows ldk /
 * ldv apart, all three as the projections left them (slices of one wider
 * output qualify: strides are multiples of 8); positions [B] int32/int64;
 * inv_freq [64] float32; ring_* [B, window, 256]; out [B, heads, 256];
 * workspace: rg_attention_decode_fused_workspace_bytes(B, heads, window) bytes
 * (0: unsupported shape).  Roundings as the separate calls, except that the
 * probabilities enter the second product unnormalised (streaming softmax). */
size_t rg_attention_decode_fused_workspace_bytes(int B, int heads, int window);
int rg_attention_decode_fused(const void* q, int64_t ldq, const void* k_new,
                              int64_t ldk, const void* v_new, int64_t ldv,
                              const void* positions, int positions_are_i64,
                              const float* inv_freq, void* ring_keys,
                              void* ring_values, int32_t* num_tokens, void* out,
                              void* workspace, size_t workspace_bytes, int B,
                              int heads, int head_dim, int window, float scale,
                              int update_cache, int dtype, void* stream);

/* The same decode step in ONE launch, for bf16 with 256-wide heads (no
 * counterpart call in the reference: it is RecurrentBlock.forward with a
 * cache, modules.py:632-643, after a one-time re-layout of the two gate
 * matrices).  rg_pack_gate_weights writes w_x and w_a ([H,256,256] each, the
 * reference's BlockDiagonalLinear layout, layers.py:105-112) into `packed`
 * (rg_packed_gate_weights_bytes(W, H, dtype) bytes, 16-byte aligned) in the
 * order the MFMA operand registers are filled: head, group of 32 output
 * channels, 16-row k-step, gate, lane, 8 values.  Pack again whenever the
 * weights change.  rg_recurrent_step_packed then takes `packed` in place of
 * w_x / w_a and needs no workspace; all other arguments are as for
 * rg_recurrent_step (outputs may alias inputs).  Both return
 * RG_ERR_UNSUPPORTED for other dtypes or head widths (the byte count is 0
 * then): use rg_recurrent_step. */
size_t rg_packed_gate_weights_bytes(int W, int H, int dtype);
int rg_pack_gate_weights(const void* w_x, const void* w_a, void* packed, int W,
                         int H, int dtype, void* stream);
int rg_recurrent_step_packed(const void* x, const void* segpos,
                             int segpos_is_i64, const void* conv_cache_in,
                             void* conv_cache_out, const void* h_in,
                             void* h_out, const void* conv_w,
                             const void* conv_b, const void* w_packed,
                             const void* b_x, const void* b_a,
                             const void* a_param, void* y, int B, int W, int H,
                             int dtype, void* stream);

/* rg_recurrent_step_packed with the recurrent block's join applied where y is
 * stored (RecurrentBlock.forward, recurrentgemma/torch/modules.py:627-628,
 * 644, on a decode step): out = y * gelu_tanh(gate_branch), gate_branch
 * [B,1,W] being the block's linear_y output before its activation.  Same
 * values, bit for bit, as rg_recurrent_step_packed followed by
 * rg_gelu_mul(y, gate_branch); out may alias gate_branch, not x.  bf16 with
 * 256-wide heads only (RG_ERR_UNSUPPORTED otherwise: use the separate calls). */
int rg_recurrent_step_gelu_mul(const void* x, const void* gate_branch,
                               const void* segpos, int segpos_is_i64,
                               const void* conv_cache_in, void* conv_cache_out,
                               const void* h_in, void* h_out,
                               const void* conv_w, const void* conv_b,
                               const void* w_packed, const void* b_x,
                               const void* b_a, const void* a_param, void* out,
                               int B, int W, int H, int dtype, void* stream);

/* The two steps between the last linear layer and the next token id:
 * rg_soft_cap: out = tanh(x / cap) * cap over n elements (griffin.py:203-206),
 *   one pass with the roundings of torch's three (quotient as x * (1 / cap),
 *   tanh, product); out may alias x.
 * rg_argmax_rows: out[r] = index of the largest of x[r, 0..n), the first among
 *   equals, NaN above everything (torch.argmax, greedy sampling,
 *   sampler.py:126-128); x [rows, n] contiguous, out int64. */
int rg_soft_cap(const void* x, void* out, int64_t n, float cap, int dtype,
                void* stream);
int rg_argmax_rows(const void* x, int64_t* out, int rows, int n, int dtype,
                   void* stream);

/* Measurement aid, no counterpart in the reference: one wave per compute unit
 * runs `iters` (1 .. 2^20) rounds of 64 dependent multiply-adds (about 260
 * cycles a round) and leaves in out[0] the shader-clock cycles and in out[1]
 * the ticks of the constant 100 MHz counter that took; out[0] / out[1] / 10 is
 * the shader clock in GHz at that moment.  out: 3 x uint64 of device memory
 * (out[2] is scratch).  bench.py reports it next to its timings, which scale
 * with that clock. */
int rg_clock_probe(uint64_t* out, int iters, void* stream);
/* The same for the clock UNDER the load of the single prefill kernel (its
 * matrix instructions pull the clock below what a light probe reads): while
 * `out` (2 x uint64 of device memory) is set, every rg_recurrent_prefill*
 * / rg_recurrent_core launch that takes that kernel has its workgroup (0, 0)
 * leave in out[0] the shader-clock cycles and in out[1] the 100 MHz ticks of
 * its tile loop.  Process-wide; pass NULL to switch it off again (the state
 * it starts in).  Measurement aid, no counterpart in the reference. */
int rg_prefill_clock_probe(uint64_t* out);

/* The linear layers around the recurrent and attention blocks for a decode
 * step (at most 64 rows), bf16: torch.nn.Linear (modules.py:579-601 linear_y /
 * linear_x / linear_out, :717-721 ffw_down, :334-352 the attention projections)
 * and the stacked Einsum of the MLP (layers.py:76-101, modules.py:711-716).
 * With so few rows a layer is one pass over its weight matrix, so the weights
 * are repacked once, into the order the MFMA operand registers are filled
 * (1 KB blocks per 32 weight rows x 16 inputs), and streamed from there.
 *
 * rg_linear_pack: w holds N weight rows of K inputs, `layout` 0 = [N, K]
 *   (nn.Linear.weight), 1 = [groups, K, N / groups] (Einsum "cdD": weight row
 *   g N/groups + j is w[g, :, j]).  gelu_pair != 0 interleaves tiles of the
 *   first and the second half of the rows for the fused MLP epilogue below.
 *   `packed`: rg_linear_packed_bytes(N, K) bytes (0 = shape unsupported:
 *   needs K % 64 == 0 and N % 32 == 0; gelu_pair N % 64 == 0).  Pack again
 *   whenever the weights change.
 * rg_linear_rows: x [M, K], M <= 64; bias [N] or null;
 *   out [groups, M, N / groups]  = x @ w^T + bias, rounded once; with
 *       `residual` (same layout as out, may alias out): that plus residual,
 *       rounded again (the separate add of modules.py:893-898);
 *   gelu_pair: out [M, N / 2] = gelu(gate) * up with gate / up = rows j and
 *       N/2 + j of x @ w^T + bias, each rounded (modules.py:752-757); groups
 *       must be 1 and residual null.
 *   workspace: rg_linear_rows_workspace_bytes(M, K, N) bytes (may be 0), for
 *   the partial sums of shapes whose K is split over the grid; the sums are
 *   added in a fixed order, results do not vary from run to run.
 *   out must not alias x.
 * rg_linear_rows_partial / rg_add_rms_norm_partial: a layer whose result goes
 *   straight into a residual sum and an RMSNorm (linear_out and proj_final into
 *   channel_pre_norm, modules.py:893-896; ffw_down into the next block's
 *   temporal_pre_norm, modules.py:886-898) without being written in between.
 *   The first writes only the fp32 partial sums `partial` [slices, M, N] of
 *   x @ w^T with K split in `slices` (1..8) over the grid -- three times the
 *   workgroups for the 2560-row layers, which alone fill a third of the CUs.
 *   The second reads them instead of x: v = round(sum over slices, in slice
 *   order, + bias); with addend, v = round(v + addend); sum_out = v,
 *   out = rg_rms_norm(v).  bf16, width % 8 == 0, width <= 4096.  The same
 *   values as those steps taken one by one (rg_linear_rows itself may split K
 *   differently and then differs in the last bit of the fp32 sum). */
size_t rg_linear_packed_bytes(int N, int K, int gelu_pair);
int rg_linear_pack(const void* w, int layout, int groups, int gelu_pair,
                   void* packed, int N, int K, void* stream);
size_t rg_linear_rows_workspace_bytes(int M, int K, int N);
int rg_linear_rows(const void* x, const void* w_packed, const void* bias,
                   const void* residual, void* out, void* workspace,
                   size_t workspace_bytes, int M, int K, int N, int groups,
                   int gelu_pair, void* stream);
int rg_linear_rows_partial(const void* x, const void* w_packed, void* partial,
                           int M, int K, int N, int slices, void* stream);
int rg_add_rms_norm_partial(const void* partial, int slices, const void* bias,
                            const void* addend, const void* scale,
                            void* sum_out, void* out, int rows, int width,
                            float eps, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RG_LRU_H_ */
