// Launcher declarations shared by the kernel files and the C-ABI file.
#ifndef RG_INTERNAL_H_
#define RG_INTERNAL_H_

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>

namespace rg {

// Raises a kernel's dynamic LDS limit the first time it is launched on a
// device; later launches on that device only read the flag (the attribute is a
// property of the loaded function, it does not have to be set per launch).
struct OncePerDevice {
  std::atomic<uint64_t> done{0};  // bit d: set on device d (d < 64)
};
inline hipError_t set_max_dynamic_lds(OncePerDevice& once, const void* fn,
                                      size_t bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (dev < 64 && (once.done.load(std::memory_order_acquire) & bit))
    return hipSuccess;
  e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)bytes);
  if (e == hipSuccess && dev < 64)
    once.done.fetch_or(bit, std::memory_order_release);
  return e;
}

struct ConvArgs {
  const void* x;
  const void* segpos;
  int seg_kind;  // 0: int32 positions, 1: int64 positions, 2: byte mask
  const void* w;
  const void* bias;
  void* out;
  void* cache_out;
  int B, T, W, K;
};

struct ConvStepArgs {
  const void* x;
  const void* cache_in;
  const void* w;
  const void* bias;
  void* out;
  void* cache_out;
  int B, W, K;
};

struct GemmArgs {
  const void* x;       // [M, W]
  int apply_conv;      // width-4 conv on load
  const void* segpos;  // [M] (only with apply_conv)
  int seg_kind;
  const void* conv_w;  // [4, W]
  const void* conv_b;  // [W]
  const void* w[2];    // [H, bw, bw] per gate
  const void* b[2];    // [H, bw] per gate
  void* out[2];        // [M, W] per gate
  int ngates;          // 1 or 2
  int64_t M;           // rows = B*T
  int T;               // sequence length (row m is token m % T of its row)
  int W, H, bw;
};

struct ScanArgs {
  int plain;  // 1: rnn_scan only (x is the recurrence input, ga holds a)
  const void* x;
  int apply_conv;
  const void* conv_w;
  const void* conv_b;
  const void* gx;
  const void* ga;
  const void* a_param;
  const void* segpos;
  int seg_kind;
  const float* h0;
  void* y;
  float* h_last;
  void* cache_out;
  int B, T, W;
  // sequences cut into `chunks` chunks of t_chunk tokens (chunks <= 1: not
  // cut), with three [B][chunks][W] float rows of workspace: every chunk's
  // product of a_t, its state from a zero start, its incoming state
  int chunks, t_chunk;
  float* ws_p;
  float* ws_h;
};

struct FusedArgs {
  const void* x;       // [B, T, W] bf16, the conv input
  const void* segpos;  // [B, T]
  int seg_kind;
  const void* conv_w;  // [4, W]
  const void* conv_b;  // [W]
  const void* w[2];    // [H, 256, 256]: input gate, a gate
  const void* w_packed;  // or null: both, see launch_pack_gate_weights
  const void* b[2];    // [H, 256]
  const void* a_param; // [W]
  const float* h0;     // [B, W] or null
  void* y;             // [B, T, W]
  // or null: [B, T, W] bf16, the other branch of the recurrent block before
  // its activation; y is then the block's join y * gelu(gate_branch)
  const void* gate_branch;
  float* h_last;       // [B, W] or null
  void* cache_out;     // [B, 3, W] or null
  int B, T, W, H;
  // sequences cut into `chunks` chunks of tiles_per_chunk 64-token tiles
  // (chunks <= 1: not cut), with two [B][chunks][W] float rows of workspace:
  // every chunk's product of a_t and its state from a zero start
  int chunks, tiles_per_chunk;
  float* ws_p;
  float* ws_h;
  // or null: workgroup (0, 0) leaves here the shader-clock cycles and the
  // 100 MHz ticks its tile loop took (rg_prefill_clock_probe)
  uint64_t* timing;
};

struct StepArgs {
  const void* x;         // [B, 1, W] bf16
  const void* segpos;    // [B, 1]
  int seg_kind;
  const void* cache_in;  // [B, 3, W] bf16
  void* cache_out;       // [B, 3, W] bf16 (may alias cache_in)
  const float* h_in;     // [B, W]
  float* h_out;          // [B, W] (may alias h_in)
  const void* conv_w;
  const void* conv_b;
  const void* w_packed;  // both gate matrices, see launch_pack_gate_weights
  const void* b[2];
  const void* a_param;
  void* y;               // [B, 1, W]
  // the block's other branch [B, 1, W] or null: y is written as
  // y * gelu(gate_branch)
  const void* gate_branch;
  int B, W, H;
};

// Prompt-pass attention (rg_attention_prefill.hip).
struct AttnPrefillArgs {
  const void* q;    // [B, T, H, 256] bf16, after the rotary embedding
  const void* k;    // [B, T, 256] bf16, after the rotary embedding
  const void* v_t;  // [B, 256, T_pad] bf16: the values transposed, zeros
                    // behind token T - 1 (T_pad a multiple of 64)
  const void* lo;   // [B, T] int32: first key each query sees (non-decreasing)
  void* out;        // [B, T, H, 256] bf16
  int B, T, T_pad, H;
  float scale;      // of the scores (head_dim ** -0.5)
};
hipError_t launch_attn_prefill_bf16(const AttnPrefillArgs& a, hipStream_t s);

// One decoded token against the ring cache (rg_attention_decode.hip).
constexpr int kAttnDecodeChunk = 256;     // ring slots per workgroup
constexpr int kAttnDecodeMaxChunks = 64;  // window <= 16384
struct AttnDecodeArgs {
  const uint16_t* q;      // [B, heads, 256] rows ldq apart, before the rotary
  const uint16_t* k_new;  // [B, 256] rows ldk apart, before the rotary
  const uint16_t* v_new;  // [B, 256] rows ldv apart
  int64_t ldq, ldk, ldv;  // in elements
  const void* pos;        // [B] positions of the new tokens
  int pos_kind;           // 0: int32, 1: int64
  const float* inv_freq;  // [64]
  uint16_t* ring_k;       // [B, window, 256]
  uint16_t* ring_v;
  int32_t* num_tokens;    // [B] tokens seen before this one
  uint16_t* out;          // [B, heads, 256]
  float* part_o;          // [B, chunks, heads, 256]
  float* part_ml;         // [B, chunks, heads, 2]: maximum, denominator
  int B, heads, window, chunks;
  float scale;
  int update;             // write the ring slot and count the token
};
hipError_t launch_attn_decode_fused(const AttnDecodeArgs& a, hipStream_t s);

struct LinearArgs {
  const void* x;         // [M, K] bf16
  const void* w_packed;  // see launch_linear_pack
  const void* bias;      // [N] or null
  const void* residual;  // laid out like out, or null
  void* out;             // [G, M, N / G]; gelu pairs: [M, N / 2]
  float* partial;        // [slices, M, N] when K is split over the grid
  int M, K, N;
  int group_width;       // N / G
};

// Each returns hipSuccess or the launch error.  dtype: 0 = f32, 1 = bf16.
hipError_t launch_conv1d_prefill(const ConvArgs& a, int dtype, hipStream_t s);
hipError_t launch_conv1d_step(const ConvStepArgs& a, int dtype, hipStream_t s);
struct ConvBwdArgs {
  const void* dout;  // [B, T, W] gradient of the conv output
  const void* x;     // [B, T, W] the conv input
  const void* segpos;
  int seg_kind;
  const void* w;     // [K, W]
  void* dx;          // [B, T, W]
  float* partial;    // [conv1d_backward_chunks(B, T)][K + 1][W]
  int B, T, W, K;
};
int conv1d_backward_chunks(int B, int T);
hipError_t launch_conv1d_backward(const ConvBwdArgs& a, int dtype,
                                  hipStream_t s);
hipError_t launch_gemm_generic(const GemmArgs& a, int dtype, hipStream_t s);
hipError_t launch_gemm_mfma_bf16(const GemmArgs& a, hipStream_t s);
hipError_t launch_gemm_mfma_f32(const GemmArgs& a, hipStream_t s);
hipError_t launch_lru_scan(const ScanArgs& a, int dtype, hipStream_t s);

// Backward pass of rnn_scan (rg_scan_bwd.hip).
struct ScanBwdArgs {
  const void* dy;        // [B, T, W] gradient of y
  const void* a;         // [B, T, W] the forward coefficients
  const void* reset;     // [B, T] bytes
  const void* y;         // [B, T, W] the forward outputs
  const float* h0;       // [B, W] or null
  const float* dh_last;  // [B, W] or null: gradient of the final state
  void* dx;              // [B, T, W]
  void* da;              // [B, T, W]
  float* dh0;            // [B, W] or null
  int B, T, W;
};
hipError_t launch_linear_scan_backward(const ScanBwdArgs& a, int dtype,
                                       hipStream_t s);
struct RglruBwdArgs {
  const void* dy;        // [B, T, W] gradient of y
  const void* x;         // [B, T, W] the RG-LRU's input (the conv output)
  const void* gx;        // [B, T, W] input gate pre-activations
  const void* ga;        // [B, T, W] recurrence gate pre-activations
  const void* a_param;   // [W]
  const void* reset;     // [B, T] bytes
  const void* y;         // [B, T, W] the forward outputs
  const float* h0;       // [B, W] or null
  const float* dh_last;  // [B, W] or null: gradient of the final state
  void* dx;              // [B, T, W]
  void* dgx;             // [B, T, W]
  void* dga;             // [B, T, W]
  float* dlam;           // [B, W]: each row's share of a_param's gradient
  float* dh0;            // [B, W] or null
  int B, T, W;
};
hipError_t launch_rglru_backward(const RglruBwdArgs& a, int dtype,
                                 hipStream_t s);
void scan_split_plan(int B, int T, int W, int granule, int* chunks,
                     int* t_chunk);
// Chunk lengths are multiples of this for the kernel that handles (dtype, W).
int scan_split_granule(int dtype, int W);
hipError_t launch_block_prefill_bf16(const FusedArgs& a, hipStream_t s);
hipError_t launch_block_prefill_teams_bf16(const FusedArgs& a, hipStream_t s);
// float32, 256-wide heads, few rows: conv, gate projections, gates and
// recurrence in one launch (rg_core_f32.hip)
bool core_f32_small_serves(int B, int T, int W, int H);
hipError_t launch_core_f32_small(const FusedArgs& a, hipStream_t s);
void prefill_chunk_plan(int B, int H, int T, int* chunks, int* tiles_per_chunk);
hipError_t launch_block_step_bf16(const StepArgs& a, hipStream_t s);
// bf16 [H,256,256] x 2 -> one buffer of the same total size in MFMA operand
// order (head, wave, k-step, gate, lane, 8 values).
// out[i] = a[i] * gelu_tanh(g[i]) over n elements (out may alias a or g).
hipError_t launch_gelu_mul(const void* a, const void* g, void* out, int64_t n,
                           int dtype, hipStream_t s);
hipError_t launch_gelu_mul_backward(const void* dout, const void* a,
                                    const void* g, void* d_a, void* d_g,
                                    int64_t n, int dtype, hipStream_t s);
// out = tanh(x / cap) * cap, n elements; out[r] = argmax(x[r, :n])
hipError_t launch_soft_cap(const void* x, void* out, int64_t n, float cap,
                           int dtype, hipStream_t s);
hipError_t launch_argmax_rows(const void* x, int64_t* out, int rows, int n,
                              int dtype, hipStream_t s);
// out[r, :] = v * rsqrt(mean(v^2) + eps) * (scale + 1) with v = x[r, :], or,
// with an addend, v = x[r, :] + addend[r, :] (also written to sum_out)
hipError_t launch_rms_norm(const void* x, const void* addend, const void* scale,
                           void* sum_out, void* out, int64_t rows, int width,
                           float eps, int dtype, hipStream_t s);
// Steps of the local-attention block around its matrix products
// (rg_attention.hip).
hipError_t launch_rope(const void* x, const void* pos, int pos_kind,
                       const float* inv_freq, void* out, int64_t rows, int n,
                       int hd, const void* x2, void* out2, int n2, int dtype,
                       hipStream_t s);
hipError_t launch_attn_decode_probs(const void* scores, const void* q,
                                    const void* k_new,
                                    const int32_t* num_tokens, void* probs,
                                    int B, int heads, int hd, int window,
                                    float scale, int dtype, hipStream_t s);
hipError_t launch_attn_decode_finish(const void* from_ring, const void* probs,
                                     const void* k_new, const void* v_new,
                                     void* out, void* ring_k, void* ring_v,
                                     int32_t* num_tokens, int B, int heads,
                                     int hd, int window, int update, int dtype,
                                     hipStream_t s);
// Linear layers for at most 64 rows (rg_linear.hip).
int linear_rows_k_slices(int K, int N);
hipError_t launch_linear_pack(const void* w, void* packed, int N, int K,
                              int layout, int groups, int pair, hipStream_t s);
hipError_t launch_linear_rows(const LinearArgs& a, int gelu_pair,
                              hipStream_t s);
// Only the fp32 partial sums a.partial[slices][M][N] of x @ W^T, K split in
// `slices`; rg_elementwise.hip's norm kernel takes them from there.
hipError_t launch_linear_rows_partial(const LinearArgs& a, int slices,
                                      hipStream_t s);
hipError_t launch_rms_norm_partial(const float* sums, int slices,
                                   const void* bias, const void* addend,
                                   const void* scale, void* sum_out, void* out,
                                   int rows, int width, float eps,
                                   hipStream_t s);
// out[0] = shader cycles, out[1] = 10 ns ticks that `iters` rounds of a short
// dependent instruction chain took (rg_elementwise.hip)
hipError_t launch_clock_probe(uint64_t* out, int iters, hipStream_t s);
// rg_gates_wgrad.hip: weight and bias gradients of both gate projections
bool gates_wgrad_serves(int64_t M, int W, int H);
size_t gates_wgrad_workspace_bytes(int64_t M, int W, int H);
hipError_t launch_gates_wgrad(const void* x, const void* dgx, const void* dga,
                              void* dwx, void* dwa, void* dbx, void* dba,
                              void* workspace, int64_t M, int W, int H,
                              hipStream_t s);
hipError_t launch_pack_gate_weights(const void* w_x, const void* w_a,
                                    void* packed, int H, hipStream_t s);

}  // namespace rg
#endif  // RG_INTERNAL_H_
