// extern "C" boundary of librg_lru.so: argument checks, dispatch, errors.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "../../include/rg_lru.h"
#include "rg_internal.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int launch_status(const char* what, hipError_t e) {
  if (e == hipSuccess) return RG_OK;
  return fail(RG_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

// Scratch of rg_recurrent_step_static: lives in the code object, one copy per
// GPU the library is loaded on, for as long as the process runs.  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels and
// copies get the per-device address kept in g_step_scratch.
static __device__ __align__(256) unsigned char scratch[RG_STEP_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
void* g_step_scratch[kMaxDevices];  // device id -> address of its `scratch`
std::mutex g_step_scratch_mutex;

// The calling thread's current device's copy of `scratch` (looked up once per
// device), or null with *err set.
void* step_scratch(hipError_t* err) {
  int dev = 0;
  *err = hipGetDevice(&dev);
  if (*err != hipSuccess) return nullptr;
  if (dev < 0 || dev >= kMaxDevices) {
    *err = hipErrorInvalidDevice;
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_step_scratch_mutex);
  if (g_step_scratch[dev] == nullptr) {
    void* ptr = nullptr;
    *err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (*err != hipSuccess) return nullptr;
    g_step_scratch[dev] = ptr;
  }
  return g_step_scratch[dev];
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t esize(int dtype) { return dtype == RG_DTYPE_F32 ? 4 : 2; }

// The entry point named in error messages: the function itself, or, in a body
// shared by two entry points, the one that was called.
#define RG_WHO __func__

#define RG_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) return fail(RG_ERR_BAD_ARG, __VA_ARGS__); \
  } while (0)

#define RG_CHECK_DTYPE(dtype)                                            \
  do {                                                                   \
    if ((dtype) != RG_DTYPE_F32 && (dtype) != RG_DTYPE_BF16)             \
      return fail(RG_ERR_UNSUPPORTED, "%s: dtype %d is not f32/bf16",    \
                  RG_WHO, (dtype));                                    \
  } while (0)

#define RG_CHECK_PTR(p)                                                     \
  do {                                                                      \
    RG_REQUIRE((p) != nullptr, "%s: %s is null", RG_WHO, #p);             \
    RG_REQUIRE(aligned16(p), "%s: %s is not 16-byte aligned", RG_WHO, #p); \
  } while (0)

#define RG_CHECK_OPT_PTR(p) \
  RG_REQUIRE(aligned16(p), "%s: %s is not 16-byte aligned", RG_WHO, #p)

}  // namespace

// rg_prefill_clock_probe: where the single prefill kernel leaves its cycle and
// tick counts (null: nowhere)
static std::atomic<uint64_t*> g_prefill_timing{nullptr};

extern "C" {

int rg_abi_version(void) { return RG_ABI_VERSION; }

const char* rg_last_error(void) { return g_err; }

int rg_conv1d_prefill(const void* x, const void* segpos, int segpos_is_i64,
                      const void* w, const void* bias, void* out,
                      void* cache_out, int B, int T, int W, int K, int dtype,
                      void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0, "%s: B=%d T=%d W=%d must be positive",
             __func__, B, T, W);
  if (K < 2 || K > RG_MAX_CONV_WIDTH)
    return fail(RG_ERR_UNSUPPORTED, "%s: temporal width %d outside [2,%d]",
                __func__, K, RG_MAX_CONV_WIDTH);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(segpos);
  RG_CHECK_PTR(w);
  RG_CHECK_PTR(bias);
  RG_CHECK_PTR(out);
  RG_CHECK_OPT_PTR(cache_out);
  RG_REQUIRE(out != x, "%s: out must not alias x", __func__);
  rg::ConvArgs a{x, segpos, segpos_is_i64 ? 1 : 0, w, bias, out, cache_out,
                 B, T, W, K};
  return launch_status(__func__,
                       rg::launch_conv1d_prefill(a, dtype, (hipStream_t)stream));
}

size_t rg_conv1d_backward_workspace_bytes(int B, int T, int W, int K) {
  if (B <= 0 || T <= 0 || W <= 0 || K < 2 || K > RG_MAX_CONV_WIDTH) return 0;
  return (size_t)rg::conv1d_backward_chunks(B, T) * (K + 1) * W * sizeof(float);
}

int rg_conv1d_backward(const void* dout, const void* x, const void* segpos,
                       int segpos_is_i64, const void* w, void* dx,
                       void* partial, size_t partial_bytes, int B, int T, int W,
                       int temporal_width, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0, "%s: B=%d T=%d W=%d must be positive",
             __func__, B, T, W);
  if (temporal_width < 2 || temporal_width > RG_MAX_CONV_WIDTH)
    return fail(RG_ERR_UNSUPPORTED, "%s: temporal width %d outside [2,%d]",
                __func__, temporal_width, RG_MAX_CONV_WIDTH);
  RG_CHECK_PTR(dout);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(segpos);
  RG_CHECK_PTR(w);
  RG_CHECK_PTR(dx);
  RG_REQUIRE(dx != dout && dx != x, "%s: dx must not alias an input", __func__);
  const size_t need =
      rg_conv1d_backward_workspace_bytes(B, T, W, temporal_width);
  if (partial == nullptr || partial_bytes < need || !aligned16(partial))
    return fail(RG_ERR_WORKSPACE,
                "%s: partial sums need %zu bytes (16-byte aligned), got %zu",
                __func__, need, partial ? partial_bytes : (size_t)0);
  rg::ConvBwdArgs a{};
  a.dout = dout;
  a.x = x;
  a.segpos = segpos;
  a.seg_kind = segpos_is_i64 ? 1 : 0;
  a.w = w;
  a.dx = dx;
  a.partial = (float*)partial;
  a.B = B;
  a.T = T;
  a.W = W;
  a.K = temporal_width;
  return launch_status(
      __func__, rg::launch_conv1d_backward(a, dtype, (hipStream_t)stream));
}

int rg_conv1d_step(const void* x, const void* cache_in, const void* w,
                   const void* bias, void* out, void* cache_out, int B, int W,
                   int K, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && W > 0, "%s: B=%d W=%d must be positive", __func__, B, W);
  if (K < 2 || K > RG_MAX_CONV_WIDTH)
    return fail(RG_ERR_UNSUPPORTED, "%s: temporal width %d outside [2,%d]",
                __func__, K, RG_MAX_CONV_WIDTH);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(cache_in);
  RG_CHECK_PTR(w);
  RG_CHECK_PTR(bias);
  RG_CHECK_PTR(out);
  RG_CHECK_OPT_PTR(cache_out);
  RG_REQUIRE(out != x, "%s: out must not alias x", __func__);
  rg::ConvStepArgs a{x, cache_in, w, bias, out, cache_out, B, W, K};
  return launch_status(__func__,
                       rg::launch_conv1d_step(a, dtype, (hipStream_t)stream));
}

// Heads the bf16 matrix-core kernel serves: its tile is 256 x 256 per head,
// narrower heads are padded with zeros inside the kernel, which still beats
// the generic kernel while at most three quarters of the products are padding
// (measured at 176: 4.35 -> 0.6 ms at B16 T4096 W5632).
static bool mfma_bf16_takes(int bw) {
  return bw >= 128 && bw <= 256 && bw % 8 == 0;
}

int rg_block_diag_linear(const void* x, const void* w, const void* b, void* y,
                         int64_t M, int H, int bw, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(M > 0 && H > 0 && bw > 0, "%s: M=%lld H=%d bw=%d must be positive",
             __func__, (long long)M, H, bw);
  RG_REQUIRE((int64_t)H * bw <= 0x7fffffff, "%s: width overflows", __func__);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(w);
  RG_CHECK_PTR(b);
  RG_CHECK_PTR(y);
  RG_REQUIRE(y != x, "%s: y must not alias x", __func__);
  rg::GemmArgs a{};
  a.x = x;
  a.w[0] = w;
  a.b[0] = b;
  a.out[0] = y;
  a.ngates = 1;
  a.M = M;
  a.T = 1;
  a.W = H * bw;
  a.H = H;
  a.bw = bw;
  if (dtype == RG_DTYPE_F32 && bw == 256)
    return launch_status(__func__,
                         rg::launch_gemm_mfma_f32(a, (hipStream_t)stream));
  // (the bf16 matrix kernel addresses rows of x and y with 32-bit offsets
  // inside one 64-row tile only)
  if (dtype == RG_DTYPE_BF16 && mfma_bf16_takes(bw) && aligned16(x) &&
      aligned16(w) && aligned16(y))
    return launch_status(__func__,
                         rg::launch_gemm_mfma_bf16(a, (hipStream_t)stream));
  return launch_status(__func__,
                       rg::launch_gemm_generic(a, dtype, (hipStream_t)stream));
}

size_t rg_gates_weight_grads_workspace_bytes(int64_t M, int W, int H) {
  return rg::gates_wgrad_workspace_bytes(M, W, H);
}

int rg_gates_weight_grads(const void* x, const void* dgx, const void* dga,
                          void* dwx, void* dwa, void* dbx, void* dba,
                          void* workspace, size_t workspace_bytes, int64_t M,
                          int W, int H, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(M > 0 && W > 0 && H > 0, "%s: M=%lld W=%d H=%d must be positive",
             __func__, (long long)M, W, H);
  if (dtype != RG_DTYPE_BF16 || !rg::gates_wgrad_serves(M, W, H))
    return fail(RG_ERR_UNSUPPORTED,
                "%s: unsupported: bf16 with 256-wide heads only (W=%d H=%d)",
                __func__, W, H);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(dgx);
  RG_CHECK_PTR(dga);
  RG_CHECK_PTR(dwx);
  RG_CHECK_PTR(dwa);
  RG_CHECK_OPT_PTR(dbx);
  RG_CHECK_OPT_PTR(dba);
  RG_REQUIRE((dbx == nullptr) == (dba == nullptr),
             "%s: dbx and dba are given together or not at all", __func__);
  RG_REQUIRE(aligned16(x) && aligned16(dgx) && aligned16(dga),
             "%s: x, dgx and dga must be 16-byte aligned", __func__);
  const size_t need = rg::gates_wgrad_workspace_bytes(M, W, H);
  if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    return fail(RG_ERR_WORKSPACE,
                "%s: workspace of %zu bytes (16-byte aligned) required, got %zu",
                __func__, need, workspace ? workspace_bytes : (size_t)0);
  return launch_status(
      __func__, rg::launch_gates_wgrad(x, dgx, dga, dwx, dwa, dbx, dba,
                                       workspace, M, W, H, (hipStream_t)stream));
}

int rg_gates_gemm(const void* x, int apply_conv, const void* segpos,
                  int segpos_is_i64, const void* conv_w, const void* conv_b,
                  const void* w_x, const void* b_x, const void* w_a,
                  const void* b_a, void* gx_pre, void* ga_pre, int B, int T,
                  int W, int H, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0 && H > 0,
             "%s: B=%d T=%d W=%d H=%d must be positive", __func__, B, T, W, H);
  RG_REQUIRE(W % H == 0, "%s: W=%d is not a multiple of H=%d", __func__, W, H);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(w_x);
  RG_CHECK_PTR(b_x);
  RG_CHECK_PTR(w_a);
  RG_CHECK_PTR(b_a);
  RG_CHECK_PTR(gx_pre);
  RG_CHECK_PTR(ga_pre);
  RG_REQUIRE(gx_pre != x && ga_pre != x && gx_pre != ga_pre,
             "%s: outputs must not alias x or each other", __func__);
  if (apply_conv) {
    RG_CHECK_PTR(segpos);
    RG_CHECK_PTR(conv_w);
    RG_CHECK_PTR(conv_b);
    // the kernels address segpos through a 32-bit buffer descriptor
    RG_REQUIRE((int64_t)B * T * (segpos_is_i64 ? 8 : 4) < ((int64_t)1 << 32),
               "%s: B*T=%lld positions exceed the 4 GiB a segpos descriptor "
               "covers", __func__, (long long)B * T);
  }
  rg::GemmArgs a{};
  a.x = x;
  a.apply_conv = apply_conv != 0;
  a.segpos = segpos;
  a.seg_kind = segpos_is_i64 ? 1 : 0;
  a.conv_w = conv_w;
  a.conv_b = conv_b;
  a.w[0] = w_x;
  a.b[0] = b_x;
  a.w[1] = w_a;
  a.b[1] = b_a;
  a.out[0] = gx_pre;
  a.out[1] = ga_pre;
  a.ngates = 2;
  a.M = (int64_t)B * T;
  a.T = T;
  a.W = W;
  a.H = H;
  a.bw = W / H;
  hipError_t e;
  if (dtype == RG_DTYPE_BF16 && mfma_bf16_takes(a.bw) && aligned16(x) &&
      aligned16(w_x) && aligned16(w_a) && aligned16(gx_pre) &&
      aligned16(ga_pre))
    e = rg::launch_gemm_mfma_bf16(a, (hipStream_t)stream);
  else if (dtype == RG_DTYPE_F32 && a.bw == 256)
    e = rg::launch_gemm_mfma_f32(a, (hipStream_t)stream);
  else
    e = rg::launch_gemm_generic(a, dtype, (hipStream_t)stream);
  return launch_status(__func__, e);
}

size_t rg_scan_split_workspace_bytes(int B, int T, int W) {
  if (B <= 0 || T <= 0 || W <= 0) return 0;
  // (the size does not know the dtype: the finest cut, float32's, is the
  // largest)
  int chunks, t_chunk;
  rg::scan_split_plan(B, T, W, 64, &chunks, &t_chunk);
  return chunks > 1 ? (size_t)2 * B * chunks * W * sizeof(float) : 0;
}

// Points the scan at its workspace if the shape is one that is cut into
// chunks; RG_OK or the error for a workspace that is missing or too small.
static int plan_scan_split(const char* who, rg::ScanArgs* a, int dtype,
                           void* workspace, size_t workspace_bytes) {
  const size_t need = rg_scan_split_workspace_bytes(a->B, a->T, a->W);
  if (need == 0) return RG_OK;
  if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    return fail(RG_ERR_WORKSPACE,
                "%s: workspace of %zu bytes (16-byte aligned) required, got %zu",
                who, need, workspace ? workspace_bytes : (size_t)0);
  rg::scan_split_plan(a->B, a->T, a->W, rg::scan_split_granule(dtype, a->W),
                      &a->chunks, &a->t_chunk);
  const size_t one = (size_t)a->B * a->chunks * a->W;
  a->ws_p = (float*)workspace;
  a->ws_h = a->ws_p + one;
  return RG_OK;
}

#undef RG_WHO
#define RG_WHO who
static int lru_scan_fused_impl(const char* who, const void* x, int apply_conv,
                               const void* conv_w, const void* conv_b,
                               const void* gx_pre, const void* ga_pre,
                               const void* a_param, const void* segpos,
                               int segpos_is_i64, const void* h0, void* y,
                               void* h_last, void* conv_cache_out,
                               void* workspace, size_t workspace_bytes,
                               bool split, int B, int T, int W, int dtype,
                               void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0, "%s: B=%d T=%d W=%d must be positive",
             who, B, T, W);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(gx_pre);
  RG_CHECK_PTR(ga_pre);
  RG_CHECK_PTR(a_param);
  RG_CHECK_PTR(segpos);
  RG_CHECK_PTR(y);
  RG_CHECK_OPT_PTR(h0);
  RG_CHECK_OPT_PTR(h_last);
  RG_CHECK_OPT_PTR(conv_cache_out);
  RG_REQUIRE(y != x && y != gx_pre && y != ga_pre,
             "%s: y must not alias an input", who);
  if (apply_conv) {
    RG_CHECK_PTR(conv_w);
    RG_CHECK_PTR(conv_b);
  } else {
    RG_REQUIRE(conv_cache_out == nullptr,
               "%s: conv_cache_out needs apply_conv", who);
  }
  rg::ScanArgs a{};
  a.x = x;
  a.apply_conv = apply_conv != 0;
  a.conv_w = conv_w;
  a.conv_b = conv_b;
  a.gx = gx_pre;
  a.ga = ga_pre;
  a.a_param = a_param;
  a.segpos = segpos;
  a.seg_kind = segpos_is_i64 ? 1 : 0;
  a.h0 = (const float*)h0;
  a.y = y;
  a.h_last = (float*)h_last;
  a.cache_out = conv_cache_out;
  a.B = B;
  a.T = T;
  a.W = W;
  if (split) {
    const int rc = plan_scan_split(who, &a, dtype, workspace, workspace_bytes);
    if (rc != RG_OK) return rc;
  }
  return launch_status(who, rg::launch_lru_scan(a, dtype, (hipStream_t)stream));
}

#undef RG_WHO
#define RG_WHO __func__

int rg_lru_scan_fused(const void* x, int apply_conv, const void* conv_w,
                      const void* conv_b, const void* gx_pre,
                      const void* ga_pre, const void* a_param,
                      const void* segpos, int segpos_is_i64, const void* h0,
                      void* y, void* h_last, void* conv_cache_out, int B, int T,
                      int W, int dtype, void* stream) {
  return lru_scan_fused_impl(__func__, x, apply_conv, conv_w, conv_b, gx_pre,
                             ga_pre, a_param, segpos, segpos_is_i64, h0, y,
                             h_last, conv_cache_out, nullptr, 0, false, B, T, W,
                             dtype, stream);
}

int rg_lru_scan_fused_split(const void* x, int apply_conv, const void* conv_w,
                            const void* conv_b, const void* gx_pre,
                            const void* ga_pre, const void* a_param,
                            const void* segpos, int segpos_is_i64,
                            const void* h0, void* y, void* h_last,
                            void* conv_cache_out, void* workspace,
                            size_t workspace_bytes, int B, int T, int W,
                            int dtype, void* stream) {
  return lru_scan_fused_impl(__func__, x, apply_conv, conv_w, conv_b, gx_pre,
                             ga_pre, a_param, segpos, segpos_is_i64, h0, y,
                             h_last, conv_cache_out, workspace, workspace_bytes,
                             true, B, T, W, dtype, stream);
}

size_t rg_recurrent_prefill_split_workspace_bytes(int B, int T, int W, int H) {
  if (B <= 0 || T <= 0 || W <= 0 || H <= 0 || W % H != 0 || W / H != 256)
    return 0;
  int chunks, per;
  rg::prefill_chunk_plan(B, H, T, &chunks, &per);
  return chunks > 1 ? (size_t)2 * B * chunks * W * sizeof(float) : 0;
}

#undef RG_WHO
#define RG_WHO who
static int recurrent_prefill_impl(const char* who, const void* x,
                                  const void* segpos, int segpos_is_i64,
                                  const void* conv_w, const void* conv_b,
                                  const void* w_x, const void* b_x,
                                  const void* w_a, const void* b_a,
                                  const void* w_packed, const void* a_param,
                                  const void* h0, const void* gate_branch,
                                  void* y, void* h_last,
                                  void* conv_cache_out, void* workspace,
                                  size_t workspace_bytes, bool split, int B,
                                  int T, int W, int H, int dtype,
                                  void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0 && H > 0,
             "%s: B=%d T=%d W=%d H=%d must be positive", who, B, T, W, H);
  RG_REQUIRE(W % H == 0, "%s: W=%d is not a multiple of H=%d", who, W, H);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(segpos);
  RG_CHECK_OPT_PTR(conv_w);
  RG_CHECK_OPT_PTR(conv_b);
  // no conv weights: x is the conv output already (a stand-alone RG-LRU)
  RG_REQUIRE((conv_w == nullptr) == (conv_b == nullptr),
             "%s: conv_w and conv_b go together", who);
  RG_REQUIRE(conv_w != nullptr || conv_cache_out == nullptr,
             "%s: no conv state without a conv", who);
  RG_CHECK_PTR(w_x);
  RG_CHECK_PTR(b_x);
  RG_CHECK_PTR(w_a);
  RG_CHECK_PTR(b_a);
  RG_CHECK_PTR(a_param);
  RG_CHECK_PTR(y);
  RG_CHECK_OPT_PTR(w_packed);
  RG_CHECK_OPT_PTR(h0);
  RG_CHECK_OPT_PTR(h_last);
  RG_CHECK_OPT_PTR(conv_cache_out);
  RG_CHECK_OPT_PTR(gate_branch);
  RG_REQUIRE(y != x, "%s: y must not alias x", who);
  // The single-launch kernel exists for bf16 with 256-wide heads and
  // sequences whose byte offsets fit 31 bits; everything else is served by
  // rg_gates_gemm + rg_lru_scan_fused.
  if (dtype != RG_DTYPE_BF16 || W / H != 256 ||
      (int64_t)T * W * 2 >= (int64_t)0x7fffffff) {
    return fail(RG_ERR_UNSUPPORTED,
                "%s: unsupported shape or dtype (needs bf16, W/H == 256, "
                "T*W*2 < 2^31): dtype=%d W=%d H=%d T=%d",
                who, dtype, W, H, T);
  }
  rg::FusedArgs a{};
  a.timing = g_prefill_timing.load(std::memory_order_relaxed);
  a.x = x;
  a.segpos = segpos;
  a.seg_kind = segpos_is_i64 ? 1 : 0;
  a.conv_w = conv_w;
  a.conv_b = conv_b;
  a.w[0] = w_x;
  a.b[0] = b_x;
  a.w[1] = w_a;
  a.b[1] = b_a;
  a.w_packed = w_packed;
  a.a_param = a_param;
  a.h0 = (const float*)h0;
  a.y = y;
  a.gate_branch = gate_branch;
  a.h_last = (float*)h_last;
  a.cache_out = conv_cache_out;
  a.B = B;
  a.T = T;
  a.W = W;
  a.H = H;
  a.chunks = 1;
  a.tiles_per_chunk = (T + 63) / 64;
  if (split) {
    const size_t need = rg_recurrent_prefill_split_workspace_bytes(B, T, W, H);
    if (need > 0) {
      if (workspace == nullptr || workspace_bytes < need ||
          !aligned16(workspace))
        return fail(RG_ERR_WORKSPACE,
                    "%s: workspace of %zu bytes (16-byte aligned) required, "
                    "got %zu", who, need, workspace ? workspace_bytes : (size_t)0);
      rg::prefill_chunk_plan(B, H, T, &a.chunks, &a.tiles_per_chunk);
      const size_t one = (size_t)B * a.chunks * W;
      a.ws_p = (float*)workspace;
      a.ws_h = a.ws_p + one;
    }
  }
  return launch_status(who,
                       rg::launch_block_prefill_bf16(a, (hipStream_t)stream));
}
#undef RG_WHO
#define RG_WHO __func__

int rg_recurrent_prefill(const void* x, const void* segpos, int segpos_is_i64,
                         const void* conv_w, const void* conv_b,
                         const void* w_x, const void* b_x, const void* w_a,
                         const void* b_a, const void* w_packed,
                         const void* a_param, const void* h0, void* y,
                         void* h_last, void* conv_cache_out, int B, int T,
                         int W, int H, int dtype, void* stream) {
  return recurrent_prefill_impl(__func__, x, segpos, segpos_is_i64, conv_w,
                                conv_b, w_x, b_x, w_a, b_a, w_packed, a_param,
                                h0, nullptr, y, h_last, conv_cache_out,
                                nullptr, 0, false, B, T, W, H, dtype, stream);
}

int rg_recurrent_prefill_split(const void* x, const void* segpos,
                               int segpos_is_i64, const void* conv_w,
                               const void* conv_b, const void* w_x,
                               const void* b_x, const void* w_a,
                               const void* b_a, const void* w_packed,
                               const void* a_param, const void* h0, void* y,
                               void* h_last, void* conv_cache_out,
                               void* workspace, size_t workspace_bytes, int B,
                               int T, int W, int H, int dtype, void* stream) {
  return recurrent_prefill_impl(__func__, x, segpos, segpos_is_i64, conv_w,
                                conv_b, w_x, b_x, w_a, b_a, w_packed, a_param,
                                h0, nullptr, y, h_last, conv_cache_out,
                                workspace, workspace_bytes, true, B, T, W, H,
                                dtype, stream);
}

int rg_recurrent_prefill_gelu_mul(
    const void* x, const void* gate_branch, const void* segpos,
    int segpos_is_i64, const void* conv_w, const void* conv_b, const void* w_x,
    const void* b_x, const void* w_a, const void* b_a, const void* w_packed,
    const void* a_param, const void* h0, void* out, void* h_last,
    void* conv_cache_out, void* workspace, size_t workspace_bytes, int B, int T,
    int W, int H, int dtype, void* stream) {
  RG_CHECK_PTR(gate_branch);
  RG_REQUIRE(gate_branch != x, "%s: gate_branch must not alias x", __func__);
  return recurrent_prefill_impl(__func__, x, segpos, segpos_is_i64, conv_w,
                                conv_b, w_x, b_x, w_a, b_a, w_packed, a_param,
                                h0, gate_branch, out, h_last, conv_cache_out,
                                workspace, workspace_bytes, true, B, T, W, H,
                                dtype, stream);
}

// Which form serves a shape: the single prefill kernel where its workgroups
// (one per row, head and time chunk) fill the GPU, else the gate GEMM and the
// scan kernel with the pre-activations of both gates in the workspace.
struct CorePlan {
  bool small_f32;      // core_f32_small_kernel: everything in one launch
  bool single;         // block_prefill_bf16_kernel
  size_t split_bytes;  // chunk summaries of whichever form runs
  size_t gate_bytes;   // one gate's pre-activations (two-kernel form), padded
};
static CorePlan core_plan(int B, int T, int W, int H, int dtype) {
  CorePlan p{};
  // float32 with few rows: one launch, no workspace (a short float32 call is
  // three launches' worth of latency otherwise)
  p.small_f32 = dtype == RG_DTYPE_F32 && rg::core_f32_small_serves(B, T, W, H);
  if (p.small_f32) return p;
  const bool fits = dtype == RG_DTYPE_BF16 && W / H == 256 &&
                    (int64_t)T * W * 2 < (int64_t)0x7fffffff;
  const size_t chunk_bytes =
      fits ? rg_recurrent_prefill_split_workspace_bytes(B, T, W, H) : 0;
  // The single kernel serves every such shape (measured against the gate GEMM
  // + scan pair at W2560 H10, 10-640 (row, head) pairs, T32-4096: 10-50 %
  // ahead everywhere, whole rows or chunks) but many very short rows: with
  // more workgroups than CUs each CU loads a head's 256 KB of gate weights
  // again for every pair it runs, and with a few tokens per row that
  // outweighs the rest (us, single / pair: 640 pairs T1 37/28, T16 40/36, T32
  // 42/48; 1280 pairs T16 68/47, T32 70/66, T48 72/85; 2560 pairs T1 122/28,
  // T32 136/112, T48 138/146).
  const int64_t pairs = (int64_t)B * H;
  const bool many_short_rows =
      (pairs > 512 && T <= 16) || (pairs > 1024 && T <= 32);
  p.single = fits && !many_short_rows;
  if (p.single) {
    p.split_bytes = chunk_bytes;
  } else {
    // (rounded up: the gate planes behind it must stay 16-byte aligned)
    p.split_bytes =
        (rg_scan_split_workspace_bytes(B, T, W) + 255) & ~(size_t)255;
    const size_t n = (size_t)B * T * W * (dtype == RG_DTYPE_F32 ? 4 : 2);
    p.gate_bytes = (n + 255) & ~(size_t)255;
  }
  return p;
}

size_t rg_recurrent_core_workspace_bytes(int B, int T, int W, int H,
                                         int dtype) {
  if (B <= 0 || T <= 0 || W <= 0 || H <= 0 || W % H != 0 ||
      (dtype != RG_DTYPE_F32 && dtype != RG_DTYPE_BF16))
    return 0;
  const CorePlan p = core_plan(B, T, W, H, dtype);
  return p.split_bytes + 2 * p.gate_bytes;
}

int rg_recurrent_core(const void* x, const void* gate_branch,
                      const void* segpos, int segpos_is_i64,
                      const void* conv_w, const void* conv_b, const void* w_x,
                      const void* b_x, const void* w_a, const void* b_a,
                      const void* w_packed, const void* a_param,
                      const void* h0, void* out, void* h_last,
                      void* conv_cache_out, void* workspace,
                      size_t workspace_bytes, int B, int T, int W, int H,
                      int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0 && H > 0,
             "%s: B=%d T=%d W=%d H=%d must be positive", __func__, B, T, W, H);
  RG_REQUIRE(W % H == 0, "%s: W=%d is not a multiple of H=%d", __func__, W, H);
  RG_CHECK_OPT_PTR(gate_branch);
  RG_REQUIRE(gate_branch == nullptr || gate_branch != x,
             "%s: gate_branch must not alias x", __func__);
  RG_REQUIRE((conv_w == nullptr) == (conv_b == nullptr),
             "%s: conv_w and conv_b go together", __func__);
  RG_REQUIRE(conv_w != nullptr || conv_cache_out == nullptr,
             "%s: no conv state without a conv", __func__);
  const int conv = conv_w != nullptr;
  const CorePlan p = core_plan(B, T, W, H, dtype);
  const size_t need = p.split_bytes + 2 * p.gate_bytes;
  if (need > 0 && (workspace == nullptr || workspace_bytes < need ||
                   !aligned16(workspace)))
    return fail(RG_ERR_WORKSPACE,
                "%s: workspace of %zu bytes (16-byte aligned) required, got %zu",
                __func__, need, workspace ? workspace_bytes : (size_t)0);
  if (p.small_f32) {
    RG_CHECK_PTR(x);
    RG_CHECK_PTR(segpos);
    RG_CHECK_OPT_PTR(conv_w);
    RG_CHECK_OPT_PTR(conv_b);
    RG_CHECK_PTR(w_x);
    RG_CHECK_PTR(b_x);
    RG_CHECK_PTR(w_a);
    RG_CHECK_PTR(b_a);
    RG_CHECK_PTR(a_param);
    RG_CHECK_PTR(out);
    RG_CHECK_OPT_PTR(h0);
    RG_CHECK_OPT_PTR(h_last);
    RG_CHECK_OPT_PTR(conv_cache_out);
    RG_REQUIRE(out != x, "%s: out must not alias x", __func__);
    rg::FusedArgs a{};
    a.x = x;
    a.segpos = segpos;
    a.seg_kind = segpos_is_i64 ? 1 : 0;
    a.conv_w = conv_w;
    a.conv_b = conv_b;
    a.w[0] = w_x;
    a.b[0] = b_x;
    a.w[1] = w_a;
    a.b[1] = b_a;
    a.a_param = a_param;
    a.h0 = (const float*)h0;
    a.y = out;
    a.h_last = (float*)h_last;
    a.cache_out = conv_cache_out;
    a.gate_branch = gate_branch;  // the join is in the kernel's y stores
    a.B = B;
    a.T = T;
    a.W = W;
    a.H = H;
    return launch_status(
        __func__, rg::launch_core_f32_small(a, (hipStream_t)stream));
  } else if (p.single) {
    // the join is part of the kernel's output stage, for rows in chunks too
    // (the launches that write y apply it)
    return recurrent_prefill_impl(
        __func__, x, segpos, segpos_is_i64, conv_w, conv_b, w_x, b_x, w_a, b_a,
        w_packed, a_param, h0, gate_branch, out, h_last, conv_cache_out,
        workspace, workspace_bytes, true, B, T, W, H, dtype, stream);
  } else {
    char* const ws = (char*)workspace;
    void* const gx = ws + p.split_bytes;
    void* const ga = ws + p.split_bytes + p.gate_bytes;
    int rc = rg_gates_gemm(x, conv, segpos, segpos_is_i64, conv_w, conv_b, w_x,
                           b_x, w_a, b_a, gx, ga, B, T, W, H, dtype, stream);
    if (rc != RG_OK) return rc;
    rc = lru_scan_fused_impl(__func__, x, conv, conv_w, conv_b, gx, ga, a_param,
                             segpos, segpos_is_i64, h0, out, h_last,
                             conv_cache_out, workspace, p.split_bytes, true, B,
                             T, W, dtype, stream);
    if (rc != RG_OK || gate_branch == nullptr) return rc;
  }
  return launch_status(
      __func__, rg::launch_gelu_mul(out, gate_branch, out, (int64_t)B * T * W,
                                    dtype, (hipStream_t)stream));
}

#undef RG_WHO
#define RG_WHO who
static int linear_scan_impl(const char* who, const void* x, const void* a,
                            const void* reset, const void* h0, void* y,
                            void* h_last, void* workspace,
                            size_t workspace_bytes, bool split, int B, int T,
                            int W, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0, "%s: B=%d T=%d W=%d must be positive",
             who, B, T, W);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(a);
  RG_CHECK_PTR(reset);
  RG_CHECK_PTR(y);
  RG_CHECK_OPT_PTR(h0);
  RG_CHECK_OPT_PTR(h_last);
  RG_REQUIRE(y != x && y != a, "%s: y must not alias an input", who);
  rg::ScanArgs s{};
  s.plain = 1;
  s.x = x;
  s.gx = x;  // unused in this mode
  s.ga = a;
  s.segpos = reset;
  s.seg_kind = 2;
  s.h0 = (const float*)h0;
  s.y = y;
  s.h_last = (float*)h_last;
  s.B = B;
  s.T = T;
  s.W = W;
  if (split) {
    const int rc = plan_scan_split(who, &s, dtype, workspace, workspace_bytes);
    if (rc != RG_OK) return rc;
  }
  return launch_status(who, rg::launch_lru_scan(s, dtype, (hipStream_t)stream));
}

#undef RG_WHO
#define RG_WHO __func__

int rg_linear_scan(const void* x, const void* a, const void* reset,
                   const void* h0, void* y, void* h_last, int B, int T, int W,
                   int dtype, void* stream) {
  return linear_scan_impl(__func__, x, a, reset, h0, y, h_last, nullptr, 0,
                          false, B, T, W, dtype, stream);
}

int rg_linear_scan_split(const void* x, const void* a, const void* reset,
                         const void* h0, void* y, void* h_last, void* workspace,
                         size_t workspace_bytes, int B, int T, int W, int dtype,
                         void* stream) {
  return linear_scan_impl(__func__, x, a, reset, h0, y, h_last, workspace,
                          workspace_bytes, true, B, T, W, dtype, stream);
}

int rg_linear_scan_backward(const void* dy, const void* a, const void* reset,
                            const void* y, const void* h0, const void* dh_last,
                            void* dx, void* da, void* dh0, int B, int T, int W,
                            int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0, "%s: B=%d T=%d W=%d must be positive",
             __func__, B, T, W);
  RG_CHECK_PTR(dy);
  RG_CHECK_PTR(a);
  RG_CHECK_PTR(reset);
  RG_CHECK_PTR(y);
  RG_CHECK_PTR(dx);
  RG_CHECK_PTR(da);
  RG_CHECK_OPT_PTR(h0);
  RG_CHECK_OPT_PTR(dh_last);
  RG_CHECK_OPT_PTR(dh0);
  RG_REQUIRE(dx != a && dx != y && da != a && da != y && da != dy && dx != da,
             "%s: dx and da must not alias a, y or each other (da nor dy)",
             __func__);
  rg::ScanBwdArgs s{};
  s.dy = dy;
  s.a = a;
  s.reset = reset;
  s.y = y;
  s.h0 = (const float*)h0;
  s.dh_last = (const float*)dh_last;
  s.dx = dx;
  s.da = da;
  s.dh0 = (float*)dh0;
  s.B = B;
  s.T = T;
  s.W = W;
  return launch_status(__func__, rg::launch_linear_scan_backward(
                                     s, dtype, (hipStream_t)stream));
}

int rg_rglru_backward(const void* dy, const void* x, const void* gx_pre,
                      const void* ga_pre, const void* a_param,
                      const void* reset, const void* y, const void* h0,
                      const void* dh_last, void* dx, void* dgx_pre,
                      void* dga_pre, void* d_a_param_rows, void* dh0, int B,
                      int T, int W, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && W > 0, "%s: B=%d T=%d W=%d must be positive",
             __func__, B, T, W);
  RG_CHECK_PTR(dy);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(gx_pre);
  RG_CHECK_PTR(ga_pre);
  RG_CHECK_PTR(a_param);
  RG_CHECK_PTR(reset);
  RG_CHECK_PTR(y);
  RG_CHECK_PTR(dx);
  RG_CHECK_PTR(dgx_pre);
  RG_CHECK_PTR(dga_pre);
  RG_CHECK_PTR(d_a_param_rows);
  RG_CHECK_OPT_PTR(h0);
  RG_CHECK_OPT_PTR(dh_last);
  RG_CHECK_OPT_PTR(dh0);
  const void* ins[] = {dy, x, gx_pre, ga_pre, y};
  void* outs[] = {dx, dgx_pre, dga_pre};
  for (void* o : outs)
    for (const void* i : ins)
      RG_REQUIRE(o != i, "%s: an output aliases an input", __func__);
  RG_REQUIRE(dx != dgx_pre && dx != dga_pre && dgx_pre != dga_pre,
             "%s: outputs alias each other", __func__);
  rg::RglruBwdArgs s{};
  s.dy = dy;
  s.x = x;
  s.gx = gx_pre;
  s.ga = ga_pre;
  s.a_param = a_param;
  s.reset = reset;
  s.y = y;
  s.h0 = (const float*)h0;
  s.dh_last = (const float*)dh_last;
  s.dx = dx;
  s.dgx = dgx_pre;
  s.dga = dga_pre;
  s.dlam = (float*)d_a_param_rows;
  s.dh0 = (float*)dh0;
  s.B = B;
  s.T = T;
  s.W = W;
  return launch_status(
      __func__, rg::launch_rglru_backward(s, dtype, (hipStream_t)stream));
}

size_t rg_recurrent_step_workspace_bytes(int B, int W, int dtype) {
  if (B <= 0 || W <= 0) return 0;
  // conv output + two gate pre-activations, each [B,W], 256-byte aligned
  size_t one = ((size_t)B * W * esize(dtype) + 255) & ~(size_t)255;
  return 3 * one;
}

int rg_recurrent_step(const void* x, const void* segpos, int segpos_is_i64,
                      const void* conv_cache_in, void* conv_cache_out,
                      const void* h_in, void* h_out, const void* conv_w,
                      const void* conv_b, const void* w_x, const void* b_x,
                      const void* w_a, const void* b_a, const void* a_param,
                      void* y, void* workspace, size_t workspace_bytes, int B,
                      int W, int H, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && W > 0 && H > 0, "%s: B=%d W=%d H=%d must be positive",
             __func__, B, W, H);
  RG_REQUIRE(W % H == 0, "%s: W=%d is not a multiple of H=%d", __func__, W, H);
  RG_CHECK_PTR(conv_cache_in);
  RG_CHECK_PTR(conv_cache_out);
  RG_CHECK_PTR(h_in);
  RG_CHECK_PTR(h_out);
  const size_t need = rg_recurrent_step_workspace_bytes(B, W, dtype);
  if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    return fail(RG_ERR_WORKSPACE,
                "%s: workspace of %zu bytes (16-byte aligned) required, got %zu",
                __func__, need, workspace ? workspace_bytes : (size_t)0);
  const size_t one = need / 3;
  char* ws = (char*)workspace;
  void* xc = ws;
  void* gx = ws + one;
  void* ga = ws + 2 * one;
  int rc = rg_conv1d_step(x, conv_cache_in, conv_w, conv_b, xc, conv_cache_out,
                          B, W, 4, dtype, stream);
  if (rc != RG_OK) return rc;
  rc = rg_gates_gemm(xc, 0, nullptr, 0, nullptr, nullptr, w_x, b_x, w_a, b_a, gx,
                     ga, B, 1, W, H, dtype, stream);
  if (rc != RG_OK) return rc;
  return rg_lru_scan_fused(xc, 0, nullptr, nullptr, gx, ga, a_param, segpos,
                           segpos_is_i64, h_in, y, h_out, nullptr, B, 1, W,
                           dtype, stream);
}

int rg_recurrent_step_static(const void* x, const void* segpos,
                             int segpos_is_i64, const void* conv_cache_in,
                             void* conv_cache_out, const void* h_in,
                             void* h_out, const void* conv_w,
                             const void* conv_b, const void* w_x,
                             const void* b_x, const void* w_a, const void* b_a,
                             const void* a_param, void* y, int B, int W, int H,
                             int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && W > 0 && H > 0, "%s: B=%d W=%d H=%d must be positive",
             __func__, B, W, H);
  const size_t need = rg_recurrent_step_workspace_bytes(B, W, dtype);
  if (need > (size_t)RG_STEP_STATIC_SCRATCH_BYTES)
    return fail(RG_ERR_WORKSPACE,
                "%s: B=%d W=%d needs %zu bytes of scratch, the built-in buffer "
                "holds %zu: use rg_recurrent_step with a workspace",
                __func__, B, W, need, (size_t)RG_STEP_STATIC_SCRATCH_BYTES);
  hipError_t e;
  void* ws = step_scratch(&e);
  if (ws == nullptr) return launch_status(__func__, e);
  // the three launches write every scratch element they later read: nothing
  // has to be cleared between calls
  return rg_recurrent_step(x, segpos, segpos_is_i64, conv_cache_in,
                           conv_cache_out, h_in, h_out, conv_w, conv_b, w_x,
                           b_x, w_a, b_a, a_param, y, ws,
                           (size_t)RG_STEP_STATIC_SCRATCH_BYTES, B, W, H, dtype,
                           stream);
}

int rg_gelu_mul(const void* a, const void* g, void* out, int64_t n, int dtype,
                void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(n > 0, "%s: n=%lld must be positive", __func__, (long long)n);
  RG_CHECK_PTR(a);
  RG_CHECK_PTR(g);
  RG_CHECK_PTR(out);
  RG_REQUIRE((((uintptr_t)a | (uintptr_t)g | (uintptr_t)out) & 15) == 0,
             "%s: a, g and out must be 16-byte aligned", __func__);
  return launch_status(
      __func__, rg::launch_gelu_mul(a, g, out, n, dtype, (hipStream_t)stream));
}

int rg_gelu_mul_backward(const void* dout, const void* a, const void* g,
                         void* d_a, void* d_g, int64_t n, int dtype,
                         void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(n > 0, "%s: n=%lld must be positive", __func__, (long long)n);
  RG_CHECK_PTR(dout);
  RG_CHECK_PTR(a);
  RG_CHECK_PTR(g);
  RG_CHECK_PTR(d_a);
  RG_CHECK_PTR(d_g);
  RG_REQUIRE((((uintptr_t)dout | (uintptr_t)a | (uintptr_t)g | (uintptr_t)d_a |
               (uintptr_t)d_g) & 15) == 0,
             "%s: every operand must be 16-byte aligned", __func__);
  RG_REQUIRE(d_a != d_g && d_a != dout && d_a != a && d_a != g &&
                 d_g != dout && d_g != a && d_g != g,
             "%s: d_a and d_g must alias neither each other nor an input",
             __func__);
  return launch_status(__func__,
                       rg::launch_gelu_mul_backward(dout, a, g, d_a, d_g, n,
                                                    dtype, (hipStream_t)stream));
}

int rg_soft_cap(const void* x, void* out, int64_t n, float cap, int dtype,
                void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(n > 0, "%s: n=%lld must be positive", __func__, (long long)n);
  RG_REQUIRE(cap > 0.0f, "%s: cap=%g must be positive", __func__, (double)cap);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(out);
  return launch_status(
      __func__, rg::launch_soft_cap(x, out, n, cap, dtype, (hipStream_t)stream));
}

int rg_prefill_clock_probe(uint64_t* out) {
  g_prefill_timing.store(out, std::memory_order_relaxed);
  return RG_OK;
}

int rg_clock_probe(uint64_t* out, int iters, void* stream) {
  RG_REQUIRE(out != nullptr, "%s: out is null", __func__);
  RG_REQUIRE(iters > 0 && iters <= (1 << 20), "%s: iters=%d out of range",
             __func__, iters);
  return launch_status(
      __func__, rg::launch_clock_probe(out, iters, (hipStream_t)stream));
}

int rg_argmax_rows(const void* x, int64_t* out, int rows, int n, int dtype,
                   void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(rows > 0 && n > 0, "%s: rows=%d n=%d must be positive", __func__,
             rows, n);
  RG_CHECK_PTR(x);
  RG_REQUIRE(out != nullptr && ((uintptr_t)out & 7) == 0,
             "%s: out is null or not 8-byte aligned", __func__);
  return launch_status(__func__,
                       rg::launch_argmax_rows(x, out, rows, n, dtype,
                                              (hipStream_t)stream));
}

int rg_rms_norm(const void* x, const void* scale, void* out, int64_t rows,
                int width, float eps, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(rows > 0 && width > 0, "%s: rows=%lld width=%d must be positive",
             __func__, (long long)rows, width);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(scale);
  RG_CHECK_PTR(out);
  return launch_status(
      __func__, rg::launch_rms_norm(x, nullptr, scale, nullptr, out, rows,
                                    width, eps, dtype, (hipStream_t)stream));
}

int rg_add_rms_norm(const void* x, const void* addend, const void* scale,
                    void* sum_out, void* out, int64_t rows, int width,
                    float eps, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(rows > 0 && width > 0, "%s: rows=%lld width=%d must be positive",
             __func__, (long long)rows, width);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(addend);
  RG_CHECK_PTR(scale);
  RG_CHECK_PTR(sum_out);
  RG_CHECK_PTR(out);
  RG_REQUIRE(out != sum_out, "%s: out must not alias sum_out", __func__);
  return launch_status(
      __func__, rg::launch_rms_norm(x, addend, scale, sum_out, out, rows, width,
                                    eps, dtype, (hipStream_t)stream));
}

int rg_rope(const void* x, const void* positions, int positions_is_i64,
            const float* inv_freq, void* out, int64_t rows, int heads,
            int head_dim, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(rows > 0 && heads > 0 && head_dim > 0,
             "%s: rows=%lld heads=%d head_dim=%d must be positive", __func__,
             (long long)rows, heads, head_dim);
  RG_REQUIRE(head_dim % 4 == 0, "%s: head_dim=%d is not a multiple of 4",
             __func__, head_dim);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(positions);
  RG_CHECK_PTR(inv_freq);
  RG_CHECK_PTR(out);
  RG_REQUIRE(out != x, "%s: out must not alias x", __func__);
  return launch_status(
      __func__, rg::launch_rope(x, positions, positions_is_i64 ? 1 : 0,
                                inv_freq, out, rows, heads, head_dim, nullptr,
                                nullptr, 0, dtype, (hipStream_t)stream));
}

int rg_rope_pair(const void* q, const void* k, const void* positions,
                 int positions_is_i64, const float* inv_freq, void* q_out,
                 void* k_out, int64_t rows, int q_heads, int k_heads,
                 int head_dim, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(rows > 0 && q_heads > 0 && k_heads > 0 && head_dim > 0,
             "%s: rows=%lld q_heads=%d k_heads=%d head_dim=%d must be positive",
             __func__, (long long)rows, q_heads, k_heads, head_dim);
  RG_REQUIRE(head_dim % 4 == 0, "%s: head_dim=%d is not a multiple of 4",
             __func__, head_dim);
  RG_CHECK_PTR(q);
  RG_CHECK_PTR(k);
  RG_CHECK_PTR(positions);
  RG_CHECK_PTR(inv_freq);
  RG_CHECK_PTR(q_out);
  RG_CHECK_PTR(k_out);
  RG_REQUIRE(q_out != q && k_out != k, "%s: outputs must not alias inputs",
             __func__);
  return launch_status(
      __func__, rg::launch_rope(q, positions, positions_is_i64 ? 1 : 0,
                                inv_freq, q_out, rows, q_heads, head_dim, k,
                                k_out, k_heads, dtype, (hipStream_t)stream));
}

int rg_attention_prefill(const void* q, const void* k, const void* v_t,
                         const void* first_key, void* out, int B, int T,
                         int T_pad, int H, int head_dim, float scale, int dtype,
                         void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && T > 0 && H > 0, "%s: B=%d T=%d H=%d must be positive",
             __func__, B, T, H);
  if (dtype != RG_DTYPE_BF16 || head_dim != 256)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs bf16 and head_dim == 256 (dtype=%d head_dim=%d)",
                __func__, dtype, head_dim);
  RG_REQUIRE(T_pad >= T && T_pad % 64 == 0,
             "%s: T_pad=%d must be a multiple of 64 and at least T=%d",
             __func__, T_pad, T);
  RG_REQUIRE((int64_t)T * H * 512 < ((int64_t)1 << 31) &&
                 (int64_t)T_pad * 512 < ((int64_t)1 << 31),
             "%s: T=%d H=%d: a row's queries exceed 2 GiB", __func__, T, H);
  RG_CHECK_PTR(q);
  RG_CHECK_PTR(k);
  RG_CHECK_PTR(v_t);
  RG_CHECK_PTR(first_key);
  RG_CHECK_PTR(out);
  RG_REQUIRE(out != q && out != k && out != v_t,
             "%s: out must not alias an input", __func__);
  rg::AttnPrefillArgs a{};
  a.q = q;
  a.k = k;
  a.v_t = v_t;
  a.lo = first_key;
  a.out = out;
  a.B = B;
  a.T = T;
  a.T_pad = T_pad;
  a.H = H;
  a.scale = scale;
  return launch_status(
      __func__, rg::launch_attn_prefill_bf16(a, (hipStream_t)stream));
}

int rg_attention_decode_probs(const void* scores, const void* q,
                              const void* k_new, const int32_t* num_tokens,
                              void* probs, int B, int heads, int head_dim,
                              int window, float scale, int dtype,
                              void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && heads > 0 && head_dim > 0 && window > 0,
             "%s: B=%d heads=%d head_dim=%d window=%d must be positive",
             __func__, B, heads, head_dim, window);
  RG_CHECK_PTR(scores);
  RG_CHECK_PTR(q);
  RG_CHECK_PTR(k_new);
  RG_CHECK_PTR(num_tokens);
  RG_CHECK_PTR(probs);
  return launch_status(
      __func__,
      rg::launch_attn_decode_probs(scores, q, k_new, num_tokens, probs, B,
                                   heads, head_dim, window, scale, dtype,
                                   (hipStream_t)stream));
}

int rg_attention_decode_finish(const void* from_ring, const void* probs,
                               const void* k_new, const void* v_new, void* out,
                               void* ring_keys, void* ring_values,
                               int32_t* num_tokens, int B, int heads,
                               int head_dim, int window, int update_cache,
                               int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && heads > 0 && head_dim > 0 && window > 0,
             "%s: B=%d heads=%d head_dim=%d window=%d must be positive",
             __func__, B, heads, head_dim, window);
  RG_CHECK_PTR(from_ring);
  RG_CHECK_PTR(probs);
  RG_CHECK_PTR(k_new);
  RG_CHECK_PTR(v_new);
  RG_CHECK_PTR(out);
  RG_CHECK_PTR(num_tokens);
  if (update_cache) {
    RG_CHECK_PTR(ring_keys);
    RG_CHECK_PTR(ring_values);
  }
  return launch_status(
      __func__,
      rg::launch_attn_decode_finish(from_ring, probs, k_new, v_new, out,
                                    ring_keys, ring_values, num_tokens, B,
                                    heads, head_dim, window,
                                    update_cache ? 1 : 0, dtype,
                                    (hipStream_t)stream));
}

size_t rg_attention_decode_fused_workspace_bytes(int B, int heads, int window) {
  if (B <= 0 || heads <= 0 || heads > 16 || window <= 0) return 0;
  const size_t chunks =
      ((size_t)window + rg::kAttnDecodeChunk - 1) / rg::kAttnDecodeChunk;
  if (chunks > (size_t)rg::kAttnDecodeMaxChunks) return 0;
  return (size_t)B * chunks * heads * (256 + 2) * sizeof(float);
}

int rg_attention_decode_fused(const void* q, int64_t ldq, const void* k_new,
                              int64_t ldk, const void* v_new, int64_t ldv,
                              const void* positions, int positions_are_i64,
                              const float* inv_freq, void* ring_keys,
                              void* ring_values, int32_t* num_tokens, void* out,
                              void* workspace, size_t workspace_bytes, int B,
                              int heads, int head_dim, int window, float scale,
                              int update_cache, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && heads > 0 && head_dim > 0 && window > 0,
             "%s: B=%d heads=%d head_dim=%d window=%d must be positive",
             __func__, B, heads, head_dim, window);
  const size_t need = rg_attention_decode_fused_workspace_bytes(B, heads, window);
  if (dtype != RG_DTYPE_BF16 || head_dim != 256 || need == 0 || B > 65535)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs bf16, head_dim 256, at most 16 heads, window <= %d, "
                "B <= 65535 (dtype=%d head_dim=%d heads=%d window=%d B=%d)",
                __func__, rg::kAttnDecodeChunk * rg::kAttnDecodeMaxChunks, dtype,
                head_dim, heads, window, B);
  RG_CHECK_PTR(q);
  RG_CHECK_PTR(k_new);
  RG_CHECK_PTR(v_new);
  RG_CHECK_PTR(positions);
  RG_CHECK_PTR(inv_freq);
  RG_CHECK_PTR(ring_keys);
  RG_CHECK_PTR(ring_values);
  RG_CHECK_PTR(num_tokens);
  RG_CHECK_PTR(out);
  RG_REQUIRE(ldq >= (int64_t)heads * 256 && ldk >= 256 && ldv >= 256 &&
                 ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0,
             "%s: row strides ldq=%lld ldk=%lld ldv=%lld must cover a row and "
             "be multiples of 8 elements", __func__, (long long)ldq,
             (long long)ldk, (long long)ldv);
  RG_REQUIRE(aligned16(q) && aligned16(k_new) && aligned16(v_new) &&
                 aligned16(ring_keys) && aligned16(ring_values) && aligned16(out),
             "%s: tensors must be 16-byte aligned", __func__);
  if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
    return fail(RG_ERR_WORKSPACE,
                "%s: workspace of %zu bytes (16-byte aligned) required, got %zu",
                __func__, need, workspace ? workspace_bytes : (size_t)0);
  rg::AttnDecodeArgs a{};
  a.q = (const uint16_t*)q;
  a.k_new = (const uint16_t*)k_new;
  a.v_new = (const uint16_t*)v_new;
  a.ldq = ldq;
  a.ldk = ldk;
  a.ldv = ldv;
  a.pos = positions;
  a.pos_kind = positions_are_i64 ? 1 : 0;
  a.inv_freq = inv_freq;
  a.ring_k = (uint16_t*)ring_keys;
  a.ring_v = (uint16_t*)ring_values;
  a.num_tokens = num_tokens;
  a.out = (uint16_t*)out;
  a.B = B;
  a.heads = heads;
  a.window = window;
  a.chunks = (window + rg::kAttnDecodeChunk - 1) / rg::kAttnDecodeChunk;
  a.part_o = (float*)workspace;
  a.part_ml = a.part_o + (size_t)B * a.chunks * heads * 256;
  a.scale = scale;
  a.update = update_cache ? 1 : 0;
  return launch_status(__func__,
                       rg::launch_attn_decode_fused(a, (hipStream_t)stream));
}

size_t rg_packed_gate_weights_bytes(int W, int H, int dtype) {
  if (W <= 0 || H <= 0 || W % H != 0 || dtype != RG_DTYPE_BF16 || W / H != 256)
    return 0;
  return (size_t)2 * H * 256 * 256 * 2;
}

int rg_pack_gate_weights(const void* w_x, const void* w_a, void* packed, int W,
                         int H, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(W > 0 && H > 0 && W % H == 0, "%s: W=%d H=%d", __func__, W, H);
  if (dtype != RG_DTYPE_BF16 || W / H != 256)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs bf16 and W/H == 256 (dtype=%d W=%d H=%d)", __func__,
                dtype, W, H);
  RG_CHECK_PTR(w_x);
  RG_CHECK_PTR(w_a);
  RG_CHECK_PTR(packed);
  RG_REQUIRE(packed != w_x && packed != w_a, "%s: packed must not alias",
             __func__);
  return launch_status(__func__, rg::launch_pack_gate_weights(
                                     w_x, w_a, packed, H, (hipStream_t)stream));
}

size_t rg_linear_packed_bytes(int N, int K, int gelu_pair) {
  if (N <= 0 || K <= 0 || K % 64 != 0 || N % 32 != 0) return 0;
  if (gelu_pair && N % 64 != 0) return 0;
  return (size_t)N * K * 2;
}

int rg_linear_pack(const void* w, int layout, int groups, int gelu_pair,
                   void* packed, int N, int K, void* stream) {
  RG_REQUIRE(N > 0 && K > 0, "%s: N=%d K=%d must be positive", __func__, N, K);
  if (rg_linear_packed_bytes(N, K, gelu_pair) == 0)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs K %% 64 == 0 and N %% 32 == 0 (64 for gelu pairs), "
                "got N=%d K=%d", __func__, N, K);
  RG_REQUIRE(layout == 0 || layout == 1, "%s: layout=%d", __func__, layout);
  RG_REQUIRE(groups >= 1 && N % groups == 0,
             "%s: N=%d is not a multiple of groups=%d", __func__, N, groups);
  RG_CHECK_PTR(w);
  RG_CHECK_PTR(packed);
  RG_REQUIRE(packed != w, "%s: packed must not alias w", __func__);
  return launch_status(
      __func__, rg::launch_linear_pack(w, packed, N, K, layout, groups,
                                       gelu_pair != 0, (hipStream_t)stream));
}

size_t rg_linear_rows_workspace_bytes(int M, int K, int N) {
  if (M <= 0 || K <= 0 || N <= 0) return 0;
  const int slices = rg::linear_rows_k_slices(K, N);
  return slices > 1 ? (size_t)slices * M * N * sizeof(float) : 0;
}

int rg_linear_rows(const void* x, const void* w_packed, const void* bias,
                   const void* residual, void* out, void* workspace,
                   size_t workspace_bytes, int M, int K, int N, int groups,
                   int gelu_pair, void* stream) {
  RG_REQUIRE(M > 0 && K > 0 && N > 0, "%s: M=%d K=%d N=%d must be positive",
             __func__, M, K, N);
  if (M > 64 || rg_linear_packed_bytes(N, K, gelu_pair) == 0)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs M <= 64, K %% 64 == 0, N %% 32 == 0 (64 for gelu "
                "pairs), got M=%d K=%d N=%d", __func__, M, K, N);
  RG_REQUIRE(groups >= 1 && N % groups == 0 && (N / groups) % 4 == 0,
             "%s: N=%d / groups=%d must be a multiple of 4", __func__, N,
             groups);
  RG_REQUIRE(!gelu_pair || (groups == 1 && residual == nullptr),
             "%s: gelu pairs take one group and no residual", __func__);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(w_packed);
  RG_CHECK_PTR(out);
  RG_CHECK_OPT_PTR(bias);
  RG_CHECK_OPT_PTR(residual);
  RG_REQUIRE(out != x, "%s: out must not alias x", __func__);
  const size_t need = rg_linear_rows_workspace_bytes(M, K, N);
  if (!gelu_pair && need > 0 &&
      (workspace == nullptr || workspace_bytes < need || !aligned16(workspace)))
    return fail(RG_ERR_WORKSPACE,
                "%s: workspace of %zu bytes (16-byte aligned) required, got %zu",
                __func__, need, workspace ? workspace_bytes : (size_t)0);
  rg::LinearArgs a;
  a.x = x;
  a.w_packed = w_packed;
  a.bias = bias;
  a.residual = residual;
  a.out = out;
  a.partial = (float*)workspace;
  a.M = M;
  a.K = K;
  a.N = N;
  a.group_width = N / groups;
  return launch_status(
      __func__, rg::launch_linear_rows(a, gelu_pair != 0, (hipStream_t)stream));
}

int rg_linear_rows_partial(const void* x, const void* w_packed, void* partial,
                           int M, int K, int N, int slices, void* stream) {
  RG_REQUIRE(M > 0 && K > 0 && N > 0, "%s: M=%d K=%d N=%d must be positive",
             __func__, M, K, N);
  if (M > 64 || rg_linear_packed_bytes(N, K, 0) == 0)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs M <= 64, K %% 64 == 0, N %% 32 == 0, got M=%d K=%d "
                "N=%d", __func__, M, K, N);
  RG_REQUIRE(slices >= 1 && slices <= 8, "%s: slices=%d not in 1..8", __func__,
             slices);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(w_packed);
  RG_CHECK_PTR(partial);
  RG_REQUIRE(partial != x, "%s: partial must not alias x", __func__);
  rg::LinearArgs a{};
  a.x = x;
  a.w_packed = w_packed;
  a.partial = (float*)partial;
  a.M = M;
  a.K = K;
  a.N = N;
  a.group_width = N;
  return launch_status(__func__, rg::launch_linear_rows_partial(
                                     a, slices, (hipStream_t)stream));
}

int rg_add_rms_norm_partial(const void* partial, int slices, const void* bias,
                            const void* addend, const void* scale,
                            void* sum_out, void* out, int rows, int width,
                            float eps, int dtype, void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(rows > 0 && width > 0, "%s: rows=%d width=%d must be positive",
             __func__, rows, width);
  if (dtype != RG_DTYPE_BF16 || width % 8 != 0 || width > 4096)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs bf16 and width %% 8 == 0, width <= 4096 (dtype=%d "
                "width=%d)", __func__, dtype, width);
  RG_REQUIRE(slices >= 1 && slices <= 8, "%s: slices=%d not in 1..8", __func__,
             slices);
  RG_CHECK_PTR(partial);
  RG_CHECK_PTR(scale);
  RG_CHECK_PTR(sum_out);
  RG_CHECK_PTR(out);
  RG_CHECK_OPT_PTR(bias);
  RG_CHECK_OPT_PTR(addend);
  RG_REQUIRE(out != sum_out, "%s: out must not alias sum_out", __func__);
  return launch_status(
      __func__, rg::launch_rms_norm_partial((const float*)partial, slices, bias,
                                            addend, scale, sum_out, out, rows,
                                            width, eps, (hipStream_t)stream));
}

#undef RG_WHO
#define RG_WHO who
static int recurrent_step_packed_impl(
    const char* who, const void* x, const void* gate_branch,
    const void* segpos, int segpos_is_i64, const void* conv_cache_in,
    void* conv_cache_out, const void* h_in, void* h_out, const void* conv_w,
    const void* conv_b, const void* w_packed, const void* b_x, const void* b_a,
    const void* a_param, void* y, int B, int W, int H, int dtype,
    void* stream) {
  RG_CHECK_DTYPE(dtype);
  RG_REQUIRE(B > 0 && W > 0 && H > 0, "%s: B=%d W=%d H=%d must be positive",
             who, B, W, H);
  RG_REQUIRE(W % H == 0, "%s: W=%d is not a multiple of H=%d", who, W, H);
  if (dtype != RG_DTYPE_BF16 || W / H != 256)
    return fail(RG_ERR_UNSUPPORTED,
                "%s: needs bf16 and W/H == 256 (dtype=%d W=%d H=%d)", who,
                dtype, W, H);
  RG_CHECK_PTR(x);
  RG_CHECK_PTR(segpos);
  RG_CHECK_PTR(conv_cache_in);
  RG_CHECK_PTR(conv_cache_out);
  RG_CHECK_PTR(h_in);
  RG_CHECK_PTR(h_out);
  RG_CHECK_PTR(conv_w);
  RG_CHECK_PTR(conv_b);
  RG_CHECK_PTR(w_packed);
  RG_CHECK_PTR(b_x);
  RG_CHECK_PTR(b_a);
  RG_CHECK_PTR(a_param);
  RG_CHECK_PTR(y);
  RG_CHECK_OPT_PTR(gate_branch);
  RG_REQUIRE(gate_branch == nullptr || gate_branch != x,
             "%s: gate_branch must not alias x", who);
  RG_REQUIRE(y != x, "%s: y must not alias x", who);
  rg::StepArgs a{};
  a.x = x;
  a.segpos = segpos;
  a.seg_kind = segpos_is_i64 ? 1 : 0;
  a.cache_in = conv_cache_in;
  a.cache_out = conv_cache_out;
  a.h_in = (const float*)h_in;
  a.h_out = (float*)h_out;
  a.conv_w = conv_w;
  a.conv_b = conv_b;
  a.w_packed = w_packed;
  a.b[0] = b_x;
  a.b[1] = b_a;
  a.a_param = a_param;
  a.y = y;
  a.gate_branch = gate_branch;
  a.B = B;
  a.W = W;
  a.H = H;
  return launch_status(who,
                       rg::launch_block_step_bf16(a, (hipStream_t)stream));
}
#undef RG_WHO
#define RG_WHO __func__

int rg_recurrent_step_packed(const void* x, const void* segpos,
                             int segpos_is_i64, const void* conv_cache_in,
                             void* conv_cache_out, const void* h_in,
                             void* h_out, const void* conv_w,
                             const void* conv_b, const void* w_packed,
                             const void* b_x, const void* b_a,
                             const void* a_param, void* y, int B, int W, int H,
                             int dtype, void* stream) {
  return recurrent_step_packed_impl(__func__, x, nullptr, segpos, segpos_is_i64,
                                    conv_cache_in, conv_cache_out, h_in, h_out,
                                    conv_w, conv_b, w_packed, b_x, b_a, a_param,
                                    y, B, W, H, dtype, stream);
}

int rg_recurrent_step_gelu_mul(const void* x, const void* gate_branch,
                               const void* segpos, int segpos_is_i64,
                               const void* conv_cache_in, void* conv_cache_out,
                               const void* h_in, void* h_out,
                               const void* conv_w, const void* conv_b,
                               const void* w_packed, const void* b_x,
                               const void* b_a, const void* a_param, void* out,
                               int B, int W, int H, int dtype, void* stream) {
  RG_CHECK_PTR(gate_branch);
  return recurrent_step_packed_impl(__func__, x, gate_branch, segpos,
                                    segpos_is_i64, conv_cache_in,
                                    conv_cache_out, h_in, h_out, conv_w, conv_b,
                                    w_packed, b_x, b_a, a_param, out, B, W, H,
                                    dtype, stream);
}

}  // extern "C"
