// Weight and bias gradients of both gate projections of RGLRU.forward in one
// pass (bf16, 256-wide heads): what autograd forms for
//   y[m, h, j] = sum_i x[m, h, i] w[h, i, j] + b[h, j]
// (recurrentgemma/torch/layers.py:127-137, called twice on the same x at
// :338-339) from the gradients dy of the two outputs:
//   dw[h, i, j] = sum_m x[m, h, i] dy[m, h, j],   db[h, j] = sum_m dy[m, h, j].
// Per head and gate that is a 256 x M by M x 256 product whose long dimension
// is the one both operands are strided in: x and dy are [M, W] with the
// channel fastest, the matrix instruction wants each lane's eight k (here: m)
// in one register quad.  The library's batched product on strided views takes
// 91 us per gate at M = 8192, W = 2560.
//
// Here a workgroup of eight waves owns a 128 x 128 tile of one head's dw for
// one gate and a range of rows m.  Per step of 64 rows, waves 0-3 load the
// 64 x 128 tile of x and waves 4-7 that of dy, each thread four consecutive
// rows of eight channels (16 bytes per row); it turns its 4 x 8 values into
// eight 4 x 1 columns in registers (v_perm_b32) and writes them into LDS as
// [channel][m] -- eight 8-byte writes --, the 16-byte chunks of a channel's
// 64 m placed so that the operand reads (16 bytes per lane: eight consecutive
// m of one channel) meet no bank twice and the writes spread evenly over the
// banks.  Wave (wi, wj) multiplies rows 32 wi .. +31 of the tile by columns
// 64 wj .. +63: per 16 m one A and two B operand reads and two
// v_mfma_f32_32x32x16_bf16.  Rows are requested two steps before they go to
// LDS; two LDS buffers, one barrier a step.  The workgroups with the tile's
// first rows also add up dy's columns for db (dot products with 1.0).  Row
// ranges (splits of M: as many as keep every workgroup resident at once, two
// to a CU) leave float32 partial sums in the workspace; a second kernel adds
// them in a fixed order and rounds once: results do not vary from run to run.
//
// Measured at M = 8192, W = 2560 (H = 10: 480 workgroups): 36 us + 6 us for
// the second kernel, where the library's two batched products and two column
// sums take 245 us.  Bound by the LDS round trip of the operands (every value
// is written once and read 1.5 times per 2 matrix instructions), not by the
// matrix pipe (0.6 PFLOP/s, a quarter of its peak) or by memory (126 MB in).
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kBW = 256;        // head width
constexpr int kTile = 128;      // tile of dw: kTile x kTile
constexpr int kStep = 64;       // rows m per step
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kChanBytes = kStep * 2;              // a channel's m of a step
constexpr int kSideBytes = kTile * kChanBytes;     // x side or dy side: 16 KB
constexpr int kBufBytes = 2 * kSideBytes;
constexpr int kLdsBytes = 2 * kBufBytes;           // two buffers: 64 KB

// Byte offset of 16-byte chunk `chunk` (eight m) of channel `ch` inside a
// side.  The chunk's place in the channel's 128 bytes is permuted by the
// channel's number so that the lanes that read chunk c of 8 (or 16)
// consecutive channels hit 8 (16) different 16-byte columns of the banks,
// whether a bank row is 128 or 256 bytes, and the 64 lanes that write 8 bytes
// each for channels 8 apart spread evenly over them.
__device__ __forceinline__ uint32_t chunk_at(int ch, int chunk) {
  return (uint32_t)ch * kChanBytes +
         (uint32_t)((chunk ^ ch ^ (ch >> 3)) & 7) * 16u;
}

struct WgradArgs {
  const void* x;        // [M, W] bf16
  const void* dy[2];    // [M, W] bf16 per gate
  float* part_w;        // [splits][2 H][256][256]
  float* part_b;        // [splits][2 H][256]
  int64_t M;
  int W, H;
  int splits;
  int rows_per_split;   // a multiple of kStep
};

// (four waves per SIMD: two workgroups share a CU, hence at most 128 registers)
__global__ void __launch_bounds__(kThreads, 4) gates_wgrad_kernel(WgradArgs p) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // The eight workgroups of a (head, split) -- two gates x four tiles -- read
  // the same rows of x and share dy by pairs.  Workgroups go to the eight XCDs
  // in turn (linear id modulo 8), each with an L2 of its own: those eight are
  // dealt to ONE XCD, so that the rows come from memory once (group g runs on
  // XCD g % 8; the grid is rounded up to whole rounds of eight groups and the
  // surplus exits).
  const int xcd = blockIdx.x & 7;
  const int in_xcd = blockIdx.x >> 3;
  const int group = (in_xcd >> 3) * 8 + xcd;
  if (group >= p.H * p.splits) return;
  const int which = in_xcd & 7;
  const int tj = which & 1;
  const int ti = (which >> 1) & 1;
  const int gate = which >> 2;
  const int head = group % p.H;
  const int split = group / p.H;
  const int64_t m_begin = (int64_t)split * p.rows_per_split;
  int64_t m_end = m_begin + p.rows_per_split;
  if (m_end > p.M) m_end = p.M;
  const int steps = m_begin < m_end ? (int)((m_end - m_begin + kStep - 1) / kStep) : 0;

  // ---- loader role: which matrix, which 8 channels, which 4 rows of a step
  const int side = wave >> 2;                // 0: x (A operand), 1: dy (B)
                                             // (the same for a whole wave)
  const int ch8 = tid & 15;                  // channels 8 ch8 .. +7 of the tile
  const int q = (tid >> 4) & 15;             // rows 4 q .. 4 q + 3 of the step
  const uint32_t row_bytes = 2u * (uint32_t)p.W;
  const char* src = (const char*)(side == 0 ? p.x : p.dy[gate]);
  const int first_ch = head * kBW + (side == 0 ? ti : tj) * kTile + 8 * ch8;
  // rows past m_end read as zeros: a descriptor over the split's rows only
  const uint64_t span = (uint64_t)(m_end > m_begin ? m_end - m_begin : 0) * row_bytes;
  const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(
      src + m_begin * (int64_t)row_bytes, (uint32_t)(span < 0xffffffffu ? span : 0xffffffffu));
  // (two sets of row registers: the rows of a step are requested two steps
  // before they go to LDS, a memory round trip being several steps long)
  u32x4 rows_even[4], rows_odd[4];
  auto request = [&](int step, u32x4 (&rows)[4]) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
      rows[r] = __builtin_amdgcn_raw_buffer_load_b128(
          rsrc, (uint32_t)(step * kStep + 4 * q + r) * row_bytes +
                    2u * (uint32_t)first_ch, 0, 0);
  };
  // the thread's 4 rows x 8 channels as eight columns of four, into buffer b
  auto deposit = [&](int b, const u32x4 (&rows)[4]) {
    unsigned char* base = lds + b * kBufBytes + side * kSideBytes;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      // dword c of a row holds channels 2 c (low half) and 2 c + 1
      const uint32_t lo01 = __builtin_amdgcn_perm(rows[1][c], rows[0][c], 0x05040100u);
      const uint32_t lo23 = __builtin_amdgcn_perm(rows[3][c], rows[2][c], 0x05040100u);
      const uint32_t hi01 = __builtin_amdgcn_perm(rows[1][c], rows[0][c], 0x07060302u);
      const uint32_t hi23 = __builtin_amdgcn_perm(rows[3][c], rows[2][c], 0x07060302u);
      const int ch = 8 * ch8 + 2 * c;
      // rows 4 q .. 4 q + 3: half (q & 1) of chunk q >> 1
      *reinterpret_cast<u32x2*>(base + chunk_at(ch, q >> 1) + 8 * (q & 1)) =
          u32x2{lo01, lo23};
      *reinterpret_cast<u32x2*>(base + chunk_at(ch + 1, q >> 1) + 8 * (q & 1)) =
          u32x2{hi01, hi23};
    }
  };

  // ---- multiplier role
  const int wi = wave >> 1;   // rows 32 wi .. of the tile (input channels)
  const int wj = wave & 1;    // columns 64 wj .. (output channels)
  const int l32 = lane & 31;
  const int kg = lane >> 5;
  f32x16 acc0, acc1;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc0[r] = acc1[r] = 0.0f;
  // db: in the workgroups with ti == 0 thread t sums 16 of a step's 64 m of
  // column t % 128 of dy (dot products with 1.0: two values an instruction);
  // the four threads of a column meet at the end
  const bool sums_bias = ti == 0;
  const int bias_col = tid & (kTile - 1);
  const int bias_part = tid >> 7;
  float bias_sum = 0.0f;

  // step `step` from buffer step % 2; the rows of step + 2 requested, those
  // of step + 1 moved to the other buffer behind the products
  auto one_step = [&](int step, u32x4 (&mine)[4], const u32x4 (&next)[4]) {
    const int b = step & 1;
    if (step + 2 < steps) request(step + 2, mine);
    const unsigned char* a_side = lds + b * kBufBytes;
    const unsigned char* b_side = a_side + kSideBytes;
#pragma unroll
    for (int ks = 0; ks < kStep / 16; ++ks) {
      union { bf16x8 v; u32x4 q; } fa, fb0, fb1;
      fa.q = *reinterpret_cast<const u32x4*>(a_side + chunk_at(32 * wi + l32, 2 * ks + kg));
      fb0.q = *reinterpret_cast<const u32x4*>(b_side + chunk_at(64 * wj + l32, 2 * ks + kg));
      fb1.q = *reinterpret_cast<const u32x4*>(b_side + chunk_at(64 * wj + 32 + l32, 2 * ks + kg));
      acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.v, fb0.v, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.v, fb1.v, acc1, 0, 0, 0);
    }
    if (sums_bias) {
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(
            b_side + chunk_at(bias_col, 2 * bias_part + c));
#pragma unroll
        for (int e = 0; e < 4; ++e)
          asm("v_dot2_f32_bf16 %0, %1, %2, %0"
              : "+v"(bias_sum)
              : "v"(v[e]), "v"(0x3f803f80u));  // (1.0, 1.0) in bf16
      }
    }
    if (step + 1 < steps) deposit(b ^ 1, next);
    __syncthreads();
  };
  if (steps > 0) {
    request(0, rows_even);
    if (steps > 1) request(1, rows_odd);
    deposit(0, rows_even);
    __syncthreads();
  }
  for (int step = 0; step < steps; step += 2) {
    one_step(step, rows_even, rows_odd);
    if (step + 1 < steps) one_step(step + 1, rows_odd, rows_even);
  }

  // ---- partial sums of this split.  Result layout of the instruction: lane
  //      (g = lane / 32, n = lane % 32) register r holds row 8 (r / 4) + 4 g +
  //      r % 4, column n of the 32 x 32 product.
  const int slot = (head * 2 + gate);
  float* out = p.part_w + ((int64_t)split * 2 * p.H + slot) * (kBW * kBW);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int i = ti * kTile + 32 * wi + 8 * (r >> 2) + 4 * kg + (r & 3);
    const int j = tj * kTile + 64 * wj + l32;
    out[i * kBW + j] = acc0[r];
    out[i * kBW + j + 32] = acc1[r];
  }
  if (sums_bias) {
    // (the dot instruction's result may be read by another kind of
    // instruction only three issue slots later)
    asm volatile("s_nop 2" : "+v"(bias_sum));
    float* meet = reinterpret_cast<float*>(lds);  // the buffers are free now
    meet[tid] = bias_sum;
    __syncthreads();
    if (tid < kTile)
      p.part_b[((int64_t)split * 2 * p.H + slot) * kBW + tj * kTile + tid] =
          (meet[tid] + meet[tid + 128]) + (meet[tid + 256] + meet[tid + 384]);
  }
}

// Sums the splits' partial sums in their order and rounds once to bf16: the
// weights' (four elements a thread) and, behind them, the biases'.
__global__ void __launch_bounds__(256)
gates_wgrad_finish_kernel(const float* __restrict__ part_w,
                          const float* __restrict__ part_b, int splits, int H,
                          uint16_t* __restrict__ dwx, uint16_t* __restrict__ dwa,
                          uint16_t* __restrict__ dbx, uint16_t* __restrict__ dba) {
  const int64_t per_w = (int64_t)2 * H * kBW * kBW;
  const int64_t per_b = (int64_t)2 * H * kBW;
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (e < per_w) {
    f32x4 sum = {0, 0, 0, 0};
    for (int k = 0; k < splits; ++k)
      sum += *reinterpret_cast<const f32x4*>(part_w + (int64_t)k * per_w + e);
    // element e of [head][gate][256][256]
    const int64_t slot = e / (kBW * kBW);
    const int64_t within = e % (kBW * kBW);
    uint16_t* out = ((slot & 1) ? dwa : dwx) + (slot >> 1) * (kBW * kBW) + within;
    *reinterpret_cast<u32x2*>(out) =
        u32x2{pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3])};
  } else if (e - per_w < per_b && dbx != nullptr) {
    const int64_t eb = e - per_w;
    f32x4 sum = {0, 0, 0, 0};
    for (int k = 0; k < splits; ++k)
      sum += *reinterpret_cast<const f32x4*>(part_b + (int64_t)k * per_b + eb);
    const int64_t slot = eb / kBW;
    const int64_t within = eb % kBW;
    uint16_t* out = ((slot & 1) ? dba : dbx) + (slot >> 1) * kBW + within;
    *reinterpret_cast<u32x2*>(out) =
        u32x2{pack_bf16x2(sum[0], sum[1]), pack_bf16x2(sum[2], sum[3])};
  }
}

int wgrad_splits(int64_t M, int H) {
  // as many row ranges as keep all workgroups (8 per head and range) resident
  // at once, two to a CU (a second round of a few would double the time);
  // ranges of whole steps, at least 4 steps each
  int64_t want = 512 / (8 * (int64_t)H);
  const int64_t most = (M + 4 * kStep - 1) / (4 * kStep);
  if (want > most) want = most;
  if (want < 1) want = 1;
  return (int)want;
}

}  // namespace

bool gates_wgrad_serves(int64_t M, int W, int H) {
  return M > 0 && H > 0 && W == H * kBW && M * (int64_t)W * 2 < ((int64_t)1 << 46);
}

size_t gates_wgrad_workspace_bytes(int64_t M, int W, int H) {
  if (!gates_wgrad_serves(M, W, H)) return 0;
  const int splits = wgrad_splits(M, H);
  return (size_t)splits * 2 * H * (kBW * kBW + kBW) * sizeof(float);
}

hipError_t launch_gates_wgrad(const void* x, const void* dgx, const void* dga,
                              void* dwx, void* dwa, void* dbx, void* dba,
                              void* workspace, int64_t M, int W, int H,
                              hipStream_t s) {
  const int splits = wgrad_splits(M, H);
  int64_t rows = (M + splits - 1) / splits;
  rows = (rows + kStep - 1) / kStep * kStep;
  // a split's rows must fit the 32-bit range of its descriptor
  if ((uint64_t)rows * (uint64_t)W * 2u >= 0xffffffffull) return hipErrorInvalidValue;
  WgradArgs a{};
  a.x = x;
  a.dy[0] = dgx;
  a.dy[1] = dga;
  a.part_w = (float*)workspace;
  a.part_b = a.part_w + (size_t)splits * 2 * H * kBW * kBW;
  a.M = M;
  a.W = W;
  a.H = H;
  a.splits = splits;
  a.rows_per_split = (int)rows;
  static OncePerDevice once;
  hipError_t e = set_max_dynamic_lds(once, (const void*)gates_wgrad_kernel, kLdsBytes);
  if (e != hipSuccess) return e;
  const int64_t rounds = ((int64_t)H * splits + 7) / 8;
  if (rounds * 64 > 0x7fffffff) return hipErrorInvalidValue;
  gates_wgrad_kernel<<<dim3((unsigned)(rounds * 64)), kThreads, kLdsBytes, s>>>(a);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  const int64_t items = ((int64_t)2 * H * kBW * kBW + (int64_t)2 * H * kBW) / 4;
  gates_wgrad_finish_kernel<<<dim3((unsigned)((items + 255) / 256)), 256, 0, s>>>(
      a.part_w, a.part_b, splits, H, (uint16_t*)dwx, (uint16_t*)dwa,
      (uint16_t*)dbx, (uint16_t*)dba);
  e = hipGetLastError();
  return e;
}

}  // namespace rg
