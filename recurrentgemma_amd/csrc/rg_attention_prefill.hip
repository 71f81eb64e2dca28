// Prompt-pass attention of the local-attention block: sliding-window,
// multi-query (all heads share one key/value head), causal within a document
// (recurrentgemma/torch/modules.py:404-476 with the mask of :86-127), bf16,
// head dimension 256, as one kernel -- scores, mask, softmax and the weighted
// sum of the values without the [T, T] matrices in memory.
//
// The mask of a prompt is a band: query t sees the keys lo[t] .. t, where
// lo[t] = max(first token of t's document, t - window) is supplied by the
// caller (non-decreasing in t).
//
// One workgroup of four waves per (row, head, 128 queries); a wave owns 32
// queries.  Keys and values come by in tiles of 64 keys, staged in LDS for the
// four waves.  Both products are v_mfma_f32_32x32x16_bf16 with the QUERIES as
// the 32 columns of the result:
//   S^T [32 keys x 32 queries]  = K tile [32 x 256]   x Q^T [256 x 32]
//   O^T [256 x 32 queries]     += V^T tile [256 x 32] x P^T [32 keys x 32]
// so a lane (query l % 32, half l / 32) holds, of every result, one query's
// values: the softmax statistics of a query are per-lane scalars (one exchange
// between the two halves per tile), the 16 scores a lane holds become, as they
// lie, its operand of the second product, and rescaling O is a multiplication
// by a per-lane scalar.  Which keys sit in which contraction slot of the second
// product is free as long as both operands agree: the S^T result gives half h
// of a lane the keys 8 j + 4 h + i (j = 0..3, i = 0..3), so the values are laid
// out in LDS in that order.  The values arrive transposed ([row, 256, T]: the
// caller's one extra pass over them), which makes the contraction index the
// contiguous one of both operands of both products.
#include <utility>

#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr int kAttnHd = 256;
constexpr int kAttnQ = 128;  // queries per workgroup
constexpr int kAttnK = 64;   // keys per tile
constexpr int kAttnKB = kAttnK / 32;  // blocks of 32 keys (one S^T result each)
constexpr int kAttnChunks = kAttnK * 32 / 256;  // 16-byte chunks per thread, tile and tensor
// K tile rows (one key, 512 B) padded to 528 B, V^T tile rows (one of the 256
// dimensions, 64 keys = 128 B) to 144 B: the 16-byte operand reads of 16
// consecutive rows fall on distinct banks.
constexpr int kKRowBytes = 528;
constexpr int kVRowBytes = 2 * kAttnK + 16;
constexpr int kKTileBytes = kAttnK * kKRowBytes;
constexpr int kVTileBytes = kAttnHd * kVRowBytes;

union AFrag {
  bf16x8 v;
  f32x4 q;
  uint32_t u[4];
};

// The 128 output accumulators of a lane (O^T: 8 blocks of 32 dimensions, 16
// registers each) live in the accumulation registers a[0:127] for the whole
// kernel, written and read by inline assembly with the register numbers
// spelled out: the second product accumulates into them tile after tile, and
// nothing else touches them but the rare rescaling and the final store (left
// to the register allocator they were moved between the two register files
// every tile, 256 moves for 32 matrix instructions).  The build checks that
// the compiler allocates no accumulation register of its own in this file.
#define RG_ATTN_LAST_AGPR "a127"

template <int N>
__device__ __forceinline__ float acc_read() {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, a[%c1]" : "=v"(t) : "n"(N));
  return t;
}
template <int N>
__device__ __forceinline__ void acc_write(float t) {
  asm volatile("v_accvgpr_write_b32 a[%c1], %0" ::"v"(t), "n"(N)
               : RG_ATTN_LAST_AGPR);
}
template <int... I>
__device__ __forceinline__ void acc_fill(float v,
                                         std::integer_sequence<int, I...>) {
  (acc_write<I>(v), ...);
}
template <int... I>
__device__ __forceinline__ void acc_scale(float f,
                                          std::integer_sequence<int, I...>) {
  (acc_write<I>(acc_read<I>() * f), ...);
}
// block BLK of O^T += a x b
template <int BLK>
__device__ __forceinline__ void acc_mfma(const f32x4& a, const f32x4& b) {
  asm volatile(
      "v_mfma_f32_32x32x16_bf16 a[%c2:%c2+15], %0, %1, a[%c2:%c2+15]" ::"v"(a),
      "v"(b), "n"(16 * BLK)
      : RG_ATTN_LAST_AGPR);
}
// The compiler does not count the wait states between a matrix instruction in
// inline assembly and a read of its result.
__device__ __forceinline__ void wait_for_matrix_results() {
  asm volatile("s_nop 15\n\ts_nop 7");
}

__global__ void __launch_bounds__(256)
attn_prefill_bf16_kernel(AttnPrefillArgs p) {
  extern __shared__ __align__(16) unsigned char attn_lds[];
  unsigned char* const k_tile = attn_lds;                    // two buffers
  unsigned char* const v_tile = attn_lds + 2 * kKTileBytes;  // two buffers

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 31, half = lane >> 5;
  const int qtiles = (p.T + kAttnQ - 1) / kAttnQ;
  // Workgroups go to the eight XCDs in turn (linear id modulo 8), each with an
  // L2 of its own: the ids are dealt out so that one XCD gets a contiguous run
  // of (row, head, query tile) triples, i.e. a row's keys and values are
  // pulled through one L2 instead of all eight.
  unsigned id = blockIdx.x;
  {
    const unsigned per_xcd = gridDim.x / 8;
    if (id < 8 * per_xcd) id = (id & 7) * per_xcd + (id >> 3);
  }
  // the longest workgroups (last query tiles) first
  const int qt = qtiles - 1 - (int)(id % qtiles);
  const int head = (int)(id / qtiles) % p.H;
  const int b = (int)(id / qtiles) / p.H;
  const int T = p.T;
  const int q0 = qt * kAttnQ;
  const int qw0 = q0 + 32 * wave;  // this wave's first query
  const int q = qw0 + n;           // this lane's query

  // descriptors over this row's tensors
  const uint32_t q_row_bytes = (uint32_t)p.H * kAttnHd * 2u;
  const __amdgpu_buffer_rsrc_t rq =
      make_rsrc((const char*)p.q + (int64_t)b * T * q_row_bytes,
                (uint32_t)T * q_row_bytes);
  const __amdgpu_buffer_rsrc_t ro = make_rsrc(
      (char*)p.out + (int64_t)b * T * q_row_bytes, (uint32_t)T * q_row_bytes);
  const __amdgpu_buffer_rsrc_t rk =
      make_rsrc((const char*)p.k + (int64_t)b * T * (kAttnHd * 2),
                (uint32_t)T * (kAttnHd * 2u));
  const uint32_t vt_row_bytes = (uint32_t)p.T_pad * 2u;
  const __amdgpu_buffer_rsrc_t rv =
      make_rsrc((const char*)p.v_t + (int64_t)b * kAttnHd * vt_row_bytes,
                (uint32_t)kAttnHd * vt_row_bytes);
  const __amdgpu_buffer_rsrc_t rlo = make_rsrc(
      (const char*)p.lo + (int64_t)b * T * 4, (uint32_t)T * 4u);

  // this lane's query as the B operand of the first product: 16 k-steps of
  // 8 dimensions (16 bytes); queries past the end read as zero
  AFrag qf[16];
  {
    const uint32_t off = (uint32_t)q * q_row_bytes + (uint32_t)head * 512u +
                         16u * (uint32_t)half;
#pragma unroll
    for (int ks = 0; ks < 16; ++ks)
      qf[ks].q = __builtin_bit_cast(
          f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                     rq, q < T ? off + 32u * ks : kBufferOutOfRange, 0, 0));
  }
  // first visible key of this lane's query, and of the tile's / wave's first
  // query (lo is non-decreasing: they bound the keys the tile / wave needs)
  auto lo_at = [&](int t) {
    return (int)__builtin_amdgcn_raw_buffer_load_b32(
        rlo, t < T ? (uint32_t)t * 4u : kBufferOutOfRange, 0, 0);
  };
  const int lo_q = q < T ? lo_at(q) : 0x7fffffff;
  const int lo_tile = __builtin_amdgcn_readfirstlane(lo_at(q0));
  const int lo_wave =
      __builtin_amdgcn_readfirstlane(qw0 < T ? lo_at(qw0) : 0x7fffffff);
  const int q_last_tile = q0 + kAttnQ - 1 < T - 1 ? q0 + kAttnQ - 1 : T - 1;
  const int q_last_wave = qw0 + 31 < T - 1 ? qw0 + 31 : T - 1;
  const int kt_begin = lo_tile / kAttnK;
  const int kt_end = q_last_tile / kAttnK;  // inclusive

  acc_fill(0.0f, std::make_integer_sequence<int, 128>{});
  float m_run = -__builtin_inff();  // running maximum, in units of log2
  float l_run = 0.0f;               // running sum over this half's keys
  const float scale_log2 = p.scale * kLog2e;

  // staging: 16-byte chunks, kAttnChunks per thread, tile and tensor; the
  // chunks of tile kt + 1 are requested as soon as tile kt is in LDS and
  // arrive while it is worked on
  u32x4 kc[kAttnChunks], vc[kAttnChunks];
  auto request_tile = [&](int kt) {
    const int key0 = kt * kAttnK;
#pragma unroll
    for (int i = 0; i < kAttnChunks; ++i) {
      const int c = tid + 256 * i;
      const int krow = c >> 5, kcol = c & 31;
      const int key = key0 + krow;
      kc[i] = __builtin_amdgcn_raw_buffer_load_b128(
          rk, key < T ? (uint32_t)key * 512u + 16u * kcol : kBufferOutOfRange,
          0, 0);
      const int d = c / (kAttnK / 8), part = c % (kAttnK / 8);
      vc[i] = __builtin_amdgcn_raw_buffer_load_b128(
          rv, (uint32_t)d * vt_row_bytes + (uint32_t)(key0 + 8 * part) * 2u, 0,
          0);
    }
  };
  auto stage_tile = [&](int buf) {
    unsigned char* const kt_ = k_tile + buf * kKTileBytes;
    unsigned char* const vt_ = v_tile + buf * kVTileBytes;
#pragma unroll
    for (int i = 0; i < kAttnChunks; ++i) {
      const int c = tid + 256 * i;
      const int krow = c >> 5, kcol = c & 31;
      *reinterpret_cast<u32x4*>(kt_ + krow * kKRowBytes + 16 * kcol) = kc[i];
      const int d = c / (kAttnK / 8), part = c % (kAttnK / 8);
      // keys 8 part .. 8 part + 7 of the tile: group s = part / 2 of 16 keys,
      // stored as [keys 0-3, 8-11 | keys 4-7, 12-15] of the group
      unsigned char* const vb =
          vt_ + d * kVRowBytes + 32 * (part >> 1) + 8 * (part & 1);
      *reinterpret_cast<u32x2*>(vb) = u32x2{vc[i][0], vc[i][1]};
      *reinterpret_cast<u32x2*>(vb + 16) = u32x2{vc[i][2], vc[i][3]};
    }
  };
  // Two LDS buffers: while tile kt is worked on out of one, tile kt + 1
  // arrives in registers and is written to the other afterwards; one barrier
  // per tile.
  request_tile(kt_begin);
  stage_tile(0);
  __syncthreads();
  if (kt_begin < kt_end) request_tile(kt_begin + 1);
  // last query of this wave sees from lo_last_wave on (lo is non-decreasing)
  const int lo_last_wave = __builtin_amdgcn_readfirstlane(lo_at(q_last_wave));
  for (int kt = kt_begin; kt <= kt_end; ++kt) {
    const int key0 = kt * kAttnK;
    const int buf = (kt - kt_begin) & 1;
    const unsigned char* const kt_ = k_tile + buf * kKTileBytes;
    const unsigned char* const vt_ = v_tile + buf * kVTileBytes;

    // tiles outside what this wave's queries can see are skipped (wave-uniform)
    if (!(key0 > q_last_wave || key0 + kAttnK - 1 < lo_wave)) {
      // ---- S^T = K tile x Q^T ----------------------------------------------
      // (inline assembly with the results in ordinary registers: a matrix
      // builtin lets the compiler pick accumulation registers for the result,
      // and it picks a[0:15].  The compiler moves no LDS read across such a
      // statement, so the operands are requested by hand, four fragments
      // ahead of the instructions that use them.)
      f32x16 s[kAttnKB];
      {
        constexpr int kFrags = 16 * kAttnKB, kBatch = 4;
        auto k_frag = [&](int f) {  // fragment f: k-step f / KB, key block f % KB
          return *reinterpret_cast<const f32x4*>(
              kt_ + (32 * (f % kAttnKB) + n) * kKRowBytes + 32 * (f / kAttnKB) +
              16 * half);
        };
        f32x4 fr[2][kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) fr[0][i] = k_frag(i);
#pragma unroll
        for (int bt = 0; bt < kFrags / kBatch; ++bt) {
          if (bt + 1 < kFrags / kBatch) {
#pragma unroll
            for (int i = 0; i < kBatch; ++i)
              fr[(bt + 1) & 1][i] = k_frag((bt + 1) * kBatch + i);
          }
#pragma unroll
          for (int i = 0; i < kBatch; ++i) {
            const int f = bt * kBatch + i;
            const int ks = f / kAttnKB, kb = f % kAttnKB;
            if (ks == 0)
              asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0"
                           : "=&v"(s[kb])
                           : "v"(fr[bt & 1][i]), "v"(qf[ks].q));
            else
              asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0"
                           : "+v"(s[kb])
                           : "v"(fr[bt & 1][i]), "v"(qf[ks].q));
          }
        }
      }
      // (tied to the scores: nothing that reads them may be scheduled above
      // the wait)
#pragma unroll
      for (int kb = 0; kb < kAttnKB; ++kb) asm volatile("" : "+v"(s[kb]));
      wait_for_matrix_results();
#pragma unroll
      for (int kb = 0; kb < kAttnKB; ++kb) asm volatile("" : "+v"(s[kb]));
      // ---- mask (only where the band's edges cross the tile) ----------------
      const bool interior = key0 + kAttnK - 1 <= qw0 && key0 >= lo_last_wave;
      if (!interior) {
#pragma unroll
        for (int kb = 0; kb < kAttnKB; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = key0 + 32 * kb + 8 * (r >> 2) + 4 * half + (r & 3);
            s[kb][r] = (key >= lo_q && key <= q) ? s[kb][r] : -__builtin_inff();
          }
      }
      // ---- running maximum (in units of log2), moved only when the tile's
      //      exceeds it by more than 2^8: the accumulators are rescaled rarely --
      float tile_max = s[0][0];
#pragma unroll
      for (int kb = 0; kb < kAttnKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) tile_max = fmaxf(tile_max, s[kb][r]);
      {
        const auto sw = __builtin_amdgcn_permlane32_swap(
            __float_as_uint(tile_max), __float_as_uint(tile_max), false, false);
        tile_max = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
      }
      tile_max *= scale_log2;  // (the scale is positive)
      if (__ballot(tile_max > m_run + 8.0f) != 0) {
        const float m_new = fmaxf(m_run, tile_max);
        // (no visible key so far: keep every exponent finite)
        const float alpha = __builtin_amdgcn_exp2f(
            m_run - (m_new == -__builtin_inff() ? 0.0f : m_new));
        m_run = m_new;
        l_run *= alpha;
        wait_for_matrix_results();
        acc_scale(alpha, std::make_integer_sequence<int, 128>{});
      }
      const float m_sub = m_run == -__builtin_inff() ? 0.0f : m_run;
      AFrag pf[2 * kAttnKB];
#pragma unroll
      for (int kb = 0; kb < kAttnKB; ++kb)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const float p0 = __builtin_amdgcn_exp2f(
              __builtin_fmaf(s[kb][r], scale_log2, -m_sub));
          const float p1 = __builtin_amdgcn_exp2f(
              __builtin_fmaf(s[kb][r + 1], scale_log2, -m_sub));
          l_run += p0 + p1;
          pf[2 * kb + (r >> 3)].u[(r & 7) >> 1] = pack_bf16x2(p0, p1);
        }
      // ---- O^T += V^T tile x P^T: the eight blocks of a 16-key step one after
      //      the other (independent accumulators), the operands of the next
      //      step requested before ------------------------------------------------
      {
        auto v_frag = [&](int ss, int blk) {
          return *reinterpret_cast<const f32x4*>(
              vt_ + (32 * blk + n) * kVRowBytes + 32 * ss + 16 * half);
        };
        // batch bt: 16-key step bt / 2, blocks 4 (bt % 2) .. + 3
        f32x4 fr[2][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) fr[0][i] = v_frag(0, i);
#pragma unroll
        for (int bt = 0; bt < 4 * kAttnKB; ++bt) {
          if (bt + 1 < 4 * kAttnKB) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              fr[(bt + 1) & 1][i] = v_frag((bt + 1) >> 1, 4 * ((bt + 1) & 1) + i);
          }
          const f32x4& pq = pf[bt >> 1].q;
          if (bt & 1) {
            acc_mfma<4>(fr[bt & 1][0], pq);
            acc_mfma<5>(fr[bt & 1][1], pq);
            acc_mfma<6>(fr[bt & 1][2], pq);
            acc_mfma<7>(fr[bt & 1][3], pq);
          } else {
            acc_mfma<0>(fr[bt & 1][0], pq);
            acc_mfma<1>(fr[bt & 1][1], pq);
            acc_mfma<2>(fr[bt & 1][2], pq);
            acc_mfma<3>(fr[bt & 1][3], pq);
          }
        }
      }
    }
    if (kt < kt_end) {
      stage_tile(buf ^ 1);  // tile kt + 1; that buffer's readers passed the
      __syncthreads();      // barrier of the previous round
      if (kt + 1 < kt_end) request_tile(kt + 2);
    }
  }

  // ---- normalise and store: this lane's query, dimensions
  //      32 blk + 8 j + 4 half + i ---------------------------------------------
  wait_for_matrix_results();
  float l_total;
  {
    const auto sw = __builtin_amdgcn_permlane32_swap(
        __float_as_uint(l_run), __float_as_uint(l_run), false, false);
    l_total = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  const float inv = l_total > 0.0f ? 1.0f / l_total : 0.0f;
  const uint32_t out_off = (uint32_t)q * q_row_bytes + (uint32_t)head * 512u;
  auto store4 = [&](int d0, float o0, float o1, float o2, float o3) {
    __builtin_amdgcn_raw_buffer_store_b64(
        u32x2{pack_bf16x2(o0 * inv, o1 * inv), pack_bf16x2(o2 * inv, o3 * inv)},
        ro, q < T ? out_off + (uint32_t)(d0 + 4 * half) * 2u : kBufferOutOfRange,
        0, 0);
  };
#define RG_ATTN_STORE(BLK, J)                                              \
  store4(32 * BLK + 8 * J, acc_read<16 * BLK + 4 * J>(),                   \
         acc_read<16 * BLK + 4 * J + 1>(), acc_read<16 * BLK + 4 * J + 2>(), \
         acc_read<16 * BLK + 4 * J + 3>());
#define RG_ATTN_STORE_BLK(BLK) \
  RG_ATTN_STORE(BLK, 0) RG_ATTN_STORE(BLK, 1) RG_ATTN_STORE(BLK, 2) RG_ATTN_STORE(BLK, 3)
  RG_ATTN_STORE_BLK(0) RG_ATTN_STORE_BLK(1) RG_ATTN_STORE_BLK(2) RG_ATTN_STORE_BLK(3)
  RG_ATTN_STORE_BLK(4) RG_ATTN_STORE_BLK(5) RG_ATTN_STORE_BLK(6) RG_ATTN_STORE_BLK(7)
#undef RG_ATTN_STORE_BLK
#undef RG_ATTN_STORE
}

}  // namespace

hipError_t launch_attn_prefill_bf16(const AttnPrefillArgs& a, hipStream_t s) {
  // needs head dimension 256, T_pad a multiple of 64 >= T, and rows whose byte
  // offsets fit 32 bits (checked by the caller)
  const int64_t qtiles = (a.T + kAttnQ - 1) / kAttnQ;
  const int64_t blocks = qtiles * a.H * a.B;
  if (blocks <= 0 || blocks > 0x7fffffff) return hipErrorInvalidValue;
  constexpr size_t lds = 2 * (size_t)(kKTileBytes + kVTileBytes);
  static_assert(lds <= 160 * 1024, "LDS of one CU");
  static OncePerDevice once;
  hipError_t e =
      set_max_dynamic_lds(once, (const void*)attn_prefill_bf16_kernel, lds);
  if (e != hipSuccess) return e;
  attn_prefill_bf16_kernel<<<dim3((unsigned)blocks), 256, lds, s>>>(a);
  return hipGetLastError();
}

}  // namespace rg
