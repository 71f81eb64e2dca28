// Shared device helpers for the gfx950 Conv1D + RG-LRU kernels.
#ifndef RG_COMMON_H_
#define RG_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rg {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// ---------------------------------------------------------------- bf16 ----
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}
// Round-to-nearest-even float -> bf16 (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 v = {lo, hi};
  bf16x2 p = __builtin_convertvector(v, bf16x2);
  return *reinterpret_cast<uint32_t*>(&p);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
  return (uint16_t)(pack_bf16x2(v, 0.0f) & 0xffffu);
}
__device__ __forceinline__ float round_to_bf16(float v) {
  return bf16_bits_to_f32(f32_to_bf16_bits(v));
}

// ------------------------------------------------------- element traits ----
// Act<T>: how CH adjacent channels of an activation tensor are read into
// floats and written back.  T is float or uint16_t (bf16 bit pattern).
template <typename T, int CH>
struct Act;

template <>
struct Act<float, 1> {
  static constexpr bool kIsBf16 = false;
  typedef float Raw;
  __device__ static Raw load_raw(const float* p) { return *p; }
  __device__ static void unpack(Raw r, float (&v)[1]) { v[0] = r; }
  __device__ static void load(const float* p, float (&v)[1]) { v[0] = *p; }
  __device__ static void store(float* p, const float (&v)[1]) { *p = v[0]; }
  __device__ static float round(float v) { return v; }
};
template <>
struct Act<float, 2> {
  static constexpr bool kIsBf16 = false;
  typedef f32x2 Raw;
  __device__ static Raw load_raw(const float* p) {
    return *reinterpret_cast<const f32x2*>(p);
  }
  __device__ static void unpack(Raw r, float (&v)[2]) {
    v[0] = r.x;
    v[1] = r.y;
  }
  __device__ static void load(const float* p, float (&v)[2]) {
    f32x2 t = *reinterpret_cast<const f32x2*>(p);
    v[0] = t.x;
    v[1] = t.y;
  }
  __device__ static void store(float* p, const float (&v)[2]) {
    f32x2 t = {v[0], v[1]};
    *reinterpret_cast<f32x2*>(p) = t;
  }
  __device__ static float round(float v) { return v; }
};
template <>
struct Act<uint16_t, 1> {
  static constexpr bool kIsBf16 = true;
  typedef uint16_t Raw;
  __device__ static Raw load_raw(const uint16_t* p) { return *p; }
  __device__ static void unpack(Raw r, float (&v)[1]) {
    v[0] = bf16_bits_to_f32(r);
  }
  __device__ static void load(const uint16_t* p, float (&v)[1]) {
    v[0] = bf16_bits_to_f32(*p);
  }
  __device__ static void store(uint16_t* p, const float (&v)[1]) {
    *p = f32_to_bf16_bits(v[0]);
  }
  __device__ static float round(float v) { return round_to_bf16(v); }
};
template <>
struct Act<uint16_t, 2> {
  static constexpr bool kIsBf16 = true;
  typedef uint32_t Raw;  // two bf16 stay packed in one register until used
  __device__ static Raw load_raw(const uint16_t* p) {
    return *reinterpret_cast<const uint32_t*>(p);
  }
  __device__ static void unpack(Raw r, float (&v)[2]) {
    v[0] = __uint_as_float(r << 16);
    v[1] = __uint_as_float(r & 0xffff0000u);
  }
  __device__ static void load(const uint16_t* p, float (&v)[2]) {
    uint32_t u = *reinterpret_cast<const uint32_t*>(p);
    v[0] = __uint_as_float(u << 16);
    v[1] = __uint_as_float(u & 0xffff0000u);
  }
  __device__ static void store(uint16_t* p, const float (&v)[2]) {
    *reinterpret_cast<uint32_t*>(p) = pack_bf16x2(v[0], v[1]);
  }
  __device__ static float round(float v) { return round_to_bf16(v); }
};

template <typename T>
__device__ __forceinline__ float load_scalar(const T* p);
template <>
__device__ __forceinline__ float load_scalar<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float load_scalar<uint16_t>(const uint16_t* p) {
  return bf16_bits_to_f32(*p);
}
template <typename T>
__device__ __forceinline__ void store_scalar(T* p, float v);
template <>
__device__ __forceinline__ void store_scalar<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ __forceinline__ void store_scalar<uint16_t>(uint16_t* p, float v) {
  *p = f32_to_bf16_bits(v);
}
template <typename T>
__device__ __forceinline__ float round_act(float v);
template <>
__device__ __forceinline__ float round_act<float>(float v) {
  return v;
}
template <>
__device__ __forceinline__ float round_act<uint16_t>(float v) {
  return round_to_bf16(v);
}

// ------------------------------------------------------ segment_pos ----
// How document starts are encoded: int32 / int64 positions (start == 0), or a
// byte mask (start != 0) as rnn_scan's `reset` argument.
enum SegKind { kSegI32 = 0, kSegI64 = 1, kSegMaskU8 = 2 };

__device__ __forceinline__ bool is_doc_start(const void* segpos, int kind,
                                             int64_t idx) {
  if (kind == kSegI64) return reinterpret_cast<const int64_t*>(segpos)[idx] == 0;
  if (kind == kSegMaskU8) return reinterpret_cast<const uint8_t*>(segpos)[idx] != 0;
  return reinterpret_cast<const int32_t*>(segpos)[idx] == 0;
}

// ------------------------------------------------------------- conv ----
// Width-4 tap chain of the float32 kernels, in one fixed order: newest tap
// first, bias as the starting value, fused multiply-adds.
// x0 = x[t], x1 = x[t-1], ... ; w3 multiplies x[t] (layers.py:514).
__device__ __forceinline__ float conv4(float x0, float x1, float x2, float x3,
                                       float w0, float w1, float w2, float w3,
                                       float bias) {
  float acc = __builtin_fmaf(x0, w3, bias);
  acc = __builtin_fmaf(x1, w2, acc);
  acc = __builtin_fmaf(x2, w1, acc);
  acc = __builtin_fmaf(x3, w0, acc);
  return acc;
}

// The bf16 kernels' width-4 conv, one arithmetic everywhere (gate GEMM with
// the conv on load, scan kernel, single prefill kernel, stand-alone conv,
// decode step), so that all of them see bit-identical conv outputs: per
// channel the rows are paired in time, P_t = (x[t-1], x[t]) as two bf16 in one
// register, the taps as w10 = (w0, w1) and w32 = (w2, w3), and
//   out[t] = (bias + P_{t-2} . w10) + P_t . w32
// is two v_dot2_f32_bf16 (float32 products and sums), rounded to bf16 by the
// caller.  Nothing is unpacked: 3.5 vector instructions per output where the
// chain of fused multiply-adds on floats takes 5.75.
constexpr uint32_t kPairSelLo = 0x05040100u;  // (lo16(earlier), lo16(later))
constexpr uint32_t kPairSelHi = 0x07060302u;  // (hi16(earlier), hi16(later))
// Two rows of a channel pair (two bf16 per register) -> the time pairs of the
// low and the high channel.
__device__ __forceinline__ void pair_up(uint32_t earlier, uint32_t later,
                                        uint32_t& lo, uint32_t& hi) {
  lo = __builtin_amdgcn_perm(later, earlier, kPairSelLo);
  hi = __builtin_amdgcn_perm(later, earlier, kPairSelHi);
}
// The result of a dot instruction may be read by an instruction of another
// kind only three issue slots later, and the compiler does not count them for
// inline assembly: each group ends with the wait itself.
__device__ __forceinline__ float conv4_dot(uint32_t p_old, uint32_t p_new,
                                           uint32_t w10, uint32_t w32,
                                           float bias) {
  float out;
  asm("v_dot2_f32_bf16 %0, %1, %3, %5\n\t"
      "v_dot2_f32_bf16 %0, %2, %4, %0\n\t"
      "s_nop 2"
      : "=&v"(out)
      : "v"(p_old), "v"(p_new), "v"(w10), "v"(w32), "v"(bias));
  return out;
}
__device__ __forceinline__ void conv4_dot_x2(
    const uint32_t (&p_old)[2], const uint32_t (&p_new)[2],
    const uint32_t (&w10)[2], const uint32_t (&w32)[2], const float (&bias)[2],
    float (&out)[2]) {
  asm("v_dot2_f32_bf16 %0, %2, %6, %10\n\t"
      "v_dot2_f32_bf16 %1, %3, %7, %11\n\t"
      "v_dot2_f32_bf16 %0, %4, %8, %0\n\t"
      "v_dot2_f32_bf16 %1, %5, %9, %1\n\t"
      "s_nop 2"
      : "=&v"(out[0]), "=&v"(out[1])
      : "v"(p_old[0]), "v"(p_old[1]), "v"(p_new[0]), "v"(p_new[1]),
        "v"(w10[0]), "v"(w10[1]), "v"(w32[0]), "v"(w32[1]), "v"(bias[0]),
        "v"(bias[1]));
}
__device__ __forceinline__ void conv4_dot_x4(
    const uint32_t (&p_old)[4], const uint32_t (&p_new)[4],
    const uint32_t (&w10)[4], const uint32_t (&w32)[4], const float (&bias)[4],
    float (&out)[4]) {
  asm("v_dot2_f32_bf16 %0, %4, %12, %20\n\t"
      "v_dot2_f32_bf16 %1, %5, %13, %21\n\t"
      "v_dot2_f32_bf16 %2, %6, %14, %22\n\t"
      "v_dot2_f32_bf16 %3, %7, %15, %23\n\t"
      "v_dot2_f32_bf16 %0, %8, %16, %0\n\t"
      "v_dot2_f32_bf16 %1, %9, %17, %1\n\t"
      "v_dot2_f32_bf16 %2, %10, %18, %2\n\t"
      "v_dot2_f32_bf16 %3, %11, %19, %3\n\t"
      "s_nop 2"
      : "=&v"(out[0]), "=&v"(out[1]), "=&v"(out[2]), "=&v"(out[3])
      : "v"(p_old[0]), "v"(p_old[1]), "v"(p_old[2]), "v"(p_old[3]),
        "v"(p_new[0]), "v"(p_new[1]), "v"(p_new[2]), "v"(p_new[3]),
        "v"(w10[0]), "v"(w10[1]), "v"(w10[2]), "v"(w10[3]), "v"(w32[0]),
        "v"(w32[1]), "v"(w32[2]), "v"(w32[3]), "v"(bias[0]), "v"(bias[1]),
        "v"(bias[2]), "v"(bias[3]));
}
// The same output from bf16 values held as floats (the element-per-thread
// kernels): packing them back is exact.  x0 = x[t], x1 = x[t-1], ...
__device__ __forceinline__ float conv4_bf16(float x0, float x1, float x2,
                                            float x3, float w0, float w1,
                                            float w2, float w3, float bias) {
  return conv4_dot(pack_bf16x2(x3, x2), pack_bf16x2(x1, x0),
                   pack_bf16x2(w0, w1), pack_bf16x2(w2, w3), bias);
}
// conv4 for the element type: float32 the multiply-add chain, bf16 the dots.
template <typename T>
__device__ __forceinline__ float conv4_as(float x0, float x1, float x2,
                                          float x3, float w0, float w1,
                                          float w2, float w3, float bias) {
  if (sizeof(T) == 2) return conv4_bf16(x0, x1, x2, x3, w0, w1, w2, w3, bias);
  return conv4(x0, x1, x2, x3, w0, w1, w2, w3, bias);
}

// Generic-width conv output at flattened row m = b*T + t, channel c, straight
// from the definition (same accumulation order as conv4 for K == 4).
template <typename T>
__device__ __forceinline__ float conv_point(const T* x, const void* segpos,
                                            int seg_kind, const T* w,
                                            const T* bias, int T_len, int W,
                                            int K, int64_t m, int c) {
  int t = (int)(m % T_len);
  if (sizeof(T) == 2 && K == 4) {
    // the bf16 kernels' width-4 arithmetic (conv4_dot)
    float xs[4];
    bool alive = true;
    for (int s = 0; s < 4; ++s) {
      if (s > t) alive = false;
      if (s > 0 && s <= t && is_doc_start(segpos, seg_kind, m - s + 1))
        alive = false;
      xs[s] = alive ? load_scalar(x + (m - s) * W + c) : 0.0f;
    }
    return round_act<T>(conv4_bf16(
        xs[0], xs[1], xs[2], xs[3], load_scalar(w + c),
        load_scalar(w + (int64_t)W + c), load_scalar(w + 2 * (int64_t)W + c),
        load_scalar(w + 3 * (int64_t)W + c), load_scalar(bias + c)));
  }
  float acc = load_scalar(bias + c);
  bool alive = true;
  for (int s = 0; s < K && s <= t; ++s) {
    if (s > 0 && is_doc_start(segpos, seg_kind, m - s + 1)) alive = false;
    float v = alive ? load_scalar(x + (m - s) * W + c) : 0.0f;
    acc = __builtin_fmaf(v, load_scalar(w + (int64_t)(K - 1 - s) * W + c), acc);
  }
  return round_act<T>(acc);
}

// Raw buffer descriptor (stride 0, 32-bit data format) over `bytes` bytes at
// `base`.  Accesses whose offset (vector + scalar part) falls outside are
// dropped (stores) or return zero (loads).
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base,
                                                            uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0,
                                           (int)bytes, 0x00020000);
}
constexpr uint32_t kBufferOutOfRange = 0x80000000u;

// 16-byte buffer store at byte offset lane_off + uniform_off.  The whole offset
// goes into the vector offset and the scalar offset stays the constant 0: for
// a store of more than 8 bytes whose scalar offset is a register the compiler
// does not keep the next vector instruction from overwriting the data
// registers, and on gfx950 such an overwrite right after the store was seen to
// reach memory (third dword of the 16 bytes, last lanes of each 16).  With a
// constant scalar offset the compiler spaces the two instructions itself.
__device__ __forceinline__ void buffer_store_16(u32x4 v,
                                                __amdgpu_buffer_rsrc_t r,
                                                uint32_t lane_off,
                                                uint32_t uniform_off) {
  __builtin_amdgcn_raw_buffer_store_b128(v, r, lane_off + uniform_off, 0, 0);
}

// ---------------------------------------------------------- barriers ----
// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits
// for every outstanding global load and store of the wave (its fence covers
// global memory), which would drain loads that were issued early on purpose.
// Use only where the waves exchange data through LDS and nothing else.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ------------------------------------------------------------- math ----
constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float softplus_precise(float v) {
  return v > 20.0f ? v : log1pf(expf(v));
}
__device__ __forceinline__ float sigmoid_precise(float v) {
  return 1.0f / (1.0f + expf(-v));
}
// Hardware exp2/rcp (about 1 ulp each): used on the bf16 path.
__device__ __forceinline__ float sigmoid_fast(float v) {
  float e = __builtin_amdgcn_exp2f(-kLog2e * v);
  return __builtin_amdgcn_rcpf(1.0f + e);
}


// a * gelu_tanh(g) for bf16 operands held as floats (modules.py:289-291, :644):
// gelu in fp32 as 0.5 g (1 + tanh u) with tanh u = 2 sigmoid(2u) - 1 rounded
// to float32 first, so that the negative tail saturates to -0 exactly where a
// float32 tanh does; gelu is rounded to bf16 like the module output it is in
// the reference; the caller rounds the product.
__device__ __forceinline__ float gelu_mul_bf16(float av, float gv) {
  constexpr float c0 = 0.7978845608028654f;  // sqrt(2/pi)
  constexpr float c1 = 0.044715f;
  const float u = c0 * __builtin_fmaf(c1 * gv * gv, gv, gv);
  const float t = __builtin_fmaf(2.0f, sigmoid_fast(2.0f * u), -1.0f);
  return av * round_to_bf16(0.5f * gv * (1.0f + t));
}

// a * gelu_tanh(g) in float32 by the reference's own formula
// (modules.py:289-291, :644), every step rounded as written (no fused
// multiply-adds), so that every kernel that has it gives the same bits.
__device__ __forceinline__ float gelu_mul_f32(float av, float gv) {
  constexpr float c0 = 0.7978845608028654f;  // sqrt(2/pi)
  constexpr float c1 = 0.044715f;
  const float cube = __fmul_rn(__fmul_rn(__fmul_rn(c1, gv), gv), gv);
  const float u = __fmul_rn(c0, __fadd_rn(gv, cube));
  const float gelu =
      __fmul_rn(__fmul_rn(0.5f, gv), __fadd_rn(1.0f, tanhf(u)));
  return __fmul_rn(av, gelu);
}

}  // namespace rg
#endif  // RG_COMMON_H_
