// out = a * gelu_tanh(g): the join of the two branches of the recurrent block
// (recurrentgemma/torch/modules.py:627-628 `y = gelu(linear_y(x))`, :289-291
// the tanh approximation, :644 `x = x * y`), one pass instead of torch's gelu
// pass plus multiply pass.  `a` is the RG-LRU output, `g` the linear_y output.
#include "rg_common.h"
#include "rg_internal.h"

namespace rg {
namespace {

constexpr float kGeluC0 = 0.7978845608028654f;  // sqrt(2/pi)
constexpr float kGeluC1 = 0.044715f;

// bf16: gelu in fp32 as 0.5 v (1 + tanh u) with tanh u = 2 sigmoid(2u) - 1
// rounded to float32 first, so that the negative tail saturates to -0 exactly
// where a float32 tanh does; gelu is rounded to bf16 like the module output it
// is in the reference, then the product is rounded once.  Eight elements (16 bytes) per thread and iteration.
__global__ void __launch_bounds__(256)
gelu_mul_bf16_kernel(const u32x4* __restrict__ a, const u32x4* __restrict__ g,
                     u32x4* __restrict__ out, int64_t n8,
                     const uint16_t* a_tail, const uint16_t* g_tail,
                     uint16_t* out_tail, int tail) {
  auto one = [](float av, float gv) {
    const float u = kGeluC0 * __builtin_fmaf(kGeluC1 * gv * gv, gv, gv);
    const float t = __builtin_fmaf(2.0f, sigmoid_fast(2.0f * u), -1.0f);
    const float y = round_to_bf16(0.5f * gv * (1.0f + t));
    return av * y;
  };
  auto eight = [&](u32x4 av, u32x4 gv) {
    u32x4 o;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float lo = one(__uint_as_float(av[k] << 16),
                           __uint_as_float(gv[k] << 16));
      const float hi = one(__uint_as_float(av[k] & 0xffff0000u),
                           __uint_as_float(gv[k] & 0xffff0000u));
      o[k] = pack_bf16x2(lo, hi);
    }
    return o;
  };
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // four independent 16-byte loads of each operand in flight per thread
  for (; i + 3 * stride < n8; i += 4 * stride) {
    u32x4 av[4], gv[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      av[k] = __builtin_nontemporal_load(a + i + k * stride);
      gv[k] = __builtin_nontemporal_load(g + i + k * stride);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      __builtin_nontemporal_store(eight(av[k], gv[k]), out + i + k * stride);
  }
  for (; i < n8; i += stride) out[i] = eight(a[i], g[i]);
  if (blockIdx.x == 0 && (int)threadIdx.x < tail)
    out_tail[threadIdx.x] = f32_to_bf16_bits(
        one(bf16_bits_to_f32(a_tail[threadIdx.x]),
            bf16_bits_to_f32(g_tail[threadIdx.x])));
}

__global__ void __launch_bounds__(256)
gelu_mul_f32_kernel(const float* __restrict__ a, const float* __restrict__ g,
                    float* __restrict__ out, int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    const float gv = g[i];
    const float u = kGeluC0 * (gv + kGeluC1 * gv * gv * gv);
    out[i] = a[i] * (0.5f * gv * (1.0f + tanhf(u)));
  }
}

}  // namespace

hipError_t launch_gelu_mul(const void* a, const void* g, void* out, int64_t n,
                           int dtype, hipStream_t s) {
  const int64_t cap = 256 * 32;  // grid-stride loop beyond this
  if (dtype == 0) {
    int64_t blocks = (n + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > cap ? cap : blocks);
    gelu_mul_f32_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const float*)a, (const float*)g, (float*)out, n);
  } else {
    const int64_t n8 = n / 8;
    const int tail = (int)(n - n8 * 8);
    int64_t blocks = (n8 + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > cap ? cap : blocks);
    gelu_mul_bf16_kernel<<<dim3((unsigned)blocks), 256, 0, s>>>(
        (const u32x4*)a, (const u32x4*)g, (u32x4*)out, n8,
        (const uint16_t*)a + n8 * 8, (const uint16_t*)g + n8 * 8,
        (uint16_t*)out + n8 * 8, tail);
  }
  return hipGetLastError();
}

}  // namespace rg
