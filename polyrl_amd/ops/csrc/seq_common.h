// Shared helpers of the sequence-mixer kernels (seq_*.hip): activation-type
// generic loads/stores (bf16 or fp32 activations, fp32 math) and accurate
// fp32 transcendental wrappers.  gfx950 only, wave size 64.
#pragma once

#include "common.h"

template <typename T>
DEV_INLINE float ldf(const T* p);
template <>
DEV_INLINE float ldf<float>(const float* p) { return *p; }
template <>
DEV_INLINE float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }

template <typename T>
DEV_INLINE void stf(T* p, float v);
template <>
DEV_INLINE void stf<float>(float* p, float v) { *p = v; }
template <>
DEV_INLINE void stf<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

DEV_INLINE float sigmoidf_acc(float x) { return 1.f / (1.f + expf(-x)); }
DEV_INLINE float siluf_acc(float x) { return x / (1.f + expf(-x)); }
DEV_INLINE float softplusf_acc(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}
DEV_INLINE float gelu_tanhf_acc(float z) {
  const float c = 0.7978845608028654f;  // sqrt(2/pi)
  return 0.5f * z * (1.f + tanhf(c * (z + 0.044715f * z * z * z)));
}

DEV_INLINE float gelu_erff_acc(float z) {
  return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
}

// sum over the 2^k lanes l, l^1, ..., l^(G-1) (G a power of two <= 64)
template <int G>
DEV_INLINE float lanegroup_sum(float x) {
#pragma unroll
  for (int off = G / 2; off > 0; off >>= 1) x += __shfl_xor(x, off, WAVE_SIZE);
  return x;
}

// activation-type dispatch on a torch dtype
#define SEQ_DISPATCH_T(dtype, ...)                                   \
  do {                                                               \
    if ((dtype) == torch::kBFloat16) {                               \
      using T = bf16_t;                                              \
      __VA_ARGS__;                                                   \
    } else if ((dtype) == torch::kFloat32) {                         \
      using T = float;                                               \
      __VA_ARGS__;                                                   \
    } else {                                                         \
      TORCH_CHECK(false, "activations must be bf16 or fp32");        \
    }                                                                \
  } while (0)

#define CHECK_I32(t) TORCH_CHECK((t).is_cuda() && (t).dtype() == torch::kInt32 && (t).is_contiguous(), #t " must be a contiguous int32 device tensor")
#define CHECK_F32(t) TORCH_CHECK((t).is_cuda() && (t).dtype() == torch::kFloat32 && (t).is_contiguous(), #t " must be a contiguous fp32 device tensor")
#define CHECK_ROWS(t) TORCH_CHECK((t).is_cuda() && (t).dim() == 2 && (t).stride(1) == 1, #t " must be 2-D with unit inner stride")
