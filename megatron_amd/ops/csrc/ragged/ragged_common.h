// Shared helpers of the ragged-batch sequence kernels (gfx950, wave64).
//
// Storage may be bf16 or fp32 (template parameter); all arithmetic is fp32
// and results are rounded once, on store.
#pragma once

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "../common.h"

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16>(const bf16* p) { return __bfloat162float(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16>(bf16* p, float v) { *p = __float2bfloat16(v); }

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + expf(-x)); }
// log(1 + e^x), stable for both signs
__device__ __forceinline__ float softplusf_(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

#define RAGGED_DISPATCH(TENSOR, ...)                                              \
  do {                                                                            \
    if ((TENSOR).scalar_type() == at::kFloat) {                                   \
      using T = float;                                                            \
      __VA_ARGS__;                                                                \
    } else if ((TENSOR).scalar_type() == at::kBFloat16) {                         \
      using T = bf16;                                                             \
      __VA_ARGS__;                                                                \
    } else {                                                                      \
      TORCH_CHECK(false, "ragged ops: tensors are float32 or bfloat16");          \
    }                                                                             \
  } while (0)

static inline void check_i32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, ": int32 contiguous device tensor");
}
static inline void check_f32(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, ": float32 contiguous device tensor");
}
