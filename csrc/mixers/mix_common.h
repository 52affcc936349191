// Element types of the mixer kernels: every kernel is built for bf16 and for fp32 activations /
// weights (a model served in float32 runs the same kernels with T = float), and accumulates,
// normalises and keeps the residual stream in fp32 in both.
#pragma once
#include "kernels/common.h"

namespace pkm {

using pk::bf16_t;

template <typename T>
__device__ __forceinline__ float ld(const T* p);
template <>
__device__ __forceinline__ float ld<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ld<bf16_t>(const bf16_t* p) { return pk::bf2f(*p); }

template <typename T>
__device__ __forceinline__ void st(T* p, float v);
template <>
__device__ __forceinline__ void st<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void st<bf16_t>(bf16_t* p, float v) { *p = pk::f2bf(v); }

__device__ __forceinline__ float sigmoidf(float z) { return 1.f / (1.f + expf(-z)); }

// dtype codes of the extern "C" launchers
constexpr int kBF16 = 0, kF32 = 1;

}  // namespace pkm

// launcher body for both element types: DISPATCH(dt, T, launch<T>(...))
#define PKM_DISPATCH(dt, T, ...)            \
  if ((dt) == pkm::kBF16) {                 \
    using T = pkm::bf16_t;                  \
    __VA_ARGS__;                            \
  } else if ((dt) == pkm::kF32) {           \
    using T = float;                        \
    __VA_ARGS__;                            \
  } else {                                  \
    return -2;                              \
  }
