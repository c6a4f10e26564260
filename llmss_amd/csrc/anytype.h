// Element access for kernels that run in either bf16 or fp32 storage (math is fp32 in both).
//
// The kernels of the fp32-residual block (resid32.hip), the strided / grouped GEMMs (gemm_any.hip, moe.hip) and
// the latent attention (attention_latent.hip) are templates over the storage type: bf16_t serves a model in its
// serving precision, float runs the same code as a true 32-bit model (no reduced-precision matrix mode).
#pragma once
#include "common.h"

template <typename T>
struct El;

template <>
struct El<float> {
  static __device__ __forceinline__ float ld(const float* p) { return *p; }
  static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};

template <>
struct El<bf16_t> {
  static __device__ __forceinline__ float ld(const bf16_t* p) { return bf2f(*p); }
  static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f2bf(v); }
};

// dtype codes shared with the Python launchers: 0 = bf16, 1 = fp32
#define DISPATCH_T(code, T, ...)                    \
  do {                                              \
    if ((code) == 0) {                              \
      typedef bf16_t T;                             \
      __VA_ARGS__;                                  \
    } else if ((code) == 1) {                       \
      typedef float T;                              \
      __VA_ARGS__;                                  \
    } else {                                        \
      throw std::runtime_error("bad dtype code");   \
    }                                               \
  } while (0)
