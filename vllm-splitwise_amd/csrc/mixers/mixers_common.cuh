// Shared pieces of the mixer kernels: the library's error slot and the ragged-step argument checks.
#pragma once

#include "../common.cuh"
#include "../../../include/splitwise_mixers.h"

namespace swm {

using sw::bf16_t;
using sw::Conv;

inline bool act_ok(int dt) { return dt == SW_F32 || dt == SW_BF16; }

template <typename T>
__device__ __forceinline__ float ld(const void* p, int64_t i) {
  return Conv<T>::to_float(static_cast<const typename Conv<T>::store_t*>(p)[i]);
}
template <typename T>
__device__ __forceinline__ void st(void* p, int64_t i, float v) {
  static_cast<typename Conv<T>::store_t*>(p)[i] = Conv<T>::from_float(v);
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
// softplus without overflow: log(1 + e^x) = max(x, 0) + log1p(e^-|x|)
__device__ __forceinline__ float softplusf_(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }

// sum over the threads of a workgroup (blockDim.x a multiple of 64, at most 1024); every thread gets it
__device__ __forceinline__ float block_sum(float v, float* lds /* >= 16 floats */) {
  v = sw::wave_sum(v);
  const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds[wave] = v;
  __syncthreads();
  float total = 0.0f;
  for (int w = 0; w < waves; ++w) total += lds[w];
  return total;
}

}  // namespace swm

// dispatch on the activation type: BODY sees `T`
#define SWM_DISPATCH_ACT(act_dtype, ...)                \
  do {                                                  \
    if ((act_dtype) == SW_F32) {                        \
      using T = float;                                  \
      __VA_ARGS__                                       \
    } else {                                            \
      using T = ::sw::bf16_t;                           \
      __VA_ARGS__                                       \
    }                                                   \
  } while (0)
