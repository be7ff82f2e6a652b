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

// exp, sigmoid-weighted unit and tanh on the hardware's exp2 and reciprocal (a few ulp; for the inner loops of kernels
// whose arithmetic is otherwise bound by these functions)
__device__ __forceinline__ float fast_expf_(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_siluf_(float x) { return x * __builtin_amdgcn_rcpf(1.0f + fast_expf_(-x)); }
// tanh(x) = 1 - 2 / (1 + e^(2x)); e^(2x) -> inf gives 1, -> 0 gives -1
__device__ __forceinline__ float fast_tanhf_(float x) {
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + fast_expf_(2.0f * x));
}

// sum over groups of LK = 8 or 16 neighbouring lanes (every lane of a group gets it): DPP quad permutes and row
// mirrors, full-rate vector instructions with no trip through the LDS crossbar
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int LK>
__device__ __forceinline__ float lanes_sum(float v) {
  static_assert(LK == 8 || LK == 16, "groups of 8 or 16 lanes");
  v += dpp_move<0xB1>(v);                                    // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);                                    // quad_perm [2, 3, 0, 1]: every lane of a quad has the quad's sum
  v += dpp_move<0x141>(v);                                   // row_half_mirror: lane i of 8 reads lane 7 - i, the other quad
  if (LK == 16) v += dpp_move<0x140>(v);                     // row_mirror: lane i of 16 reads lane 15 - i, the other half
  return v;
}

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

// -> sequence and first new token of tile `tile` when every sequence's new tokens are cut into runs of `tpt`;
//    returns the tokens in the tile (0: no such tile)
__device__ __forceinline__ int find_query_tile(const int32_t* __restrict__ q_start, int num_seqs, int tile, int tpt,
                                               int* seq, int* tok0) {
  for (int s = 0; s < num_seqs; ++s) {
    const int n = q_start[s + 1] - q_start[s];
    const int tiles = (n + tpt - 1) / tpt;
    if (tile < tiles) {
      *seq = s;
      *tok0 = tile * tpt;
      return min(tpt, n - tile * tpt);
    }
    tile -= tiles;
  }
  return 0;
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
