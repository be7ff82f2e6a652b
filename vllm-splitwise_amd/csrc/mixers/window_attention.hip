// Attention over a sliding window plus kept first tokens, paged keys / values, heads' weights mixed after
// the softmax ("talking heads"), no rotation.
//
// Mixing after the softmax means head h's output is  sum_g talk[h, g] * (P_g V_c(h)),  P_g the NORMALISED
// weights of head g and c(h) the key/value head of h.  So every query head g accumulates P_g against the
// values of ALL key/value heads, flash-style with a running maximum (the normalisation happens once, at the
// end, which keeps the result independent of how the keys were tiled), and a second stage in the same
// workgroup mixes the heads through LDS.
//
// Token kernel: one workgroup per new token, its waves take the query heads in turn; a wave scores 64 keys
// at a time (a key per lane) and accumulates values with a lane per value channel.
#include "mixers_common.cuh"

namespace swm {

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / 64;

template <typename T>
__device__ __forceinline__ float dot_row(const float* __restrict__ q, const void* __restrict__ krow, int dim);

template <>
__device__ __forceinline__ float dot_row<float>(const float* __restrict__ q, const void* __restrict__ krow, int dim) {
  const float* k = static_cast<const float*>(krow);
  float s = 0.0f;
  if ((dim & 3) == 0) {
    for (int d = 0; d < dim; d += 4) {
      const float4 kv = *reinterpret_cast<const float4*>(k + d);
      s += q[d] * kv.x + q[d + 1] * kv.y + q[d + 2] * kv.z + q[d + 3] * kv.w;
    }
  } else {
    for (int d = 0; d < dim; ++d) s += q[d] * k[d];
  }
  return s;
}

template <>
__device__ __forceinline__ float dot_row<bf16_t>(const float* __restrict__ q, const void* __restrict__ krow, int dim) {
  const uint16_t* k = static_cast<const uint16_t*>(krow);
  float s = 0.0f;
  if ((dim & 7) == 0) {
    for (int d = 0; d < dim; d += 8) {
      const uint4 kv = *reinterpret_cast<const uint4*>(k + d);
      const uint32_t w[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        s += q[d + 2 * e] * __uint_as_float(w[e] << 16);
        s += q[d + 2 * e + 1] * __uint_as_float(w[e] & 0xffff0000u);
      }
    }
  } else {
    for (int d = 0; d < dim; ++d) s += q[d] * sw::bf16_bits_to_float(k[d]);
  }
  return s;
}

// GMAX >= kv_heads, NV >= ceil(vdim / 64)
template <typename T, int GMAX, int NV>
__global__ __launch_bounds__(kAttnThreads) void window_attention_token_kernel(
    void* __restrict__ out, const float* __restrict__ q, const void* __restrict__ key_cache,
    const void* __restrict__ value_cache, const float* __restrict__ talk, const int32_t* __restrict__ block_tables,
    int table_width, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ token_seq, int heads, int kv_heads, int dim, int vdim, int page_size, float scale,
    int window, int keep_first) {
  extern __shared__ float lds[];
  float* q_lds = lds;                                   // [heads * dim]
  float* mixed = lds + heads * dim;                     // [heads][kv_heads][vdim]
  const int64_t t = blockIdx.x;
  const int s = token_seq[t];
  const int i = ctx_len[s] + (int)(t - q_start[s]);     // position of this token in its sequence
  for (int e = threadIdx.x; e < heads * dim; e += kAttnThreads) q_lds[e] = q[t * (int64_t)heads * dim + e];
  __syncthreads();
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int32_t* table = block_tables + (int64_t)s * table_width;
  const int lo = max(0, i - window + 1);
  const int n_first = min(keep_first, lo);              // kept first tokens that the window does not cover
  const int total = n_first + (i - lo + 1);
  const int group = heads / kv_heads;
  const size_t esz = sizeof(typename Conv<T>::store_t);
  for (int g = wave; g < heads; g += kAttnWaves) {
    const int c0 = g / group;
    const float* qg = q_lds + g * dim;
    float m = -INFINITY, l = 0.0f;
    float acc[GMAX][NV];
#pragma unroll
    for (int cc = 0; cc < GMAX; ++cc)
#pragma unroll
      for (int dd = 0; dd < NV; ++dd) acc[cc][dd] = 0.0f;
    for (int base = 0; base < total; base += 64) {
      const int idx = base + lane;
      const bool valid = idx < total;
      const int j = idx < n_first ? idx : lo + idx - n_first;
      int64_t phys = 0;
      float sc = -INFINITY;
      if (valid) {
        phys = (int64_t)table[j / page_size] * page_size + j % page_size;
        sc = dot_row<T>(qg, static_cast<const char*>(key_cache) + (phys * kv_heads + c0) * dim * esz, dim) * scale;
      }
      const float m_new = fmaxf(m, sw::wave_max(sc));
      const float corr = expf(m - m_new);               // 0 at the first tile (m = -inf)
      const float p = valid ? expf(sc - m_new) : 0.0f;
      l = l * corr + sw::wave_sum(p);
#pragma unroll
      for (int cc = 0; cc < GMAX; ++cc)
#pragma unroll
        for (int dd = 0; dd < NV; ++dd) acc[cc][dd] *= corr;
      const int cnt = min(64, total - base);
      for (int jj = 0; jj < cnt; ++jj) {
        const float pj = __shfl(p, jj, 64);
        const int64_t pr = __shfl(phys, jj, 64);
#pragma unroll
        for (int cc = 0; cc < GMAX; ++cc) {
          if (cc < kv_heads) {
#pragma unroll
            for (int dd = 0; dd < NV; ++dd) {
              const int d = lane + 64 * dd;
              if (d < vdim) acc[cc][dd] += pj * ld<T>(value_cache, (pr * kv_heads + cc) * vdim + d);
            }
          }
        }
      }
      m = m_new;
    }
    const float inv = 1.0f / l;
#pragma unroll
    for (int cc = 0; cc < GMAX; ++cc) {
      if (cc < kv_heads) {
#pragma unroll
        for (int dd = 0; dd < NV; ++dd) {
          const int d = lane + 64 * dd;
          if (d < vdim) mixed[((int64_t)g * kv_heads + cc) * vdim + d] = acc[cc][dd] * inv;
        }
      }
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < heads * vdim; e += kAttnThreads) {
    const int h = e / vdim, d = e % vdim;
    const int c = h / group;
    float o = 0.0f;
    for (int g = 0; g < heads; ++g) o += talk[h * heads + g] * mixed[((int64_t)g * kv_heads + c) * vdim + d];
    st<T>(out, t * (int64_t)heads * vdim + e, o);
  }
}

template <typename T, int GMAX, int NV>
int launch_token(void* out, const float* q, const void* key_cache, const void* value_cache, const float* talk,
                 const int32_t* block_tables, int table_width, const int32_t* q_start, const int32_t* ctx_len,
                 const int32_t* token_seq, int64_t rows, int heads, int kv_heads, int dim, int vdim, int page_size,
                 float scale, int window, int keep_first, hipStream_t stream) {
  const size_t lds = sizeof(float) * ((size_t)heads * dim + (size_t)heads * kv_heads * vdim);
  auto kernel = window_attention_token_kernel<T, GMAX, NV>;
  if (lds > 64 * 1024) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)rows), dim3(kAttnThreads), lds, stream, out, q, key_cache, value_cache,
                     talk, block_tables, table_width, q_start, ctx_len, token_seq, heads, kv_heads, dim, vdim,
                     page_size, scale, window, keep_first);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

#define SWM_DISPATCH_G(kv_heads, ...)                              \
  do {                                                             \
    if ((kv_heads) <= 1) { constexpr int GMAX = 1; __VA_ARGS__ }         \
    else if ((kv_heads) <= 2) { constexpr int GMAX = 2; __VA_ARGS__ }    \
    else if ((kv_heads) <= 4) { constexpr int GMAX = 4; __VA_ARGS__ }    \
    else if ((kv_heads) <= 8) { constexpr int GMAX = 8; __VA_ARGS__ }    \
    else { constexpr int GMAX = 16; __VA_ARGS__ }                        \
  } while (0)
#define SWM_DISPATCH_NV(vdim, ...)                                 \
  do {                                                             \
    if ((vdim) <= 64) { constexpr int NV = 1; __VA_ARGS__ }              \
    else if ((vdim) <= 128) { constexpr int NV = 2; __VA_ARGS__ }        \
    else { constexpr int NV = 4; __VA_ARGS__ }                           \
  } while (0)

extern "C" {

int swm_window_attention(void* out, const float* q, const void* key_cache, const void* value_cache,
                         const float* talk, const int32_t* block_tables, int table_width,
                         const int32_t* q_start, const int32_t* ctx_len, const int32_t* token_seq,
                         int64_t rows, int num_seqs, int heads, int kv_heads, int dim, int vdim, int page_size,
                         float scale, int window, int keep_first, int tiled, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "window_attention: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && kv_heads <= 16 && dim > 0 && vdim > 0 &&
                   vdim <= 256 && page_size > 0 && table_width > 0 && window > 0 && keep_first >= 0 &&
                   rows < (1ll << 31),
               "window_attention: heads %d, kv heads %d (up to 16), key size %d, value size %d (up to 256), page %d, "
               "window %d, kept first %d", heads, kv_heads, dim, vdim, page_size, window, keep_first);
  const size_t lds = sizeof(float) * ((size_t)heads * dim + (size_t)heads * kv_heads * vdim);
  SW_CHECK_ARG(lds <= 160 * 1024 - 1024, "window_attention: heads x kv heads x value size needs %zu bytes of LDS", lds);
  hipStream_t s = static_cast<hipStream_t>(stream);
  (void)tiled;
  (void)num_seqs;
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_G(kv_heads, SWM_DISPATCH_NV(vdim, return (launch_token<T, GMAX, NV>(
      out, q, key_cache, value_cache, talk, block_tables, table_width, q_start, ctx_len, token_seq, rows, heads,
      kv_heads, dim, vdim, page_size, scale, window, keep_first, s)););););
  return SW_OK;
}

}  // extern "C"
