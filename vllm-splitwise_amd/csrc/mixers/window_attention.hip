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

// ------------------------------------------------------------------------------------------ staged kernel
// One workgroup per new token, all heads together.  A tile of 16 keys and their values (every key/value head) is
// staged ONCE in LDS as fp32 and shared by all heads: scores by threads (head, key), the running softmax by one
// thread per head, the value accumulation by threads (head, 4 + 4 value channels) for all key/value heads.  Needs
// key size % 4 == 0, value size % 8 == 0 and whole 16-byte vectors per cached row; other shapes take the
// kernel above.
constexpr int kTileKeys = 16;
constexpr int kKeyPad = 4;           // floats between staged key rows: 16 keys fall on 16 different bank groups

// key position of the idx-th visible key, and its slot in the cache (-1 past the end)
struct Visible {
  int lo, n_first, total, page_size;
  const int32_t* table;
  __device__ __forceinline__ int64_t slot(int idx) const {
    if (idx >= total) return -1;
    const int j = idx < n_first ? idx : lo + idx - n_first;
    return (int64_t)table[j / page_size] * page_size + j % page_size;
  }
};

template <typename T>
__device__ __forceinline__ void stage_rows(float* __restrict__ dst, int dst_stride, const void* __restrict__ cache,
                                           const Visible& vis, int base, int row_elems) {
  // kTileKeys rows of `row_elems` cache elements -> fp32; rows past the last visible key become zeros
  constexpr int V = sizeof(typename Conv<T>::store_t) == 2 ? 8 : 4;          // elements per 16-byte vector
  const int per_row = row_elems / V;
  for (int e = threadIdx.x; e < kTileKeys * per_row; e += kAttnThreads) {
    const int k = e / per_row, off = (e % per_row) * V;
    float* d = dst + k * dst_stride + off;
    const int64_t ph = vis.slot(base + k);
    if (ph < 0) {
#pragma unroll
      for (int i = 0; i < V; ++i) d[i] = 0.0f;
      continue;
    }
    const uint4 raw = *reinterpret_cast<const uint4*>(static_cast<const char*>(cache) +
                                                      (ph * row_elems + off) * sizeof(typename Conv<T>::store_t));
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
    if (V == 8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        d[2 * i] = __uint_as_float(w[i] << 16);
        d[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) d[i] = __uint_as_float(w[i]);
    }
  }
}

// NR: (head, 8-channel chunk) items per thread; GMAX >= kv_heads.
// gridDim.y > 1: the visible keys are cut into gridDim.y runs (whole tiles) and every workgroup leaves its
// un-normalised sums, running maximum and denominator in `partial`; window_attention_join_kernel finishes.
template <typename T, int GMAX, int NR>
__global__ __launch_bounds__(kAttnThreads) void window_attention_staged_kernel(
    void* __restrict__ out, const float* __restrict__ q, const void* __restrict__ key_cache,
    const void* __restrict__ value_cache, const float* __restrict__ talk, const int32_t* __restrict__ block_tables,
    int table_width, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ token_seq, int heads, int kv_heads, int dim, int vdim, int page_size, float scale,
    int window, int keep_first, float* __restrict__ partial) {
  extern __shared__ float lds[];
  const int krow = kv_heads * dim + kKeyPad, vrow = kv_heads * vdim;
  float* q_lds = lds;                                   // [heads * dim]
  float* p_lds = q_lds + heads * dim;                   // [heads][16] weights of the tile
  float* corr_lds = p_lds + heads * kTileKeys;          // [heads]
  float* m_lds = corr_lds + heads;                      // [heads] running maximum
  float* l_lds = m_lds + heads;                         // [heads] running denominator
  float* k_lds = l_lds + heads + heads % 4;             // [16][krow], on a 16-byte boundary
  float* v_lds = k_lds + kTileKeys * krow;              // [16][vrow]
  float* mixed = k_lds;                                 // [heads][kv_heads][vdim] once the tiles are done
  const int64_t t = blockIdx.x;
  const int s = token_seq[t];
  const int i = ctx_len[s] + (int)(t - q_start[s]);
  for (int e = threadIdx.x; e < heads * dim; e += kAttnThreads) q_lds[e] = q[t * (int64_t)heads * dim + e];
  for (int e = threadIdx.x; e < heads; e += kAttnThreads) {
    m_lds[e] = -INFINITY;
    l_lds[e] = 0.0f;
  }
  Visible vis;
  vis.table = block_tables + (int64_t)s * table_width;
  vis.page_size = page_size;
  vis.lo = max(0, i - window + 1);
  vis.n_first = min(keep_first, vis.lo);
  vis.total = vis.n_first + (i - vis.lo + 1);
  const int group = heads / kv_heads;
  const int chunks = vdim / 8;                          // per head
  // this workgroup's run of keys
  const int tiles = (vis.total + kTileKeys - 1) / kTileKeys;
  const int per_split = (tiles + gridDim.y - 1) / gridDim.y;
  const int first = blockIdx.y * per_split * kTileKeys;
  const int last = min(vis.total, first + per_split * kTileKeys);
  float acc[NR][GMAX][8];
#pragma unroll
  for (int r = 0; r < NR; ++r)
#pragma unroll
    for (int c = 0; c < GMAX; ++c)
#pragma unroll
      for (int x = 0; x < 8; ++x) acc[r][c][x] = 0.0f;
  for (int base = first; base < last; base += kTileKeys) {
    __syncthreads();                                    // the previous tile is consumed (and q_lds is written)
    stage_rows<T>(k_lds, krow, key_cache, vis, base, kv_heads * dim);
    stage_rows<T>(v_lds, vrow, value_cache, vis, base, vrow);
    __syncthreads();
    // scores and the running softmax: the 16 keys of a head sit in 16 neighbouring lanes
    for (int item0 = 0; item0 < heads * kTileKeys; item0 += kAttnThreads) {
      const int item = item0 + threadIdx.x;
      const bool live = item < heads * kTileKeys;
      const int g = live ? item / kTileKeys : 0, k = item % kTileKeys;
      float sc = -INFINITY;
      if (live && base + k < vis.total) {
        const float4* qv = reinterpret_cast<const float4*>(q_lds + g * dim);
        const float4* kv = reinterpret_cast<const float4*>(k_lds + k * krow + (g / group) * dim);
        float dot = 0.0f;
        for (int d4 = 0; d4 < dim / 4; ++d4) {
          const float4 a = qv[d4], b = kv[d4];
          dot += a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
        }
        sc = dot * scale;
      }
      float m_tile = sc;
#pragma unroll
      for (int x = 8; x >= 1; x >>= 1) m_tile = fmaxf(m_tile, __shfl_xor(m_tile, x, 64));
      const float m_old = m_lds[g];
      const float m_new = fmaxf(m_old, m_tile);         // finite: the tile's first key is visible
      const float w = expf(sc - m_new);                 // 0 for keys past the end
      float sum = w;
#pragma unroll
      for (int x = 8; x >= 1; x >>= 1) sum += __shfl_xor(sum, x, 64);
      if (live) {
        p_lds[item] = w;
        if (k == 0) {
          const float corr = expf(m_old - m_new);       // 0 at the first tile
          corr_lds[g] = corr;
          l_lds[g] = l_lds[g] * corr + sum;
          m_lds[g] = m_new;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const int item = threadIdx.x + r * kAttnThreads;
      if (item >= heads * chunks) continue;
      const int g = item / chunks, ch = item % chunks;
      const float corr = corr_lds[g];
#pragma unroll
      for (int c = 0; c < GMAX; ++c)
#pragma unroll
        for (int x = 0; x < 8; ++x) acc[r][c][x] *= corr;
      const float* p = p_lds + g * kTileKeys;
#pragma unroll 4
      for (int k = 0; k < kTileKeys; ++k) {
        const float w = p[k];
#pragma unroll
        for (int c = 0; c < GMAX; ++c) {
          if (c < kv_heads) {
            // channels 4 ch .. 4 ch + 3 of each half of the head: 16 lanes read 256 contiguous bytes
            const float* vr = v_lds + k * vrow + c * vdim + ch * 4;
            const float4 a = *reinterpret_cast<const float4*>(vr), b = *reinterpret_cast<const float4*>(vr + vdim / 2);
            acc[r][c][0] += w * a.x; acc[r][c][1] += w * a.y; acc[r][c][2] += w * a.z; acc[r][c][3] += w * a.w;
            acc[r][c][4] += w * b.x; acc[r][c][5] += w * b.y; acc[r][c][6] += w * b.z; acc[r][c][7] += w * b.w;
          }
        }
      }
    }
  }
  __syncthreads();                                      // tiles are done: their space becomes `mixed`
  if (gridDim.y > 1) {
    // [token][split]{ m[heads], l[heads], acc[heads][kv_heads][vdim] }
    const int64_t stride = 2 * heads + (int64_t)heads * kv_heads * vdim;
    float* dst = partial + (t * gridDim.y + blockIdx.y) * stride;
    for (int e = threadIdx.x; e < heads; e += kAttnThreads) {
      dst[e] = m_lds[e];
      dst[heads + e] = l_lds[e];
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const int item = threadIdx.x + r * kAttnThreads;
      if (item >= heads * chunks) continue;
      const int g = item / chunks, ch = item % chunks;
#pragma unroll
      for (int c = 0; c < GMAX; ++c)
        if (c < kv_heads)
#pragma unroll
          for (int x = 0; x < 8; ++x)
            dst[2 * heads + ((int64_t)g * kv_heads + c) * vdim + (x < 4 ? 0 : vdim / 2) + ch * 4 + (x & 3)] = acc[r][c][x];
    }
    return;
  }
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    const int item = threadIdx.x + r * kAttnThreads;
    if (item >= heads * chunks) continue;
    const int g = item / chunks, ch = item % chunks;
    const float inv = 1.0f / l_lds[g];
#pragma unroll
    for (int c = 0; c < GMAX; ++c)
      if (c < kv_heads)
#pragma unroll
        for (int x = 0; x < 8; ++x)
          mixed[((int64_t)g * kv_heads + c) * vdim + (x < 4 ? 0 : vdim / 2) + ch * 4 + (x & 3)] = acc[r][c][x] * inv;
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

// joins the runs of keys of one token: weights exp(m_s - M) / sum, then the mix of the heads
template <typename T>
__global__ __launch_bounds__(kAttnThreads) void window_attention_join_kernel(
    void* __restrict__ out, const float* __restrict__ partial, const float* __restrict__ talk, int splits, int heads,
    int kv_heads, int vdim) {
  extern __shared__ float lds[];
  float* wgt = lds;                                     // [splits][heads]: exp(m_s - M) / l
  float* mixed = lds + splits * heads + (splits * heads) % 4;
  const int64_t t = blockIdx.x;
  const int64_t stride = 2 * heads + (int64_t)heads * kv_heads * vdim;
  const float* src = partial + t * splits * stride;
  for (int g = threadIdx.x; g < heads; g += kAttnThreads) {
    float M = -INFINITY;
    for (int sp = 0; sp < splits; ++sp) M = fmaxf(M, src[sp * stride + g]);
    float l = 0.0f;
    for (int sp = 0; sp < splits; ++sp) {
      const float m = src[sp * stride + g];
      const float f = m == -INFINITY ? 0.0f : expf(m - M);         // a run without keys
      wgt[sp * heads + g] = f;
      l += f * src[sp * stride + heads + g];
    }
    for (int sp = 0; sp < splits; ++sp) wgt[sp * heads + g] /= l;
  }
  __syncthreads();
  const int n = heads * kv_heads * vdim;
  for (int e = threadIdx.x; e < n; e += kAttnThreads) {
    const int g = e / (kv_heads * vdim);
    float a = 0.0f;
    for (int sp = 0; sp < splits; ++sp) a += wgt[sp * heads + g] * src[sp * stride + 2 * heads + e];
    mixed[e] = a;
  }
  __syncthreads();
  const int group = heads / kv_heads;
  for (int e = threadIdx.x; e < heads * vdim; e += kAttnThreads) {
    const int h = e / vdim, d = e % vdim;
    const int c = h / group;
    float o = 0.0f;
    for (int g = 0; g < heads; ++g) o += talk[h * heads + g] * mixed[((int64_t)g * kv_heads + c) * vdim + d];
    st<T>(out, t * (int64_t)heads * vdim + e, o);
  }
}

inline size_t staged_lds_bytes(int heads, int kv_heads, int dim, int vdim) {
  const size_t tiles = (size_t)kTileKeys * (kv_heads * dim + kKeyPad) + (size_t)kTileKeys * kv_heads * vdim;
  const size_t mixed = (size_t)heads * kv_heads * vdim;
  // `mixed` lies over the tiles, which come last
  const size_t body = (size_t)heads * dim + (tiles > mixed ? tiles : mixed) + (size_t)heads * (kTileKeys + 3) + 4;
  return body * sizeof(float);
}

template <typename T, int GMAX, int NR>
int launch_staged(void* out, const float* q, const void* key_cache, const void* value_cache, const float* talk,
                  const int32_t* block_tables, int table_width, const int32_t* q_start, const int32_t* ctx_len,
                  const int32_t* token_seq, int64_t rows, int heads, int kv_heads, int dim, int vdim, int page_size,
                  float scale, int window, int keep_first, int splits, float* partial, hipStream_t stream) {
  const size_t lds = staged_lds_bytes(heads, kv_heads, dim, vdim);
  auto kernel = window_attention_staged_kernel<T, GMAX, NR>;
  static thread_local size_t allowed = 64 * 1024;       // what this instantiation may use so far
  if (lds > allowed) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    allowed = lds;
  }
  hipLaunchKernelGGL(kernel, dim3((unsigned)rows, (unsigned)splits), dim3(kAttnThreads), lds, stream, out, q, key_cache,
                     value_cache, talk, block_tables, table_width, q_start, ctx_len, token_seq, heads, kv_heads, dim,
                     vdim, page_size, scale, window, keep_first, partial);
  SW_CHECK_LAUNCH();
  if (splits > 1) {
    const size_t jl = sizeof(float) * ((size_t)splits * heads + 4 + (size_t)heads * kv_heads * vdim);
    auto join = window_attention_join_kernel<T>;
    static thread_local size_t join_allowed = 64 * 1024;
    if (jl > join_allowed) {
      SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(join), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)jl));
      join_allowed = jl;
    }
    hipLaunchKernelGGL(join, dim3((unsigned)rows), dim3(kAttnThreads), jl, stream, out, partial, talk, splits, heads,
                       kv_heads, vdim);
    SW_CHECK_LAUNCH();
  }
  return SW_OK;
}

template <typename T, int GMAX, int NV>
int launch_token(void* out, const float* q, const void* key_cache, const void* value_cache, const float* talk,
                 const int32_t* block_tables, int table_width, const int32_t* q_start, const int32_t* ctx_len,
                 const int32_t* token_seq, int64_t rows, int heads, int kv_heads, int dim, int vdim, int page_size,
                 float scale, int window, int keep_first, hipStream_t stream) {
  const size_t lds = sizeof(float) * ((size_t)heads * dim + (size_t)heads * kv_heads * vdim);
  auto kernel = window_attention_token_kernel<T, GMAX, NV>;
  static thread_local size_t allowed = 64 * 1024;
  if (lds > allowed) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    allowed = lds;
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
                         float scale, int window, int keep_first, int splits, float* partial, int act_dtype,
                         void* stream) {
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
  (void)num_seqs;
  SW_CHECK_ARG(splits >= 1 && splits <= 64 && (splits == 1 || partial != nullptr), "window_attention: %d runs of keys", splits);
  // the staged kernel for shapes made of whole vectors whose accumulators fit the registers
  const int vec = act_dtype == SW_BF16 ? 8 : 4;
  const int items = heads * (vdim / 8);
  const int nr = (items + kAttnThreads - 1) / kAttnThreads;
  const int gmax = kv_heads <= 1 ? 1 : kv_heads <= 2 ? 2 : kv_heads <= 4 ? 4 : kv_heads <= 8 ? 8 : 16;
  if (dim % 4 == 0 && vdim % 8 == 0 && (kv_heads * dim) % vec == 0 && (kv_heads * vdim) % vec == 0 && heads <= kAttnThreads &&
      nr * gmax <= 16 && nr <= 4 && staged_lds_bytes(heads, kv_heads, dim, vdim) <= 150 * 1024) {
    SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_G(kv_heads, {
      if (nr <= 1) return (launch_staged<T, GMAX, 1>(out, q, key_cache, value_cache, talk, block_tables, table_width, q_start, ctx_len, token_seq, rows, heads, kv_heads, dim, vdim, page_size, scale, window, keep_first, splits, partial, s));
      if (nr <= 2) return (launch_staged<T, GMAX, 2>(out, q, key_cache, value_cache, talk, block_tables, table_width, q_start, ctx_len, token_seq, rows, heads, kv_heads, dim, vdim, page_size, scale, window, keep_first, splits, partial, s));
      return (launch_staged<T, GMAX, 4>(out, q, key_cache, value_cache, talk, block_tables, table_width, q_start, ctx_len, token_seq, rows, heads, kv_heads, dim, vdim, page_size, scale, window, keep_first, splits, partial, s));
    }););
  }
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_G(kv_heads, SWM_DISPATCH_NV(vdim, return (launch_token<T, GMAX, NV>(
      out, q, key_cache, value_cache, talk, block_tables, table_width, q_start, ctx_len, token_seq, rows, heads,
      kv_heads, dim, vdim, page_size, scale, window, keep_first, s)););););
  return SW_OK;
}

}  // extern "C"
