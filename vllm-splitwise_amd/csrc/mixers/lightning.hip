// Linear attention with one decay per head ("lightning attention"):  S_t = decay_h S_(t-1) + k_t v_t^T,
// o_t = S_t^T q_t, with q, k, v = silu of their projections and the state S [key size, value size] carried in fp32
// per sequence.  A run of new tokens is taken in chunks of 32: inside a chunk the recurrence is three fp32
// matrix products on the matrix cores (v_mfma_f32_32x32x2_f32),
//     A   = (Q K^T) * D,  D[i, j] = decay^(i - j) for j <= i          (tokens of the chunk among themselves)
//     O   = A V + diag(decay^(i + 1)) Q S                              (plus what the carried state holds)
//     S  <- decay^n S + (K * decay^(n - 1 - j))^T V                    (n tokens in the chunk)
// which is the recurrence itself with its sums reordered.  Powers of the decay come from a table built by
// repeated multiplication, never from a quotient, so small decays do not overflow.
//
// One wave owns (sequence, head, 32 value channels) and keeps its slice of the state in registers across the
// whole run (the waves of a workgroup share the chunk's queries and keys, staged once in LDS), in the matrix cores' accumulator layout (lane l: value channel l % 32; element r of block b:
// key coordinate 32 b + 8 (r / 4) + 4 (l / 32) + r % 4).  That layout is also what the A operand of S^T q needs
// when q is read in the same order of coordinates, so the state never moves between registers.  A decoded
// token is a chunk of one.
#include "mixers_common.cuh"

namespace swm {

using f32x16 = __attribute__((ext_vector_type(16))) float;
constexpr int kChunk = 32;

__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }

// NDB: 32-coordinate blocks of the key size.  A workgroup owns (sequence, head) and up to 8 blocks of 32 value
// channels, one wave each; the chunk's silu(q) and silu(k) are staged once in LDS for all of them.
template <typename T, int NDB>
__global__ __launch_bounds__(512) void lightning_kernel(
    float* __restrict__ out, const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    int64_t in_stride, const float* __restrict__ decay, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int heads, int dim, int vdim) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DS = NDB * 32 + 4;                           // row stride of the staged tiles
  float* Qs = lds;                                           // [32][DS]
  float* Ks = Qs + kChunk * DS;                              // [32][DS]
  float* pw = Ks + kChunk * DS;                              // [kChunk + 1] powers of the decay
  const int seq = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, hl = lane >> 5;
  const int vb = blockIdx.z * (blockDim.x >> 6) + wave;
  const int row0 = q_start[seq], n = q_start[seq + 1] - row0;
  if (n <= 0) return;                                        // the whole workgroup
  const float lam = decay[h];
  if (threadIdx.x == 0) {
    float p = 1.0f;
    for (int e = 0; e <= kChunk; ++e) {
      pw[e] = p;
      p *= lam;
    }
  }
  const int vc = vb * 32 + li;                               // this lane's value channel
  const bool vc_ok = vc < vdim;
  float* sp = state + ((int64_t)state_slot[seq] * heads + h) * (int64_t)dim * vdim;

  f32x16 S[NDB];
  const bool fresh = ctx_len[seq] == 0;
#pragma unroll
  for (int b = 0; b < NDB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
      S[b][r] = (!fresh && vc_ok && c < dim) ? sp[(int64_t)c * vdim + vc] : 0.0f;
    }

  const int64_t qk_col = (int64_t)h * dim, v_col = (int64_t)h * vdim;
  for (int c0 = 0; c0 < n; c0 += kChunk) {
    const int cn = min(kChunk, n - c0);
    const int64_t base = (int64_t)(row0 + c0) * in_stride;
    __syncthreads();                                         // the last chunk's tiles have been read (and pw written)
    for (int e = threadIdx.x; e < kChunk * NDB * 32; e += blockDim.x) {
      const int r = e / (NDB * 32), c = e % (NDB * 32);
      float qv = 0.0f, kv = 0.0f;
      if (r < cn && c < dim) {
        qv = siluf_(ld<T>(q, base + r * in_stride + qk_col + c));
        kv = siluf_(ld<T>(k, base + r * in_stride + qk_col + c));
      }
      Qs[r * DS + c] = qv;
      Ks[r * DS + c] = kv;
    }
    // ---- values of the chunk: channel vc of token (r, hl)
    float vt[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 8 * (r / 4) + 4 * hl + (r % 4);
      vt[r] = (vc_ok && j < cn) ? siluf_(ld<T>(v, base + j * in_stride + v_col + vc)) : 0.0f;
    }
    __syncthreads();
    // ---- A^T = K Q^T (rows: keys, columns: queries); this lane: token li of the chunk as key and as query
    f32x16 a;
#pragma unroll
    for (int r = 0; r < 16; ++r) a[r] = 0.0f;
#pragma unroll
    for (int b = 0; b < NDB; ++b) {
      if (32 * b < dim) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int c = 32 * b + 8 * g4 + 4 * hl;
          const float4 qv = *reinterpret_cast<const float4*>(Qs + li * DS + c);
          const float4 kv = *reinterpret_cast<const float4*>(Ks + li * DS + c);
          a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qv.x, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qv.y, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qv.z, a, 0, 0, 0);
          a = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qv.w, a, 0, 0, 0);
        }
      }
    }
    // element r: key j = 8 (r / 4) + 4 hl + r % 4, query i = li
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 8 * (r / 4) + 4 * hl + (r % 4);
      a[r] = (j <= li && li < cn) ? a[r] * pw[max(li - j, 0)] : 0.0f;
    }
    // ---- O^T = V^T A^T + S^T (Q^T decay^(i + 1))
    f32x16 o;
#pragma unroll
    for (int r = 0; r < 16; ++r) o[r] = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) o = __builtin_amdgcn_mfma_f32_32x32x2f32(vt[r], a[r], o, 0, 0, 0);
    const float carry = pw[li + 1];
#pragma unroll
    for (int b = 0; b < NDB; ++b) {
      if (32 * b < dim) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const float4 qv = *reinterpret_cast<const float4*>(Qs + li * DS + 32 * b + 8 * g4 + 4 * hl);
          o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4], qv.x * carry, o, 0, 0, 0);
          o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4 + 1], qv.y * carry, o, 0, 0, 0);
          o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4 + 2], qv.z * carry, o, 0, 0, 0);
          o = __builtin_amdgcn_mfma_f32_32x32x2f32(S[b][4 * g4 + 3], qv.w * carry, o, 0, 0, 0);
        }
      }
    }
    if (li < cn && vb * 32 < vdim) {
      float* dst = out + (int64_t)(row0 + c0 + li) * heads * vdim + v_col + vb * 32;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 8 * (r / 4) + 4 * hl + (r % 4);
        if (vb * 32 + c < vdim) dst[c] = o[r];
      }
    }
    // ---- S <- decay^cn S + (K decay^(cn - 1 - j))^T V : A = keys transposed (coordinate li of block b, token (r, hl))
    const float keep = pw[cn];
#pragma unroll
    for (int b = 0; b < NDB; ++b) {
      if (32 * b < dim) {
#pragma unroll
        for (int r = 0; r < 16; ++r) S[b][r] *= keep;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = 8 * (r / 4) + 4 * hl + (r % 4);
          const float kv = j < cn ? Ks[j * DS + 32 * b + li] * pw[max(cn - 1 - j, 0)] : 0.0f;
          S[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(kv, vt[r], S[b], 0, 0, 0);
        }
      }
    }
  }
  if (vc_ok) {
#pragma unroll
    for (int b = 0; b < NDB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
        if (c < dim) sp[(int64_t)c * vdim + vc] = S[b][r];
      }
  }
}

template <typename T, int NDB>
int launch_lightning(float* out, const void* q, const void* k, const void* v, int64_t in_stride, const float* decay,
                     float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                     int num_seqs, int heads, int dim, int vdim, hipStream_t stream) {
  const int vblocks = (vdim + 31) / 32;
  const int waves = std::min(vblocks, 8);
  const size_t lds_bytes = (size_t)(2 * kChunk * (NDB * 32 + 4) + kChunk + 2) * sizeof(float);
  auto kernel = lightning_kernel<T, NDB>;
  static bool raised = false;                                // per instantiation
  if (lds_bytes > 64 * 1024 && !raised) {
    SW_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds_bytes));
    raised = true;
  }
  const dim3 grid((unsigned)num_seqs, (unsigned)heads, (unsigned)((vblocks + waves - 1) / waves));
  hipLaunchKernelGGL(kernel, grid, dim3(64 * waves), lds_bytes, stream, out, q, k, v, in_stride, decay, state, q_start,
                     ctx_len, state_slot, heads, dim, vdim);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

extern "C" int swm_lightning(float* out, const void* q, const void* k, const void* v, int64_t in_stride,
                             const float* decay, float* state, const int32_t* q_start, const int32_t* ctx_len,
                             const int32_t* state_slot, int64_t rows, int num_seqs, int heads, int dim, int vdim,
                             int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0 || num_seqs == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "lightning: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && heads < 65536 && dim > 0 && dim <= 256 && vdim > 0 && (vdim + 255) / 256 < 65536,
               "lightning: %d heads, key size %d (at most 256), value size %d", heads, dim, vdim);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SWM_LIGHTNING_CASE(N)                                                                                       \
  case N:                                                                                                           \
    SWM_DISPATCH_ACT(act_dtype, return (launch_lightning<T, N>(out, q, k, v, in_stride, decay, state, q_start,      \
                                                               ctx_len, state_slot, num_seqs, heads, dim, vdim, s));); \
    break;
  switch ((dim + 31) / 32) {
    SWM_LIGHTNING_CASE(1)
    SWM_LIGHTNING_CASE(2)
    SWM_LIGHTNING_CASE(3)
    SWM_LIGHTNING_CASE(4)
    SWM_LIGHTNING_CASE(5)
    SWM_LIGHTNING_CASE(6)
    SWM_LIGHTNING_CASE(7)
    SWM_LIGHTNING_CASE(8)
  }
#undef SWM_LIGHTNING_CASE
  return SW_OK;
}
