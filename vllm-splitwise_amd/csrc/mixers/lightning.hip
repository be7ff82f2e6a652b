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
constexpr int kWhole = 0, kLocal = 1, kFinal = 2;
constexpr int kSegment = 128;          // tokens per segment of a long run (a multiple of kChunk)


// NDB: 32-coordinate blocks of the key size.  A workgroup owns (sequence, head) and up to 8 blocks of 32 value
// channels, one wave each; the chunk's silu(q) and silu(k) are staged once in LDS for all of them.
template <typename T, int NDB>
__global__ __launch_bounds__(512) void lightning_kernel(
    float* __restrict__ out, const void* __restrict__ q, const void* __restrict__ k, const void* __restrict__ v,
    int64_t in_stride, const float* __restrict__ decay, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int num_seqs, int heads, int dim,
    int vdim, int mode, int seg_len, float* __restrict__ seg_state) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int DS = NDB * 32 + 4;                           // row stride of the staged tiles
  float* Qs = lds;                                           // [32][DS]
  float* Ks = Qs + kChunk * DS;                              // [32][DS]
  float* pw = Ks + kChunk * DS;                              // [kChunk + 1] powers of the decay
  const int h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, li = lane & 31, hl = lane >> 5;
  const int vb = blockIdx.z * (blockDim.x >> 6) + wave;
  // mode 0: blockIdx.x is a sequence and its whole run is taken from the slot's state to the slot's state.
  // Long runs are cut into segments of seg_len tokens that run side by side: mode 1 takes every segment but a
  // sequence's last from the EMPTY state and leaves its end state in seg_state[segment]; a scan (below) turns these
  // into the states at the segments' ends; mode 2 then takes every segment from its true start state (the slot's for
  // a sequence's first segment), writes the outputs, and a sequence's last segment leaves its state in the slot.
  int seq = blockIdx.x, tok0 = 0, n;
  if (mode == kWhole) {
    n = q_start[seq + 1] - q_start[seq];
  } else {
    n = find_query_tile(q_start, num_seqs, blockIdx.x, seg_len, &seq, &tok0);
  }
  if (n <= 0) return;                                        // the whole workgroup
  const int row0 = q_start[seq] + tok0;
  const bool last_seg = tok0 + n == q_start[seq + 1] - q_start[seq];
  if (mode == kLocal && last_seg) return;
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

  float* seg_out = seg_state + ((int64_t)blockIdx.x * heads + h) * (int64_t)dim * vdim;      // modes 1, 2 only
  const float* start = (mode == kFinal && tok0 > 0) ? seg_out - (int64_t)heads * dim * vdim : sp;

  f32x16 S[NDB];
  const bool fresh = mode == kLocal || (tok0 == 0 && ctx_len[seq] == 0);
#pragma unroll
  for (int b = 0; b < NDB; ++b)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
      S[b][r] = (!fresh && vc_ok && c < dim) ? start[(int64_t)c * vdim + vc] : 0.0f;
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
        qv = fast_siluf_(ld<T>(q, base + r * in_stride + qk_col + c));
        kv = fast_siluf_(ld<T>(k, base + r * in_stride + qk_col + c));
      }
      Qs[r * DS + c] = qv;
      Ks[r * DS + c] = kv;
    }
    // ---- values of the chunk: channel vc of token (r, hl)
    float vt[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int j = 8 * (r / 4) + 4 * hl + (r % 4);
      vt[r] = (vc_ok && j < cn) ? fast_siluf_(ld<T>(v, base + j * in_stride + v_col + vc)) : 0.0f;
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
    if (mode != kLocal && li < cn && vb * 32 < vdim) {
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
  if (mode == kFinal && !last_seg) return;                  // its end state is the next segment's start: known already
  float* end = mode == kLocal ? seg_out : sp;
  if (vc_ok) {
#pragma unroll
    for (int b = 0; b < NDB; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 32 * b + 8 * (r / 4) + 4 * hl + (r % 4);
        if (c < dim) end[(int64_t)c * vdim + vc] = S[b][r];
      }
  }
}

// seg_state[segment] (its end state from the empty state) -> the state at the segment's end:
// S_end(j) = decay^seg_len S_end(j - 1) + local(j), S_end(-1) = the slot's state (nothing for a new sequence)
__global__ __launch_bounds__(256) void lightning_scan_kernel(
    float* __restrict__ seg_state, const float* __restrict__ state, const float* __restrict__ decay,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot,
    int heads, int dim, int vdim, int seg_len) {
  const int seq = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int size = dim * vdim;
  if (e >= size) return;
  const int n = q_start[seq + 1] - q_start[seq];
  const int segs = (n + seg_len - 1) / seg_len;
  if (segs <= 1) return;
  int first = 0;
  for (int s = 0; s < seq; ++s) first += (q_start[s + 1] - q_start[s] + seg_len - 1) / seg_len;
  float keep = 1.0f;
  const float lam = decay[h];
  for (int i = 0; i < seg_len; ++i) keep *= lam;
  float S = ctx_len[seq] == 0 ? 0.0f : state[((int64_t)state_slot[seq] * heads + h) * size + e];
  // eight segments at a time: their loads do not wait for one another
  const int64_t stride = (int64_t)heads * size;
  float* p = seg_state + ((int64_t)first * heads + h) * size + e;
  for (int j0 = 0; j0 + 1 < segs; j0 += 8) {
    float local[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) local[i] = j0 + i + 1 < segs ? p[(j0 + i) * stride] : 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (j0 + i + 1 < segs) {
        S = keep * S + local[i];
        p[(j0 + i) * stride] = S;
      }
    }
  }
}

template <typename T, int NDB>
int launch_lightning(float* out, const void* q, const void* k, const void* v, int64_t in_stride, const float* decay,
                     float* state, const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                     int64_t rows, int num_seqs, int max_query_len, int heads, int dim, int vdim, float* seg_state,
                     hipStream_t stream) {
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
  const unsigned zgroups = (unsigned)((vblocks + waves - 1) / waves);
  if (seg_state == nullptr || max_query_len <= 2 * kSegment) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)num_seqs, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream,
                       out, q, k, v, in_stride, decay, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim,
                       kWhole, kSegment, seg_state);
    SW_CHECK_LAUNCH();
    return SW_OK;
  }
  const unsigned items = (unsigned)(rows / kSegment + num_seqs);
  hipLaunchKernelGGL(kernel, dim3(items, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream, out, q, k, v,
                     in_stride, decay, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, kLocal, kSegment,
                     seg_state);
  SW_CHECK_LAUNCH();
  hipLaunchKernelGGL(lightning_scan_kernel, dim3((unsigned)num_seqs, (unsigned)heads, (unsigned)((dim * vdim + 255) / 256)),
                     dim3(256), 0, stream, seg_state, state, decay, q_start, ctx_len, state_slot, heads, dim, vdim,
                     kSegment);
  SW_CHECK_LAUNCH();
  hipLaunchKernelGGL(kernel, dim3(items, (unsigned)heads, zgroups), dim3(64 * waves), lds_bytes, stream, out, q, k, v,
                     in_stride, decay, state, q_start, ctx_len, state_slot, num_seqs, heads, dim, vdim, kFinal, kSegment,
                     seg_state);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

extern "C" int64_t swm_lightning_workspace_floats(int64_t rows, int num_seqs, int max_query_len, int heads, int dim,
                                                  int vdim) {
  if (max_query_len <= 2 * swm::kSegment) return 0;
  return (rows / swm::kSegment + num_seqs) * (int64_t)heads * dim * vdim;
}

extern "C" int swm_lightning(float* out, const void* q, const void* k, const void* v, int64_t in_stride,
                             const float* decay, float* state, const int32_t* q_start, const int32_t* ctx_len,
                             const int32_t* state_slot, int64_t rows, int num_seqs, int max_query_len, int heads,
                             int dim, int vdim, float* workspace, int act_dtype, void* stream) {
  using namespace swm;
  if (rows == 0 || num_seqs == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "lightning: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && heads < 65536 && dim > 0 && dim <= 256 && vdim > 0 && (vdim + 255) / 256 < 65536,
               "lightning: %d heads, key size %d (at most 256), value size %d", heads, dim, vdim);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define SWM_LIGHTNING_CASE(N)                                                                                       \
  case N:                                                                                                           \
    SWM_DISPATCH_ACT(act_dtype, return (launch_lightning<T, N>(out, q, k, v, in_stride, decay, state, q_start,      \
                                                               ctx_len, state_slot, rows, num_seqs, max_query_len,  \
                                                               heads, dim, vdim, workspace, s)););                  \
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
