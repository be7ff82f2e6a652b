// Delta-rule recurrences with an fp32 state per (sequence slot, head): S is [dim, vdim], keys index rows.
//
// Two launches per layer.  A PROLOGUE, parallel over tokens, computes everything of a token that does not depend
// on the state (unit vectors, decays with their softplus / exponentials, removal rates, beta) into one fp32
// operand block per (token, head).  The RECURRENCE then only multiplies and adds.
//
// Work split of the recurrence for wave64: one wave owns 16 columns of one head's state; a column is spread over
// 4 lanes that each hold a quarter of its rows in registers (lane = 4 * column + row group).  A product with a
// key-side vector (S^T k, S^T q) is a per-lane partial sum over its rows plus two xor-shuffles; no LDS, no
// barriers, so the only serial dependence is the recurrence itself.  The state is read once at the first token
// of the step (not at all when the sequence starts here) and written once after the last: a decode step moves
// exactly the state, a prompt portion moves it once per portion.  The next token's operands are fetched
// (float4 loads) before the current token's arithmetic.
#include "mixers_common.cuh"

namespace swm {

constexpr int kColsPerWave = 16;
constexpr int kPrepThreads = 256;

__device__ __forceinline__ float group_sum(float v) {      // over the 4 lanes of a column
  v += __shfl_xor(v, 1, 64);
  v += __shfl_xor(v, 2, 64);
  return v;
}

// ---------------------------------------------------------------------------------------- prologues
// Everything of a token that does not depend on the state is computed once, in parallel over tokens, into
// an fp32 operand block per (token, head): the recurrence then only multiplies and adds.
//
// channel rule: ops[t, h] = { q (unit, times dim^-1/2) | k (unit) | g (decay) }, beta[t, h]
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void channel_delta_prep_kernel(
    float* __restrict__ ops, float* __restrict__ beta, const float* __restrict__ qkv,
    const void* __restrict__ beta_pre, int64_t beta_stride, const void* __restrict__ decay_pre,
    const float* __restrict__ dt_bias, const float* __restrict__ a_log, int heads, int kv_heads, int dim, int vdim) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t row_w = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  const float* row = qkv + t * row_w;
  const int group = heads / kv_heads;
  const float qscale = 1.0f / sqrtf((float)dim);
  for (int h = wave; h < heads; h += kPrepThreads / 64) {
    const int c = h / group;
    const float* q = row + c * dim;
    const float* k = row + (int64_t)kv_heads * dim + c * dim;
    float qq = 0.0f, kk = 0.0f;
    for (int i = lane; i < dim; i += 64) {
      qq += q[i] * q[i];
      kk += k[i] * k[i];
    }
    qq = sw::wave_sum(qq);
    kk = sw::wave_sum(kk);
    const float qf = qscale / sqrtf(qq + 1e-6f), kf = 1.0f / sqrtf(kk + 1e-6f);
    const float rate = expf(a_log[h]);
    float* o = ops + (t * heads + h) * 3 * (int64_t)dim;
    for (int i = lane; i < dim; i += 64) {
      o[i] = q[i] * qf;
      o[dim + i] = k[i] * kf;
      o[2 * dim + i] = expf(-rate * softplusf_(ld<T>(decay_pre, (t * heads + h) * (int64_t)dim + i) + dt_bias[h * dim + i]));
    }
    if (lane == 0) beta[t * heads + h] = sigmoidf_(ld<T>(beta_pre, t * beta_stride + h));
  }
}

// general rule: ops[t, h] = { r | k | w (decay) | a k / (|k|^2 + 1e-6) }: with u = k / |k| the removal term
// (a * u)(u^T S) equals (a k / |k|^2)(k^T S)
template <typename T>
__global__ __launch_bounds__(kPrepThreads) void general_delta_prep_kernel(
    float* __restrict__ ops, const void* __restrict__ rp, const void* __restrict__ kp, int64_t rkv_stride,
    const void* __restrict__ decay_pre, int64_t decay_stride, const float* __restrict__ w0,
    const void* __restrict__ rate_pre, int64_t rate_stride, const float* __restrict__ a_bias, int heads, int dim) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float kDecay = 0.60653065971263342f;            // exp(-1/2)
  for (int h = wave; h < heads; h += kPrepThreads / 64) {
    float kk = 0.0f;
    for (int i = lane; i < dim; i += 64) {
      const float k = ld<T>(kp, t * rkv_stride + h * dim + i);
      kk += k * k;
    }
    kk = sw::wave_sum(kk);
    const float inv = 1.0f / (kk + 1e-6f);
    float* o = ops + (t * heads + h) * 4 * (int64_t)dim;
    for (int i = lane; i < dim; i += 64) {
      const float k = ld<T>(kp, t * rkv_stride + h * dim + i);
      o[i] = ld<T>(rp, t * rkv_stride + h * dim + i);
      o[dim + i] = k;
      o[2 * dim + i] = expf(-kDecay * sigmoidf_(ld<T>(decay_pre, t * decay_stride + h * dim + i) + w0[h * dim + i]));
      o[3 * dim + i] = sigmoidf_(ld<T>(rate_pre, t * rate_stride + h * dim + i) + a_bias[h * dim + i]) * k * inv;
    }
  }
}

// ---------------------------------------------------------------------------------------- recurrences
// RQ rows per lane (a multiple of 4; dim <= 4 * RQ): lane group rg holds rows [rg * RQ, (rg + 1) * RQ).
// NOPS operand vectors of `dim` floats per (token, head), read as float4 when dim is a multiple of 4.
template <int RQ, int NOPS>
struct Operands {
  float v[NOPS][RQ];
  __device__ __forceinline__ void fetch(const float* __restrict__ base, int dim, int row0) {
    if ((dim & 3) == 0) {
#pragma unroll
      for (int a = 0; a < NOPS; ++a)
#pragma unroll
        for (int i = 0; i < RQ; i += 4) {
          float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
          if (row0 + i < dim) x = *reinterpret_cast<const float4*>(base + a * dim + row0 + i);
          v[a][i] = x.x; v[a][i + 1] = x.y; v[a][i + 2] = x.z; v[a][i + 3] = x.w;
        }
    } else {
#pragma unroll
      for (int a = 0; a < NOPS; ++a)
#pragma unroll
        for (int i = 0; i < RQ; ++i) v[a][i] = row0 + i < dim ? base[a * dim + row0 + i] : 0.0f;
    }
  }
};

template <int RQ>
__global__ __launch_bounds__(64) void channel_delta_kernel(
    float* __restrict__ out, const float* __restrict__ ops, const float* __restrict__ beta,
    const float* __restrict__ qkv, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ state_slot, int heads, int kv_heads, int dim,
    int vdim) {
  const int lane = threadIdx.x, rg = lane & 3, row0 = rg * RQ;
  const int col = blockIdx.x * kColsPerWave + (lane >> 2);
  const int h = blockIdx.y, s = blockIdx.z;
  const int first = q_start[s], n = q_start[s + 1] - first;
  if (n == 0) return;
  const bool col_ok = col < vdim;
  const int colc = col_ok ? col : vdim - 1;             // out-of-range lanes shadow the last column, never store
  const int64_t row_w = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  const int64_t v_off = 2 * (int64_t)kv_heads * dim + (int64_t)h * vdim + colc;
  float* S = state + ((int64_t)state_slot[s] * heads + h) * dim * vdim;
  float Sr[RQ];
#pragma unroll
  for (int i = 0; i < RQ; ++i) Sr[i] = (ctx_len[s] > 0 && row0 + i < dim) ? S[(int64_t)(row0 + i) * vdim + colc] : 0.0f;
  Operands<RQ, 3> nxt;
  float vn, bn;
  auto fetch = [&](int t) {
    nxt.fetch(ops + ((int64_t)t * heads + h) * 3 * dim, dim, row0);
    vn = qkv[(int64_t)t * row_w + v_off];
    bn = beta[(int64_t)t * heads + h];
  };
  fetch(first);
  for (int t = first; t < first + n; ++t) {
    const Operands<RQ, 3> cur = nxt;
    const float v = vn, b = bn;
    if (t + 1 < first + n) fetch(t + 1);
    float ks = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      Sr[i] *= cur.v[2][i];
      ks += cur.v[1][i] * Sr[i];
    }
    ks = group_sum(ks);
    const float u = b * (v - ks);
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      Sr[i] += cur.v[1][i] * u;
      o += cur.v[0][i] * Sr[i];
    }
    o = group_sum(o);
    if (rg == 0 && col_ok) out[((int64_t)t * heads + h) * vdim + col] = o;
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RQ; ++i)
      if (row0 + i < dim) S[(int64_t)(row0 + i) * vdim + col] = Sr[i];
  }
}

template <typename T, int RQ>
__global__ __launch_bounds__(64) void general_delta_kernel(
    float* __restrict__ out, const float* __restrict__ ops, const void* __restrict__ vp, int64_t v_stride,
    float* __restrict__ state, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ state_slot, int heads, int dim) {
  const int lane = threadIdx.x, rg = lane & 3, row0 = rg * RQ;
  const int col = blockIdx.x * kColsPerWave + (lane >> 2);
  const int h = blockIdx.y, s = blockIdx.z;
  const int first = q_start[s], n = q_start[s + 1] - first;
  if (n == 0) return;
  const bool col_ok = col < dim;
  const int colc = col_ok ? col : dim - 1;
  float* S = state + ((int64_t)state_slot[s] * heads + h) * dim * dim;
  float Sr[RQ];
#pragma unroll
  for (int i = 0; i < RQ; ++i) Sr[i] = (ctx_len[s] > 0 && row0 + i < dim) ? S[(int64_t)(row0 + i) * dim + colc] : 0.0f;
  Operands<RQ, 4> nxt;
  float vn;
  auto fetch = [&](int t) {
    nxt.fetch(ops + ((int64_t)t * heads + h) * 4 * dim, dim, row0);
    vn = ld<T>(vp, (int64_t)t * v_stride + h * dim + colc);
  };
  fetch(first);
  for (int t = first; t < first + n; ++t) {
    const Operands<RQ, 4> cur = nxt;
    const float v = vn;
    if (t + 1 < first + n) fetch(t + 1);
    float ks = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) ks += cur.v[1][i] * Sr[i];
    ks = group_sum(ks);                                  // k^T S of the OLD state
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      Sr[i] = cur.v[2][i] * Sr[i] - cur.v[3][i] * ks + cur.v[1][i] * v;
      o += cur.v[0][i] * Sr[i];
    }
    o = group_sum(o);
    if (rg == 0 && col_ok) out[((int64_t)t * heads + h) * dim + col] = o;
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RQ; ++i)
      if (row0 + i < dim) S[(int64_t)(row0 + i) * dim + col] = Sr[i];
  }
}

}  // namespace swm

// rows per lane for a key size: 4, 8, 16, 32 or 64 (key sizes up to 256)
#define SWM_DISPATCH_ROWS(dim, ...)                       \
  do {                                                    \
    if ((dim) <= 16) { constexpr int RQ = 4; __VA_ARGS__ }        \
    else if ((dim) <= 32) { constexpr int RQ = 8; __VA_ARGS__ }   \
    else if ((dim) <= 64) { constexpr int RQ = 16; __VA_ARGS__ }  \
    else if ((dim) <= 128) { constexpr int RQ = 32; __VA_ARGS__ } \
    else { constexpr int RQ = 64; __VA_ARGS__ }                   \
  } while (0)

extern "C" {

int64_t swm_channel_delta_workspace_floats(int64_t rows, int heads, int dim) { return rows * heads * (3 * (int64_t)dim + 1); }
int64_t swm_general_delta_workspace_floats(int64_t rows, int heads, int dim) { return rows * heads * 4 * (int64_t)dim; }

int swm_channel_delta(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                      const void* decay_pre, const float* dt_bias, const float* a_log, float* state,
                      const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot, int64_t rows,
                      int num_seqs, int heads, int kv_heads, int dim, int vdim, float* workspace, int act_dtype,
                      void* stream) {
  using namespace swm;
  if (num_seqs == 0 || rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "channel_delta: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 256 && vdim > 0 &&
                   workspace != nullptr && rows < (1ll << 31),
               "channel_delta: heads %d, kv heads %d, key size %d (up to 256), value size %d", heads, kv_heads, dim,
               vdim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* ops = workspace;
  float* beta = workspace + rows * heads * 3 * (int64_t)dim;
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(channel_delta_prep_kernel<T>, dim3((unsigned)rows), dim3(kPrepThreads), 0,
                                                 s, ops, beta, qkv, beta_pre, beta_stride, decay_pre, dt_bias, a_log,
                                                 heads, kv_heads, dim, vdim););
  SW_CHECK_LAUNCH();
  const dim3 grid((unsigned)((vdim + kColsPerWave - 1) / kColsPerWave), (unsigned)heads, (unsigned)num_seqs);
  SWM_DISPATCH_ROWS(dim, hipLaunchKernelGGL((channel_delta_kernel<RQ>), grid, dim3(64), 0, s, out, ops, beta, qkv, state,
                                            q_start, ctx_len, state_slot, heads, kv_heads, dim, vdim););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

int swm_general_delta(float* out, const void* r, const void* k, const void* v, int64_t rkv_stride,
                      const void* decay_pre, int64_t decay_stride, const float* w0, const void* rate_pre,
                      int64_t rate_stride, const float* a_bias, float* state, const int32_t* q_start,
                      const int32_t* ctx_len, const int32_t* state_slot, int64_t rows, int num_seqs, int heads,
                      int dim, float* workspace, int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0 || rows == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "general_delta: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && dim > 0 && dim <= 256 && workspace != nullptr && rows < (1ll << 31),
               "general_delta: heads %d, key size %d (up to 256)", heads, dim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  SWM_DISPATCH_ACT(act_dtype, hipLaunchKernelGGL(general_delta_prep_kernel<T>, dim3((unsigned)rows), dim3(kPrepThreads), 0,
                                                 s, workspace, r, k, rkv_stride, decay_pre, decay_stride, w0, rate_pre,
                                                 rate_stride, a_bias, heads, dim););
  SW_CHECK_LAUNCH();
  const dim3 grid((unsigned)((dim + kColsPerWave - 1) / kColsPerWave), (unsigned)heads, (unsigned)num_seqs);
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_ROWS(dim, hipLaunchKernelGGL((general_delta_kernel<T, RQ>), grid, dim3(64), 0, s,
                                                                        out, workspace, v, rkv_stride, state, q_start,
                                                                        ctx_len, state_slot, heads, dim);););
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // extern "C"
