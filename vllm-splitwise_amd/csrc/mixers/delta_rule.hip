// Delta-rule recurrences with an fp32 state per (sequence slot, head): S is [dim, vdim], keys index rows.
//
// Work split for wave64: one wave owns 16 columns of one head's state; a column is spread over 4 lanes that
// hold every 4th row in registers (lane = 4 * column + row group).  A product with a key-side vector
// (S^T k, S^T q) is a per-lane partial sum over its rows plus two xor-shuffles; no LDS, no barriers, so the
// only serial dependence is the recurrence itself.  The state is read once at the first token of the step
// (not at all when the sequence starts here) and written once after the last: a decode step moves exactly
// the state, a prompt portion moves it once per portion.  The next token's operands are fetched before
// the current token's arithmetic.
#include "mixers_common.cuh"

namespace swm {

constexpr int kRowGroups = 4;
constexpr int kColsPerWave = 16;

__device__ __forceinline__ float group_sum(float v) {      // over the 4 lanes of a column
  v += __shfl_xor(v, 1, 64);
  v += __shfl_xor(v, 2, 64);
  return v;
}

// RQ = rows held per lane (dim <= 4 * RQ)
template <typename T, int RQ>
__global__ __launch_bounds__(64) void channel_delta_kernel(
    float* __restrict__ out, const float* __restrict__ qkv, const void* __restrict__ beta_pre, int64_t beta_stride,
    const void* __restrict__ decay_pre, const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    float* __restrict__ state, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ state_slot, int heads, int kv_heads, int dim, int vdim) {
  const int lane = threadIdx.x, rg = lane & 3;
  const int col = blockIdx.x * kColsPerWave + (lane >> 2);
  const int h = blockIdx.y, s = blockIdx.z;
  const int c = h / (heads / kv_heads);
  const int first = q_start[s], n = q_start[s + 1] - first;
  if (n == 0) return;
  const bool col_ok = col < vdim;
  const int colc = col_ok ? col : vdim - 1;             // out-of-range lanes shadow the last column, never store
  const int64_t row_w = 2 * (int64_t)kv_heads * dim + (int64_t)heads * vdim;
  float* S = state + ((int64_t)state_slot[s] * heads + h) * dim * vdim;
  float Sr[RQ];
#pragma unroll
  for (int i = 0; i < RQ; ++i) {
    const int r = 4 * i + rg;
    Sr[i] = (ctx_len[s] > 0 && r < dim) ? S[(int64_t)r * vdim + colc] : 0.0f;
  }
  const float rate = expf(a_log[h]);
  const float qscale = 1.0f / sqrtf((float)dim);
  float bias[RQ];
#pragma unroll
  for (int i = 0; i < RQ; ++i) {
    const int r = 4 * i + rg;
    bias[i] = r < dim ? dt_bias[h * dim + r] : 0.0f;
  }
  float qn[RQ], kn[RQ], dn[RQ], vn, bn;
  auto fetch = [&](int t) {
    const float* row = qkv + (int64_t)t * row_w;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      const int r = 4 * i + rg;
      const bool ok = r < dim;
      qn[i] = ok ? row[c * dim + r] : 0.0f;
      kn[i] = ok ? row[(int64_t)kv_heads * dim + c * dim + r] : 0.0f;
      dn[i] = ok ? ld<T>(decay_pre, ((int64_t)t * heads + h) * dim + r) : 0.0f;
    }
    vn = row[2 * (int64_t)kv_heads * dim + h * vdim + colc];
    bn = ld<T>(beta_pre, (int64_t)t * beta_stride + h);
  };
  fetch(first);
  for (int t = first; t < first + n; ++t) {
    float q[RQ], k[RQ], g[RQ];
    const float v = vn, beta = sigmoidf_(bn);
    float qq = 0.0f, kk = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      q[i] = qn[i];
      k[i] = kn[i];
      g[i] = expf(-rate * softplusf_(dn[i] + bias[i]));
      qq += q[i] * q[i];
      kk += k[i] * k[i];
    }
    if (t + 1 < first + n) fetch(t + 1);
    qq = group_sum(qq);
    kk = group_sum(kk);
    const float qf = qscale / sqrtf(qq + 1e-6f), kf = 1.0f / sqrtf(kk + 1e-6f);
    float ks = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      k[i] *= kf;
      Sr[i] *= g[i];
      ks += k[i] * Sr[i];
    }
    ks = group_sum(ks);
    const float u = beta * (v - ks);
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      Sr[i] += k[i] * u;
      o += q[i] * Sr[i];
    }
    o = group_sum(o) * qf;
    if (rg == 0 && col_ok) out[((int64_t)t * heads + h) * vdim + col] = o;
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      const int r = 4 * i + rg;
      if (r < dim) S[(int64_t)r * vdim + col] = Sr[i];
    }
  }
}

template <typename T, int RQ>
__global__ __launch_bounds__(64) void general_delta_kernel(
    float* __restrict__ out, const void* __restrict__ rp, const void* __restrict__ kp, const void* __restrict__ vp,
    int64_t rkv_stride, const void* __restrict__ decay_pre, int64_t decay_stride, const float* __restrict__ w0,
    const void* __restrict__ rate_pre, int64_t rate_stride, const float* __restrict__ a_bias,
    float* __restrict__ state, const int32_t* __restrict__ q_start, const int32_t* __restrict__ ctx_len,
    const int32_t* __restrict__ state_slot, int heads, int dim) {
  const int lane = threadIdx.x, rg = lane & 3;
  const int col = blockIdx.x * kColsPerWave + (lane >> 2);
  const int h = blockIdx.y, s = blockIdx.z;
  const int first = q_start[s], n = q_start[s + 1] - first;
  if (n == 0) return;
  const bool col_ok = col < dim;
  const int colc = col_ok ? col : dim - 1;
  float* S = state + ((int64_t)state_slot[s] * heads + h) * dim * dim;
  float Sr[RQ], wb[RQ], ab[RQ];
#pragma unroll
  for (int i = 0; i < RQ; ++i) {
    const int r = 4 * i + rg;
    const bool ok = r < dim;
    Sr[i] = (ctx_len[s] > 0 && ok) ? S[(int64_t)r * dim + colc] : 0.0f;
    wb[i] = ok ? w0[h * dim + r] : 0.0f;
    ab[i] = ok ? a_bias[h * dim + r] : 0.0f;
  }
  const float kDecay = 0.60653065971263342f;            // exp(-1/2)
  float rn[RQ], kn[RQ], dn[RQ], an[RQ], vn;
  auto fetch = [&](int t) {
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      const int r = 4 * i + rg;
      const bool ok = r < dim;
      rn[i] = ok ? ld<T>(rp, (int64_t)t * rkv_stride + h * dim + r) : 0.0f;
      kn[i] = ok ? ld<T>(kp, (int64_t)t * rkv_stride + h * dim + r) : 0.0f;
      dn[i] = ok ? ld<T>(decay_pre, (int64_t)t * decay_stride + h * dim + r) : 0.0f;
      an[i] = ok ? ld<T>(rate_pre, (int64_t)t * rate_stride + h * dim + r) : 0.0f;
    }
    vn = ld<T>(vp, (int64_t)t * rkv_stride + h * dim + colc);
  };
  fetch(first);
  for (int t = first; t < first + n; ++t) {
    float r[RQ], k[RQ], w[RQ], a[RQ];
    const float v = vn;
    float kk = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      const bool ok = 4 * i + rg < dim;
      r[i] = rn[i];
      k[i] = kn[i];
      w[i] = expf(-kDecay * sigmoidf_(dn[i] + wb[i]));
      a[i] = ok ? sigmoidf_(an[i] + ab[i]) : 0.0f;
      kk += k[i] * k[i];
    }
    if (t + 1 < first + n) fetch(t + 1);
    kk = group_sum(kk);
    const float kf = 1.0f / sqrtf(kk + 1e-6f);
    float us = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) us += (k[i] * kf) * Sr[i];
    us = group_sum(us);                                  // u^T S of the OLD state
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      Sr[i] = w[i] * Sr[i] - a[i] * (k[i] * kf) * us + k[i] * v;
      o += r[i] * Sr[i];
    }
    o = group_sum(o);
    if (rg == 0 && col_ok) out[((int64_t)t * heads + h) * dim + col] = o;
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < RQ; ++i) {
      const int r = 4 * i + rg;
      if (r < dim) S[(int64_t)r * dim + col] = Sr[i];
    }
  }
}

template <typename T, int RQ>
int launch_channel(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride, const void* decay_pre,
                   const float* dt_bias, const float* a_log, float* state, const int32_t* q_start,
                   const int32_t* ctx_len, const int32_t* state_slot, int num_seqs, int heads, int kv_heads, int dim,
                   int vdim, hipStream_t stream) {
  const dim3 grid((unsigned)((vdim + kColsPerWave - 1) / kColsPerWave), (unsigned)heads, (unsigned)num_seqs);
  hipLaunchKernelGGL((channel_delta_kernel<T, RQ>), grid, dim3(64), 0, stream, out, qkv, beta_pre, beta_stride,
                     decay_pre, dt_bias, a_log, state, q_start, ctx_len, state_slot, heads, kv_heads, dim, vdim);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

template <typename T, int RQ>
int launch_general(float* out, const void* r, const void* k, const void* v, int64_t rkv_stride, const void* decay_pre,
                   int64_t decay_stride, const float* w0, const void* rate_pre, int64_t rate_stride,
                   const float* a_bias, float* state, const int32_t* q_start, const int32_t* ctx_len,
                   const int32_t* state_slot, int num_seqs, int heads, int dim, hipStream_t stream) {
  const dim3 grid((unsigned)((dim + kColsPerWave - 1) / kColsPerWave), (unsigned)heads, (unsigned)num_seqs);
  hipLaunchKernelGGL((general_delta_kernel<T, RQ>), grid, dim3(64), 0, stream, out, r, k, v, rkv_stride, decay_pre,
                     decay_stride, w0, rate_pre, rate_stride, a_bias, state, q_start, ctx_len, state_slot, heads, dim);
  SW_CHECK_LAUNCH();
  return SW_OK;
}

}  // namespace swm

// rows per lane for a key size: 8, 16, 32 or 64 (key sizes up to 256)
#define SWM_DISPATCH_ROWS(dim, ...)                       \
  do {                                                    \
    if ((dim) <= 32) { constexpr int RQ = 8; __VA_ARGS__ }        \
    else if ((dim) <= 64) { constexpr int RQ = 16; __VA_ARGS__ }  \
    else if ((dim) <= 128) { constexpr int RQ = 32; __VA_ARGS__ } \
    else { constexpr int RQ = 64; __VA_ARGS__ }                   \
  } while (0)

extern "C" {

int swm_channel_delta(float* out, const float* qkv, const void* beta_pre, int64_t beta_stride,
                      const void* decay_pre, const float* dt_bias, const float* a_log, float* state,
                      const int32_t* q_start, const int32_t* ctx_len, const int32_t* state_slot,
                      int num_seqs, int heads, int kv_heads, int dim, int vdim, int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "channel_delta: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && dim <= 256 && vdim > 0,
               "channel_delta: heads %d, kv heads %d, key size %d (up to 256), value size %d", heads, kv_heads, dim,
               vdim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_ROWS(dim, return (launch_channel<T, RQ>(
      out, qkv, beta_pre, beta_stride, decay_pre, dt_bias, a_log, state, q_start, ctx_len, state_slot, num_seqs,
      heads, kv_heads, dim, vdim, s));););
  return SW_OK;
}

int swm_general_delta(float* out, const void* r, const void* k, const void* v, int64_t rkv_stride,
                      const void* decay_pre, int64_t decay_stride, const float* w0, const void* rate_pre,
                      int64_t rate_stride, const float* a_bias, float* state, const int32_t* q_start,
                      const int32_t* ctx_len, const int32_t* state_slot, int num_seqs, int heads, int dim,
                      int act_dtype, void* stream) {
  using namespace swm;
  if (num_seqs == 0) return SW_OK;
  SW_CHECK_ARG(act_ok(act_dtype), "general_delta: unsupported dtype %d", act_dtype);
  SW_CHECK_ARG(heads > 0 && dim > 0 && dim <= 256, "general_delta: heads %d, key size %d (up to 256)", heads, dim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  SWM_DISPATCH_ACT(act_dtype, SWM_DISPATCH_ROWS(dim, return (launch_general<T, RQ>(
      out, r, k, v, rkv_stride, decay_pre, decay_stride, w0, rate_pre, rate_stride, a_bias, state, q_start, ctx_len,
      state_slot, num_seqs, heads, dim, s));););
  return SW_OK;
}

}  // extern "C"
