// Linear recurrences with one fp32 matrix per (sequence, head); the plain one:
//     S_t = diag(a_t) S_{t-1} + k_t v_t^T        S [dk, dv]
//     o_t = S_t^T (q_t * q_scale)
// a_t either per key channel and token, a = exp(logsigmoid(z + b) / tau) from gate logits z (fp32), or one number per head,
// or (state-space form) one number per head and token from a step size: dt = softplus(z_t[h] + dt_bias[h]),
// a_t = exp(-exp(rate_log[h]) dt), the write scaled by the same step, S_t = a_t S_{t-1} + dt k_t v_t^T, and a skip term
// skip[h] v_t added to the read-out.  q and k may have fewer heads than v (head h reads q / k head h / (heads / qk_heads)).
//
// One workgroup per (sequence of the step, head, block of 32 value columns): it loads the block's dk x 32 part of the
// sequence's matrix (zero at position 0), runs the step's tokens of that sequence through it in order, and stores it
// back.  A lane owns ONE column and R consecutive key channels of it in registers (8 lanes share a column, a wave holds 8
// columns, the 4 waves 32); per token it does R (mul, fma, fma) and the 8 partial dot products of a column meet over
// three lane exchanges.  q, k and the decays of the next TC tokens are staged in LDS (all fp32 from there on).  A decode
// step is the same launch with one token per sequence; what bounds it then is the matrix's trip through HBM, which each
// workgroup makes in whole 128-byte rows.
#include "common.cuh"

namespace mi355 {
namespace {

constexpr int RC_COLS = 32;   // value columns per workgroup
constexpr int RC_RG = 8;      // lanes that share a column
constexpr int RC_TC = 16;     // tokens staged at a time

__device__ __forceinline__ float log_sigmoid_f(float z) {
  // log(1 / (1 + exp(-z))) without overflow on either side
  return fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
}

__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

template <typename QT, typename VT, int R>
__global__ __launch_bounds__(256) void linear_recurrence_kernel(
    float* __restrict__ out, float* __restrict__ state, const QT* __restrict__ q, const QT* __restrict__ k,
    const VT* __restrict__ v, const float* __restrict__ gate_logits, const VT* __restrict__ gate_bias,
    const float* __restrict__ head_decay, const int32_t* __restrict__ req_to_state, const int64_t* __restrict__ req_pool_indices,
    const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len, const int64_t* __restrict__ positions, int heads,
    int dk, int dv, int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, int64_t gate_token_stride,
    float q_scale, float inv_tau, int qk_heads, const float* __restrict__ dt_logits, int64_t dt_token_stride,
    const float* __restrict__ dt_bias, const float* __restrict__ rate_log, const float* __restrict__ skip) {
  constexpr int DKP = R * RC_RG;     // key channels with padding
  __shared__ float dts[RC_TC], das[RC_TC];
  __shared__ __attribute__((aligned(16))) float qs[RC_TC][DKP];
  __shared__ __attribute__((aligned(16))) float ks[RC_TC][DKP];
  __shared__ __attribute__((aligned(16))) float as[RC_TC][DKP];
  __shared__ float vs[RC_TC][RC_COLS];
  const int b = blockIdx.z, h = blockIdx.y, c0 = blockIdx.x * RC_COLS;
  const int tid = threadIdx.x;
  const int rg = tid & (RC_RG - 1), cl = tid >> 3;       // lane = column * 8 + row group
  const int col = c0 + cl;
  const int64_t t0 = seg_start != nullptr ? seg_start[b] : b;
  const int n = seg_len != nullptr ? seg_len[b] : 1;
  if (n <= 0) return;
  const int64_t slot = req_to_state[req_pool_indices[b]];
  float* sp = state + ((slot * heads + h) * (int64_t)dk) * dv;
  float S[R];
  const bool fresh = positions[t0] == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = rg * R + r;
    S[r] = (!fresh && i < dk && col < dv) ? sp[(int64_t)i * dv + col] : 0.f;
  }
  const float hd = head_decay != nullptr ? head_decay[h] : 1.f;
  const int hq = h / (heads / qk_heads);
  const float rate = dt_logits != nullptr ? expf(rate_log[h]) : 0.f;
  const float skip_h = skip != nullptr ? skip[h] : 0.f;
  for (int base = 0; base < n; base += RC_TC) {
    const int m = min(RC_TC, n - base);
    __syncthreads();
    if (dt_logits != nullptr) {
      if (tid < m) {
        const float dt = softplus_f(dt_logits[(t0 + base + tid) * dt_token_stride + h] + dt_bias[h]);
        dts[tid] = dt;
        das[tid] = expf(-rate * dt);
      }
      __syncthreads();
    }
    for (int e = tid; e < m * DKP; e += 256) {
      const int tt = e / DKP, i = e - tt * DKP;
      const int64_t t = t0 + base + tt;
      float qv = 0.f, kv = 0.f, av = 1.f;
      if (i < dk) {
        qv = to_f32(q[t * q_token_stride + (int64_t)hq * dk + i]) * q_scale;
        kv = to_f32(k[t * k_token_stride + (int64_t)hq * dk + i]);
        if (dt_logits != nullptr) {
          kv *= dts[tt];
          av = das[tt];
        } else if (gate_logits != nullptr) {
          float z = gate_logits[t * gate_token_stride + (int64_t)h * dk + i];
          if (gate_bias != nullptr) z += to_f32(gate_bias[(int64_t)h * dk + i]);
          av = expf(log_sigmoid_f(z) * inv_tau);
        } else {
          av = hd;
        }
      }
      qs[tt][i] = qv;
      ks[tt][i] = kv;
      as[tt][i] = av;
    }
    for (int e = tid; e < m * RC_COLS; e += 256) {
      const int tt = e / RC_COLS, c = e - tt * RC_COLS;
      vs[tt][c] = (c0 + c < dv) ? to_f32(v[(t0 + base + tt) * v_token_stride + (int64_t)h * dv + c0 + c]) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < m; ++tt) {
      const float vj = vs[tt][cl];
      float acc = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R; r4 += 4) {
        const float4 a4 = *reinterpret_cast<const float4*>(&as[tt][rg * R + r4]);
        const float4 k4 = *reinterpret_cast<const float4*>(&ks[tt][rg * R + r4]);
        const float4 q4 = *reinterpret_cast<const float4*>(&qs[tt][rg * R + r4]);
        S[r4 + 0] = fmaf(a4.x, S[r4 + 0], k4.x * vj);
        S[r4 + 1] = fmaf(a4.y, S[r4 + 1], k4.y * vj);
        S[r4 + 2] = fmaf(a4.z, S[r4 + 2], k4.z * vj);
        S[r4 + 3] = fmaf(a4.w, S[r4 + 3], k4.w * vj);
        acc = fmaf(S[r4 + 0], q4.x, acc);
        acc = fmaf(S[r4 + 1], q4.y, acc);
        acc = fmaf(S[r4 + 2], q4.z, acc);
        acc = fmaf(S[r4 + 3], q4.w, acc);
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 4, 64);
      if (rg == 0 && col < dv) out[((t0 + base + tt) * heads + h) * (int64_t)dv + col] = fmaf(skip_h, vj, acc);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = rg * R + r;
    if (i < dk && col < dv) sp[(int64_t)i * dv + col] = S[r];
  }
}

template <typename QT, typename VT>
int launch_recurrence(float* out, float* state, const void* q, const void* k, const void* v, const float* gate_logits,
                      const void* gate_bias, const float* head_decay, const int32_t* req_to_state, const int64_t* req_pool_indices,
                      const int32_t* seg_start, const int32_t* seg_len, const int64_t* positions, int64_t batch, int heads, int dk,
                      int dv, int64_t qs, int64_t ks, int64_t vs, int64_t gs, float q_scale, float tau, int qk_heads, const float* dt_logits,
                      int64_t dts, const float* dt_bias, const float* rate_log, const float* skip, hipStream_t stream) {
  const dim3 grid((unsigned)cdiv(dv, RC_COLS), (unsigned)heads, (unsigned)batch);
#define MI355_RC_LAUNCH(R)                                                                                                     \
  hipLaunchKernelGGL((linear_recurrence_kernel<QT, VT, R>), grid, dim3(256), 0, stream, out, state, (const QT*)q, (const QT*)k, \
                     (const VT*)v, gate_logits, (const VT*)gate_bias, head_decay, req_to_state, req_pool_indices, seg_start,   \
                     seg_len, positions, heads, dk, dv, qs, ks, vs, gs, q_scale, 1.0f / tau, qk_heads, dt_logits, dts, dt_bias,  \
                     rate_log, skip)
  if (dk <= 32) MI355_RC_LAUNCH(4);
  else if (dk <= 64) MI355_RC_LAUNCH(8);
  else if (dk <= 128) MI355_RC_LAUNCH(16);
  else MI355_RC_LAUNCH(32);
#undef MI355_RC_LAUNCH
  return MI355_OK;
}


// Gated delta rule on the same layout: per token
//     S <- diag(a_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T (q_t * q_scale)
// with a_t[i] = exp(-exp(rate_log[h]) * softplus(z_t[h, i] + rate_bias[h, i])) from fp32 logits z and beta_t = sigmoid of a
// logit per head.  With gate_per_head the decay is one number per head and token: z_t[h], rate_bias[h].  beta logits come
// in v's type or (beta_f32) in fp32.  q and k may have fewer heads than v (head h reads q / k head h / (heads / qk_heads)).  A column's
// S^T k and S^T q are each a sum over its eight lanes, so a token costs two rounds of lane exchanges.
template <typename QT, typename VT, int R>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(
    float* __restrict__ out, float* __restrict__ state, const QT* __restrict__ q, const QT* __restrict__ k,
    const VT* __restrict__ v, const VT* __restrict__ beta_logits, const float* __restrict__ gate_logits,
    const float* __restrict__ rate_bias, const float* __restrict__ rate_log, const int32_t* __restrict__ req_to_state,
    const int64_t* __restrict__ req_pool_indices, const int32_t* __restrict__ seg_start, const int32_t* __restrict__ seg_len,
    const int64_t* __restrict__ positions, int heads, int qk_heads, int dk, int dv, int64_t q_token_stride, int64_t k_token_stride,
    int64_t v_token_stride, int64_t beta_token_stride, int64_t gate_token_stride, float q_scale, int gate_per_head, int beta_f32) {
  constexpr int DKP = R * RC_RG;
  __shared__ __attribute__((aligned(16))) float qs[RC_TC][DKP];
  __shared__ __attribute__((aligned(16))) float ks[RC_TC][DKP];
  __shared__ __attribute__((aligned(16))) float as[RC_TC][DKP];
  __shared__ float vs[RC_TC][RC_COLS];
  __shared__ float bs[RC_TC];
  const int b = blockIdx.z, h = blockIdx.y, c0 = blockIdx.x * RC_COLS;
  const int hq = h / (heads / qk_heads);
  const int tid = threadIdx.x;
  const int rg = tid & (RC_RG - 1), cl = tid >> 3;
  const int col = c0 + cl;
  const int64_t t0 = seg_start != nullptr ? seg_start[b] : b;
  const int n = seg_len != nullptr ? seg_len[b] : 1;
  if (n <= 0) return;
  const int64_t slot = req_to_state[req_pool_indices[b]];
  float* sp = state + ((slot * heads + h) * (int64_t)dk) * dv;
  float S[R];
  const bool fresh = positions[t0] == 0;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = rg * R + r;
    S[r] = (!fresh && i < dk && col < dv) ? sp[(int64_t)i * dv + col] : 0.f;
  }
  const float rate = expf(rate_log[h]);
  for (int base = 0; base < n; base += RC_TC) {
    const int m = min(RC_TC, n - base);
    __syncthreads();
    for (int e = tid; e < m * DKP; e += 256) {
      const int tt = e / DKP, i = e - tt * DKP;
      const int64_t t = t0 + base + tt;
      float qv = 0.f, kv = 0.f, av = 1.f;
      if (i < dk) {
        qv = to_f32(q[t * q_token_stride + (int64_t)hq * dk + i]) * q_scale;
        kv = to_f32(k[t * k_token_stride + (int64_t)hq * dk + i]);
        const int64_t gi = gate_per_head ? h : (int64_t)h * dk + i;
        const float z = gate_logits[t * gate_token_stride + gi] + rate_bias[gi];
        av = expf(-rate * softplus_f(z));
      }
      qs[tt][i] = qv;
      ks[tt][i] = kv;
      as[tt][i] = av;
    }
    for (int e = tid; e < m * RC_COLS; e += 256) {
      const int tt = e / RC_COLS, c = e - tt * RC_COLS;
      vs[tt][c] = (c0 + c < dv) ? to_f32(v[(t0 + base + tt) * v_token_stride + (int64_t)h * dv + c0 + c]) : 0.f;
    }
    if (tid < m) {
      const int64_t bi = (t0 + base + tid) * beta_token_stride + h;
      const float bl = beta_f32 ? reinterpret_cast<const float*>(beta_logits)[bi] : to_f32(beta_logits[bi]);
      bs[tid] = 1.0f / (1.0f + expf(-bl));
    }
    __syncthreads();
    for (int tt = 0; tt < m; ++tt) {
      float dot = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R; r4 += 4) {
        const float4 a4 = *reinterpret_cast<const float4*>(&as[tt][rg * R + r4]);
        const float4 k4 = *reinterpret_cast<const float4*>(&ks[tt][rg * R + r4]);
        S[r4 + 0] *= a4.x;
        S[r4 + 1] *= a4.y;
        S[r4 + 2] *= a4.z;
        S[r4 + 3] *= a4.w;
        dot = fmaf(S[r4 + 0], k4.x, dot);
        dot = fmaf(S[r4 + 1], k4.y, dot);
        dot = fmaf(S[r4 + 2], k4.z, dot);
        dot = fmaf(S[r4 + 3], k4.w, dot);
      }
      dot += __shfl_xor(dot, 1, 64);
      dot += __shfl_xor(dot, 2, 64);
      dot += __shfl_xor(dot, 4, 64);
      const float u = bs[tt] * (vs[tt][cl] - dot);
      float acc = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R; r4 += 4) {
        const float4 k4 = *reinterpret_cast<const float4*>(&ks[tt][rg * R + r4]);
        const float4 q4 = *reinterpret_cast<const float4*>(&qs[tt][rg * R + r4]);
        S[r4 + 0] = fmaf(k4.x, u, S[r4 + 0]);
        S[r4 + 1] = fmaf(k4.y, u, S[r4 + 1]);
        S[r4 + 2] = fmaf(k4.z, u, S[r4 + 2]);
        S[r4 + 3] = fmaf(k4.w, u, S[r4 + 3]);
        acc = fmaf(S[r4 + 0], q4.x, acc);
        acc = fmaf(S[r4 + 1], q4.y, acc);
        acc = fmaf(S[r4 + 2], q4.z, acc);
        acc = fmaf(S[r4 + 3], q4.w, acc);
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 4, 64);
      if (rg == 0 && col < dv) out[((t0 + base + tt) * heads + h) * (int64_t)dv + col] = acc;
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = rg * R + r;
    if (i < dk && col < dv) sp[(int64_t)i * dv + col] = S[r];
  }
}

template <typename QT, typename VT>
int launch_delta(float* out, float* state, const void* q, const void* k, const void* v, const void* beta_logits,
                 const float* gate_logits, const float* rate_bias, const float* rate_log, const int32_t* req_to_state,
                 const int64_t* req_pool_indices, const int32_t* seg_start, const int32_t* seg_len, const int64_t* positions,
                 int64_t batch, int heads, int qk_heads, int dk, int dv, int64_t qs, int64_t ks, int64_t vs, int64_t bs, int64_t gs,
                 float q_scale, int gate_per_head, int beta_f32, hipStream_t stream) {
  const dim3 grid((unsigned)cdiv(dv, RC_COLS), (unsigned)heads, (unsigned)batch);
#define MI355_GD_LAUNCH(R)                                                                                                     \
  hipLaunchKernelGGL((gated_delta_rule_kernel<QT, VT, R>), grid, dim3(256), 0, stream, out, state, (const QT*)q, (const QT*)k,  \
                     (const VT*)v, (const VT*)beta_logits, gate_logits, rate_bias, rate_log, req_to_state, req_pool_indices,   \
                     seg_start, seg_len, positions, heads, qk_heads, dk, dv, qs, ks, vs, bs, gs, q_scale, gate_per_head, beta_f32)
  if (dk <= 32) MI355_GD_LAUNCH(4);
  else if (dk <= 64) MI355_GD_LAUNCH(8);
  else if (dk <= 128) MI355_GD_LAUNCH(16);
  else MI355_GD_LAUNCH(32);
#undef MI355_GD_LAUNCH
  return MI355_OK;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_linear_recurrence(float* out, float* state, const void* q, const void* k, const void* v, const float* gate_logits,
                            const void* gate_bias, const float* head_decay, const int32_t* req_to_state,
                            const int64_t* req_pool_indices, const int32_t* seg_start, const int32_t* seg_len,
                            const int64_t* positions, int64_t batch, int heads, int key_dim, int value_dim, int64_t q_token_stride,
                            int64_t k_token_stride, int64_t v_token_stride, int64_t gate_token_stride, float q_scale, float tau,
                            int qk_dtype, int v_dtype, void* stream) {
  MI355_REQUIRE((gate_logits != nullptr) != (head_decay != nullptr), MI355_ERR_INVALID,
                "linear_recurrence: the decay is either gate logits per channel or one number per head");
  return mi355_linear_recurrence_ssm(out, state, q, k, v, gate_logits, gate_bias, head_decay, nullptr, 0, nullptr, nullptr, nullptr,
                                     req_to_state, req_pool_indices, seg_start, seg_len, positions, batch, heads, heads, key_dim,
                                     value_dim, q_token_stride, k_token_stride, v_token_stride, gate_token_stride, q_scale, tau,
                                     qk_dtype, v_dtype, stream);
}

int mi355_linear_recurrence_ssm(float* out, float* state, const void* q, const void* k, const void* v, const float* gate_logits,
                                const void* gate_bias, const float* head_decay, const float* dt_logits, int64_t dt_token_stride,
                                const float* dt_bias, const float* rate_log, const float* skip, const int32_t* req_to_state,
                                const int64_t* req_pool_indices, const int32_t* seg_start, const int32_t* seg_len,
                                const int64_t* positions, int64_t batch, int heads, int qk_heads, int key_dim, int value_dim,
                                int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, int64_t gate_token_stride,
                                float q_scale, float tau, int qk_dtype, int v_dtype, void* stream) {
  MI355_REQUIRE(out && state && q && k && v && req_to_state && req_pool_indices && positions, MI355_ERR_INVALID,
                "linear_recurrence: null pointer");
  MI355_REQUIRE((gate_logits != nullptr) + (head_decay != nullptr) + (dt_logits != nullptr) == 1, MI355_ERR_INVALID,
                "linear_recurrence: the decay is gate logits per channel, one number per head, or a step size per head and token");
  MI355_REQUIRE(dt_logits == nullptr || (dt_bias && rate_log && dt_token_stride >= heads), MI355_ERR_INVALID,
                "linear_recurrence: step sizes come with their bias and the heads' rates");
  MI355_REQUIRE((seg_start == nullptr) == (seg_len == nullptr), MI355_ERR_INVALID,
                "linear_recurrence: seg_start and seg_len come together");
  MI355_REQUIRE(batch >= 0 && batch <= 65535 && heads > 0 && heads <= 65535 && key_dim > 0 && value_dim > 0 && tau > 0.f &&
                    qk_heads > 0 && heads % qk_heads == 0, MI355_ERR_INVALID, "linear_recurrence: bad shape");
  MI355_REQUIRE(key_dim <= 256, MI355_ERR_UNSUPPORTED, "linear_recurrence: key width %d above 256", key_dim);
  MI355_REQUIRE(qk_dtype == v_dtype || qk_dtype == MI355_F32, MI355_ERR_UNSUPPORTED,
                "linear_recurrence: q and k come in the type of v or in fp32");
  if (batch == 0) return MI355_OK;
  int rc = MI355_OK;
  MI355_DISPATCH_DTYPE(v_dtype, "linear_recurrence", {
    if (qk_dtype == v_dtype)
      rc = launch_recurrence<T, T>(out, state, q, k, v, gate_logits, gate_bias, head_decay, req_to_state, req_pool_indices,
                                   seg_start, seg_len, positions, batch, heads, key_dim, value_dim, q_token_stride, k_token_stride,
                                   v_token_stride, gate_token_stride, q_scale, tau, qk_heads, dt_logits, dt_token_stride, dt_bias,
                                   rate_log, skip, (hipStream_t)stream);
    else
      rc = launch_recurrence<float, T>(out, state, q, k, v, gate_logits, gate_bias, head_decay, req_to_state, req_pool_indices,
                                       seg_start, seg_len, positions, batch, heads, key_dim, value_dim, q_token_stride,
                                       k_token_stride, v_token_stride, gate_token_stride, q_scale, tau, qk_heads, dt_logits,
                                       dt_token_stride, dt_bias, rate_log, skip, (hipStream_t)stream);
  });
  if (rc != MI355_OK) return rc;
  MI355_CHECK_LAUNCH("linear_recurrence");
  return MI355_OK;
}

int mi355_gated_delta_rule(float* out, float* state, const void* q, const void* k, const void* v, const void* beta_logits,
                           const float* gate_logits, const float* rate_bias, const float* rate_log, const int32_t* req_to_state,
                           const int64_t* req_pool_indices, const int32_t* seg_start, const int32_t* seg_len,
                           const int64_t* positions, int64_t batch, int heads, int qk_heads, int key_dim, int value_dim,
                           int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, int64_t beta_token_stride,
                           int64_t gate_token_stride, float q_scale, int qk_dtype, int v_dtype, void* stream) {
  return mi355_gated_delta_rule_ex(out, state, q, k, v, beta_logits, gate_logits, rate_bias, rate_log, req_to_state, req_pool_indices,
                                   seg_start, seg_len, positions, batch, heads, qk_heads, key_dim, value_dim, q_token_stride,
                                   k_token_stride, v_token_stride, beta_token_stride, gate_token_stride, q_scale, 0, 0, qk_dtype,
                                   v_dtype, stream);
}

int mi355_gated_delta_rule_ex(float* out, float* state, const void* q, const void* k, const void* v, const void* beta_logits,
                              const float* gate_logits, const float* rate_bias, const float* rate_log, const int32_t* req_to_state,
                              const int64_t* req_pool_indices, const int32_t* seg_start, const int32_t* seg_len,
                              const int64_t* positions, int64_t batch, int heads, int qk_heads, int key_dim, int value_dim,
                              int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, int64_t beta_token_stride,
                              int64_t gate_token_stride, float q_scale, int gate_per_head, int beta_f32, int qk_dtype, int v_dtype,
                              void* stream) {
  MI355_REQUIRE(out && state && q && k && v && beta_logits && gate_logits && rate_bias && rate_log && req_to_state &&
                    req_pool_indices && positions, MI355_ERR_INVALID, "gated_delta_rule: null pointer");
  MI355_REQUIRE((seg_start == nullptr) == (seg_len == nullptr), MI355_ERR_INVALID,
                "gated_delta_rule: seg_start and seg_len come together");
  MI355_REQUIRE(batch >= 0 && batch <= 65535 && heads > 0 && heads <= 65535 && qk_heads > 0 && heads % qk_heads == 0 &&
                    key_dim > 0 && value_dim > 0, MI355_ERR_INVALID, "gated_delta_rule: bad shape");
  MI355_REQUIRE(key_dim <= 256, MI355_ERR_UNSUPPORTED, "gated_delta_rule: key width %d above 256", key_dim);
  MI355_REQUIRE(qk_dtype == v_dtype || qk_dtype == MI355_F32, MI355_ERR_UNSUPPORTED,
                "gated_delta_rule: q and k come in the type of v or in fp32");
  if (batch == 0) return MI355_OK;
  int rc = MI355_OK;
  MI355_DISPATCH_DTYPE(v_dtype, "gated_delta_rule", {
    if (qk_dtype == v_dtype)
      rc = launch_delta<T, T>(out, state, q, k, v, beta_logits, gate_logits, rate_bias, rate_log, req_to_state, req_pool_indices,
                              seg_start, seg_len, positions, batch, heads, qk_heads, key_dim, value_dim, q_token_stride,
                              k_token_stride, v_token_stride, beta_token_stride, gate_token_stride, q_scale, gate_per_head, beta_f32,
                              (hipStream_t)stream);
    else
      rc = launch_delta<float, T>(out, state, q, k, v, beta_logits, gate_logits, rate_bias, rate_log, req_to_state,
                                  req_pool_indices, seg_start, seg_len, positions, batch, heads, qk_heads, key_dim, value_dim,
                                  q_token_stride, k_token_stride, v_token_stride, beta_token_stride, gate_token_stride, q_scale,
                                  gate_per_head, beta_f32, (hipStream_t)stream);
  });
  if (rc != MI355_OK) return rc;
  MI355_CHECK_LAUNCH("gated_delta_rule");
  return MI355_OK;
}
