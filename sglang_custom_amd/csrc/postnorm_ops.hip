// Kernels around a 32-bit residual stream that is normed AFTER every residual sum:
//   * x <- N(alpha x + branch) * w, N an RMS norm over equal consecutive groups of the row; the branch is a row of a
//     tensor or a weighted sum of rows picked by an index list (the outputs of a token's experts); the kernel also
//     writes the activation-dtype copy of the new row,
//   * x <- x + y / rms(y) * w with the same second output,
//   * per (token, head): optional RMS norm with a weight shared by the heads, rotation of the leading features by
//     position-dependent angles in either pairing, a scale; to a tensor or straight into cache rows,
//   * per (token, head): fp32 row / rms(row) (* weight) * silu(gate) in the activation dtype,
//   * gelu_tanh(gate) * table[id][column window].
// Every reduction, normalisation, angle and gate runs in fp32 whatever the activation dtype T is.
#include "common.cuh"

#include <algorithm>

namespace mi355 {
namespace {

__device__ __forceinline__ float pn_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float pn_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// Eight consecutive features of a row of T: one 16-byte load for 16-bit types, two for fp32.
template <typename T> __device__ __forceinline__ Vec<T, 8> ld_row8(const T* p) {
  if constexpr (sizeof(T) == 2) {
    return ldvec<T, 8>(p);
  } else {
    Vec<T, 8> r;
    const Vec<T, 4> a = ldvec<T, 4>(p), b = ldvec<T, 4>(p + 4);
#pragma unroll
    for (int k = 0; k < 4; ++k) { r.v[k] = a.v[k]; r.v[4 + k] = b.v[k]; }
    return r;
  }
}

// One workgroup per token.  sm holds the row (D floats) and then one 1/rms per group.
template <typename T>
__global__ __launch_bounds__(256) void scaled_add_group_rmsnorm_kernel(
    float* x_out, T* __restrict__ h_out, const float* x, const T* __restrict__ branch,
    int64_t branch_stride, const int32_t* __restrict__ rows, const float* __restrict__ coef, int n_branch, float alpha,
    const T* __restrict__ w, int64_t D, int groups, float eps, bool vec8) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  __shared__ float red[16];
  float* row = sm;
  float* inv = sm + D;
  const int64_t t = blockIdx.x;
  if (vec8) {
    // eight features per thread and access: 16-byte loads of the branch rows, two of the fp32 row
    for (int64_t i = 8 * threadIdx.x; i < D; i += 8 * blockDim.x) {
      const float4 x0 = *reinterpret_cast<const float4*>(x + t * D + i), x1 = *reinterpret_cast<const float4*>(x + t * D + i + 4);
      float s[8] = {alpha * x0.x, alpha * x0.y, alpha * x0.z, alpha * x0.w, alpha * x1.x, alpha * x1.y, alpha * x1.z, alpha * x1.w};
      if (branch != nullptr) {
        if (rows == nullptr) {
          const Vec<T, 8> b = ld_row8<T>(branch + t * branch_stride + i);
#pragma unroll
          for (int k = 0; k < 8; ++k) s[k] += to_f32(b.v[k]);
        } else {
          float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          for (int j = 0; j < n_branch; ++j) {      // fixed order: the sum does not depend on where the rows lie
            const float c = coef[t * n_branch + j];
            const Vec<T, 8> b = ld_row8<T>(branch + (int64_t)rows[t * n_branch + j] * branch_stride + i);
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[k] += c * to_f32(b.v[k]);
          }
#pragma unroll
          for (int k = 0; k < 8; ++k) s[k] += acc[k];
        }
      }
#pragma unroll
      for (int k = 0; k < 8; ++k) row[i + k] = s[k];
    }
  } else {
    for (int64_t i = threadIdx.x; i < D; i += blockDim.x) {
      float s = alpha * x[t * D + i];
      if (branch != nullptr) {
        if (rows == nullptr) {
          s += to_f32(branch[t * branch_stride + i]);
        } else {
          float b = 0.f;
          for (int j = 0; j < n_branch; ++j)      // fixed order: the sum does not depend on where the rows lie
            b += coef[t * n_branch + j] * to_f32(branch[(int64_t)rows[t * n_branch + j] * branch_stride + i]);
          s += b;
        }
      }
      row[i] = s;
    }
  }
  __syncthreads();
  const int64_t gs = D / groups;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, nw = blockDim.x >> 6;
  if (groups >= nw) {
    for (int g = wv; g < groups; g += nw) {
      float q = 0.f;
      for (int64_t i = lane; i < gs; i += 64) q += row[g * gs + i] * row[g * gs + i];
      q = wave_sum(q);
      if (lane == 0) inv[g] = 1.0f / sqrtf(q / (float)gs + eps);
    }
    __syncthreads();
  } else {
    for (int g = 0; g < groups; ++g) {
      float q = 0.f;
      for (int64_t i = threadIdx.x; i < gs; i += blockDim.x) q += row[g * gs + i] * row[g * gs + i];
      q = block_sum(q, red);
      if (threadIdx.x == 0) inv[g] = 1.0f / sqrtf(q / (float)gs + eps);
    }
    __syncthreads();
  }
  for (int64_t i = threadIdx.x; i < D; i += blockDim.x) {
    const float y = row[i] * inv[i / gs] * to_f32(w[i]);
    if (x_out != nullptr) x_out[t * D + i] = y;
    if (h_out != nullptr) h_out[t * D + i] = from_f32<T>(y);
  }
}

// One workgroup per token: x[t] += mult * ls * y[t] / sqrt(mean(y[t]^2) + eps) * (offset + w)   (ls null: ones).  VEC: eight
// features per access (16-byte loads of y, w and ls, two 16-byte loads and stores of the fp32 row, 16-byte stores of the
// copy); the second pass over y finds it in the cache.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rmsnorm_residual_add_kernel(float* __restrict__ x, T* __restrict__ h_out,
                                                                   const T* __restrict__ y, int64_t y_stride,
                                                                   const T* __restrict__ w, const T* __restrict__ ls, float offset,
                                                                   float mult, int64_t D, float eps) {
  __shared__ float red[16];
  constexpr int W = VEC ? 8 : 1;
  const int64_t t = blockIdx.x;
  float q = 0.f;
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
    const Vec<T, W> v = ldvec<T, W>(y + t * y_stride + i);
#pragma unroll
    for (int k = 0; k < W; ++k) q += to_f32(v.v[k]) * to_f32(v.v[k]);
  }
  q = block_sum(q, red);
  const float inv = 1.0f / sqrtf(q / (float)D + eps);
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
    const Vec<T, W> v = ldvec<T, W>(y + t * y_stride + i);
    const Vec<T, W> wv = ldvec<T, W>(w + i);
    Vec<T, W> lv;
    if (ls != nullptr) lv = ldvec<T, W>(ls + i);
    float r[W];
    if constexpr (VEC) {
      const float4 a = *reinterpret_cast<const float4*>(x + t * D + i), b = *reinterpret_cast<const float4*>(x + t * D + i + 4);
      r[0] = a.x; r[1] = a.y; r[2] = a.z; r[3] = a.w; r[4] = b.x; r[5] = b.y; r[6] = b.z; r[7] = b.w;
    } else {
      r[0] = x[t * D + i];
    }
    Vec<T, W> hv;
#pragma unroll
    for (int k = 0; k < W; ++k) {
      float n = to_f32(v.v[k]) * inv * (offset + to_f32(wv.v[k]));
      if (ls != nullptr) n *= to_f32(lv.v[k]);
      r[k] += mult * n;
      hv.v[k] = from_f32<T>(r[k]);
    }
    if constexpr (VEC) {
      *reinterpret_cast<float4*>(x + t * D + i) = make_float4(r[0], r[1], r[2], r[3]);
      *reinterpret_cast<float4*>(x + t * D + i + 4) = make_float4(r[4], r[5], r[6], r[7]);
    } else {
      x[t * D + i] = r[0];
    }
    if (h_out != nullptr) stvec<T, W>(h_out + t * D + i, hv);
  }
}

// One wave per (token, head); four per workgroup.  sm: 4 rows of d floats.
template <typename T, typename OT>
__global__ __launch_bounds__(256) void head_norm_rope_kernel(
    OT* __restrict__ out, const T* __restrict__ src, const T* __restrict__ w, const int64_t* __restrict__ positions,
    const int64_t* __restrict__ loc, const float* __restrict__ inv_freq, int64_t tokens, int heads, int d, int64_t src_token_stride,
    int64_t src_head_stride, int64_t out_token_stride, int64_t out_head_stride, int rot_dims, int interleaved, float scale,
    float eps, float rot_mag) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t idx = (int64_t)blockIdx.x * 4 + wv;
  const bool valid = idx < tokens * heads;
  const int64_t t = valid ? idx / heads : 0;
  const int h = valid ? (int)(idx - t * heads) : 0;
  float* row = sm + (int64_t)wv * d;
  const T* s = src + t * src_token_stride + (int64_t)h * src_head_stride;
  float q = 0.f;
  if (valid) {
    for (int i = lane; i < d; i += 64) {
      const float v = to_f32(s[i]);
      row[i] = v;
      q += v * v;
    }
  }
  float inv = 1.0f;
  if (w != nullptr) {
    q = wave_sum(q);
    inv = 1.0f / sqrtf(q / (float)d + eps);
  }
  __syncthreads();
  if (!valid) return;
  const float pos = (float)positions[t];
  const int64_t orow = loc != nullptr ? loc[t] : t;
  OT* o = out + orow * out_token_stride + (int64_t)h * out_head_stride;
  const int half = rot_dims / 2;
  for (int i = lane; i < d; i += 64) {
    float v = row[i] * inv * (w != nullptr ? to_f32(w[i]) : 1.0f);
    if (i < rot_dims) {
      int pair, partner;
      bool second;
      if (interleaved) {
        pair = i >> 1;
        second = (i & 1) != 0;
        partner = i ^ 1;
      } else {
        second = i >= half;
        pair = second ? i - half : i;
        partner = second ? i - half : i + half;
      }
      const float u = row[partner] * inv * (w != nullptr ? to_f32(w[partner]) : 1.0f);
      float sn, cs;
      sincosf(pos * inv_freq[pair], &sn, &cs);
      sn *= rot_mag;
      cs *= rot_mag;
      // (a, b) -> (a cos - b sin, b cos + a sin): v is a for the first of the pair, b for the second
      v = second ? v * cs + u * sn : v * cs - u * sn;
    }
    o[i] = from_f32<OT>(v * scale);
  }
}

// The three head norms of an attention layer in one launch.  One wave per (token, unit), unit = a query head (RMS norm with
// wq, rotation, to q_out [tokens, heads, d]), a key head (RMS norm with wk, rotation, into k_cache[loc[t]]) or a value head
// (division by its root mean square alone, into v_cache[loc[t]]); the arithmetic per row is head_norm_rope_kernel's.
// sm: 4 rows of max(d, dv) floats.
template <typename T>
__global__ __launch_bounds__(256) void qkv_norm_rope_write_kernel(
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, const T* __restrict__ wq,
    const T* __restrict__ wk, const int64_t* __restrict__ positions, const int64_t* __restrict__ loc,
    const float* __restrict__ inv_freq, int64_t tokens, int heads, int kv_heads, int d, int dv, int rot_dims, int interleaved,
    float eps, float rot_mag) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int units = heads + 2 * kv_heads;
  const int64_t idx = (int64_t)blockIdx.x * 4 + wv;
  const bool valid = idx < tokens * units;
  const int64_t t = valid ? idx / units : 0;
  const int u = valid ? (int)(idx - t * units) : 0;
  const T* s;
  const T* w;
  T* o;
  int width, rot;
  if (u < heads) {
    s = q + t * q_token_stride + (int64_t)u * d; w = wq; width = d; rot = rot_dims;
    o = q_out + (t * heads + u) * (int64_t)d;
  } else if (u < heads + kv_heads) {
    const int g = u - heads;
    s = k + t * k_token_stride + (int64_t)g * d; w = wk; width = d; rot = rot_dims;
    o = k_cache + (loc[t] * kv_heads + g) * (int64_t)d;
  } else {
    const int g = u - heads - kv_heads;
    s = v + t * v_token_stride + (int64_t)g * dv; w = nullptr; width = dv; rot = 0;
    o = v_cache + (loc[t] * kv_heads + g) * (int64_t)dv;
  }
  float* row = sm + (int64_t)wv * max(d, dv);
  float qs = 0.f;
  if (valid) {
    for (int i = lane; i < width; i += 64) {
      const float x = to_f32(s[i]);
      row[i] = x;
      qs += x * x;
    }
  }
  qs = wave_sum(qs);
  const float inv = 1.0f / sqrtf(qs / (float)width + eps);
  __syncthreads();
  if (!valid) return;
  const float pos = (float)positions[t];
  const int half = rot / 2;
  for (int i = lane; i < width; i += 64) {
    float x = row[i] * inv * (w != nullptr ? to_f32(w[i]) : 1.0f);
    if (i < rot) {
      int pair, partner;
      bool second;
      if (interleaved) {
        pair = i >> 1;
        second = (i & 1) != 0;
        partner = i ^ 1;
      } else {
        second = i >= half;
        pair = second ? i - half : i;
        partner = second ? i - half : i + half;
      }
      const float y = row[partner] * inv * (w != nullptr ? to_f32(w[partner]) : 1.0f);
      float sn, cs;
      sincosf(pos * inv_freq[pair], &sn, &cs);
      sn *= rot_mag;
      cs *= rot_mag;
      x = second ? x * cs + y * sn : x * cs - y * sn;
    }
    o[i] = from_f32<T>(x);
  }
}

// One workgroup per (token, part): out = N(y * silu(gate)) * w over one of `groups` equal consecutive parts of the row, the
// gate applied BEFORE the norm.  y fp32 [tokens, D] contiguous, gate T row-strided, w T [D].  A part of up to 2048 features
// keeps its gated values in registers between the two passes.
constexpr int GGN_KEEP = 8;
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ y,
                                                                  const T* __restrict__ gate, int64_t gate_stride,
                                                                  const T* __restrict__ w, int64_t D, int groups, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x / groups;
  const int part = (int)(blockIdx.x - t * groups);
  const int64_t n = D / groups, c0 = (int64_t)part * n;
  const float* yr = y + t * D + c0;
  const T* gr = gate + t * gate_stride + c0;
  float keep[GGN_KEEP];
  float q = 0.f;
#pragma unroll
  for (int u = 0; u < GGN_KEEP; ++u) {
    const int64_t i = threadIdx.x + 256 * u;
    float v = 0.f;
    if (i < n) {
      const float z = to_f32(gr[i]);
      v = yr[i] * (z * pn_sigmoid(z));
    }
    keep[u] = v;
    q += v * v;
  }
  for (int64_t i = threadIdx.x + 256 * GGN_KEEP; i < n; i += 256) {
    const float z = to_f32(gr[i]);
    const float v = yr[i] * (z * pn_sigmoid(z));
    q += v * v;
  }
  q = block_sum(q, red);
  const float inv = 1.0f / sqrtf(q / (float)n + eps);
#pragma unroll
  for (int u = 0; u < GGN_KEEP; ++u) {
    const int64_t i = threadIdx.x + 256 * u;
    if (i < n) out[t * D + c0 + i] = from_f32<T>(keep[u] * inv * to_f32(w[c0 + i]));
  }
  for (int64_t i = threadIdx.x + 256 * GGN_KEEP; i < n; i += 256) {
    const float z = to_f32(gr[i]);
    out[t * D + c0 + i] = from_f32<T>(yr[i] * (z * pn_sigmoid(z)) * inv * to_f32(w[c0 + i]));
  }
}

// One wave per (token, head): out = o / rms(o) (* w) * silu(gate), or * sigmoid(gate) with gate_act 1
template <typename T>
__global__ __launch_bounds__(256) void head_rmsnorm_gate_kernel(T* __restrict__ out, const float* __restrict__ o,
                                                                const T* __restrict__ w, const T* __restrict__ gate,
                                                                int64_t gate_stride, int64_t tokens, int heads, int dv, float eps,
                                                                int gate_act) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t idx = (int64_t)blockIdx.x * 4 + wv;
  if (idx >= tokens * heads) return;
  const int64_t t = idx / heads;
  const int h = (int)(idx - t * heads);
  const float* r = o + idx * dv;
  float q = 0.f;
  for (int i = lane; i < dv; i += 64) q += r[i] * r[i];
  q = wave_sum(q);
  const float inv = 1.0f / sqrtf(q / (float)dv + eps);
  const T* g = gate + t * gate_stride + (int64_t)h * dv;
  T* dst = out + idx * dv;
  for (int i = lane; i < dv; i += 64) {
    const float z = to_f32(g[i]);
    const float n = r[i] * inv * (w != nullptr ? to_f32(w[i]) : 1.0f);
    dst[i] = from_f32<T>(gate_act == 1 ? n * pn_sigmoid(z) : n * z * pn_sigmoid(z));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gelu_tanh_mul_rows_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                                                 int64_t gate_stride, const T* __restrict__ table,
                                                                 int64_t table_stride, int64_t col_off,
                                                                 const int64_t* __restrict__ ids, int64_t rows, int64_t d) {
  const int64_t n = rows * d;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / d, i = idx - r * d;
    out[idx] = from_f32<T>(pn_gelu_tanh(to_f32(gate[r * gate_stride + i])) * to_f32(table[ids[r] * table_stride + col_off + i]));
  }
}


// One workgroup per token: h = x / sqrt(mean(x^2) + eps) * (offset + w).  VEC: eight features per access (two 16-byte loads
// of the fp32 row, 16-byte weight loads and stores); the second pass over the row finds it in the cache.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void offset_rmsnorm_kernel(T* __restrict__ h, const float* __restrict__ x, const T* __restrict__ w,
                                                             int64_t D, float eps, float offset) {
  __shared__ float red[16];
  constexpr int W = VEC ? 8 : 1;
  const int64_t t = blockIdx.x;
  float q = 0.f;
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
    if constexpr (VEC) {
      const float4 a = *reinterpret_cast<const float4*>(x + t * D + i), b = *reinterpret_cast<const float4*>(x + t * D + i + 4);
      q += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
    } else {
      const float v = x[t * D + i];
      q += v * v;
    }
  }
  q = block_sum(q, red);
  const float inv = 1.0f / sqrtf(q / (float)D + eps);
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
    if constexpr (VEC) {
      const float4 a = *reinterpret_cast<const float4*>(x + t * D + i), b = *reinterpret_cast<const float4*>(x + t * D + i + 4);
      const float xs[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
      const Vec<T, 8> wv = ld_row8<T>(w + i);
      if constexpr (sizeof(T) == 2) {
        Vec<T, 8> o;
#pragma unroll
        for (int k = 0; k < 8; ++k) o.v[k] = from_f32<T>(xs[k] * inv * (offset + to_f32(wv.v[k])));
        stvec<T, 8>(h + t * D + i, o);
      } else {
#pragma unroll
        for (int k = 0; k < 8; ++k) h[t * D + i + k] = from_f32<T>(xs[k] * inv * (offset + to_f32(wv.v[k])));
      }
    } else {
      h[t * D + i] = from_f32<T>(x[t * D + i] * inv * (offset + to_f32(w[i])));
    }
  }
}

// One workgroup per token:  x[t] += s * (A + B) + F,  A = a / rms(a) * wa (wa null: a as it is), B likewise (b null: none),
// F = f[t], or the sum over j of coef[t][j] * f[rows[t][j]] in that order, or nothing.  VEC: rows move as 16-byte vectors of
// eight 16-bit (two vectors of four fp32) features; the second pass over a and b finds them in the cache.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void branch_residual_add_kernel(
    float* __restrict__ x, const T* __restrict__ a, int64_t a_stride, const T* __restrict__ wa, const T* __restrict__ b,
    int64_t b_stride, const T* __restrict__ wb, float s, const T* __restrict__ f, int64_t f_stride, const int32_t* __restrict__ rows,
    const float* __restrict__ coef, int n_branch, int64_t D, float eps) {
  __shared__ float red[16];
  constexpr int W = VEC ? 8 : 1;
  const int64_t t = blockIdx.x;
  float inv_a = 1.f, inv_b = 1.f;
  if (wa != nullptr) {
    float q = 0.f;
    for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
      if constexpr (VEC) {
        const Vec<T, 8> v = ld_row8<T>(a + t * a_stride + i);
#pragma unroll
        for (int k = 0; k < 8; ++k) q += to_f32(v.v[k]) * to_f32(v.v[k]);
      } else {
        const float v = to_f32(a[t * a_stride + i]);
        q += v * v;
      }
    }
    q = block_sum(q, red);
    inv_a = 1.0f / sqrtf(q / (float)D + eps);
  }
  if (b != nullptr && wb != nullptr) {
    float q = 0.f;
    for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
      if constexpr (VEC) {
        const Vec<T, 8> v = ld_row8<T>(b + t * b_stride + i);
#pragma unroll
        for (int k = 0; k < 8; ++k) q += to_f32(v.v[k]) * to_f32(v.v[k]);
      } else {
        const float v = to_f32(b[t * b_stride + i]);
        q += v * v;
      }
    }
    q = block_sum(q, red);
    inv_b = 1.0f / sqrtf(q / (float)D + eps);
  }
  for (int64_t i = W * threadIdx.x; i < D; i += W * blockDim.x) {
    float m[W];
    Vec<T, W> va, vb, vwa, vwb, vf;
    if constexpr (VEC) {
      va = ld_row8<T>(a + t * a_stride + i);
      if (wa != nullptr) vwa = ld_row8<T>(wa + i);
      if (b != nullptr) vb = ld_row8<T>(b + t * b_stride + i);
      if (wb != nullptr) vwb = ld_row8<T>(wb + i);
    } else {
      va.v[0] = a[t * a_stride + i];
      if (wa != nullptr) vwa.v[0] = wa[i];
      if (b != nullptr) vb.v[0] = b[t * b_stride + i];
      if (wb != nullptr) vwb.v[0] = wb[i];
    }
#pragma unroll
    for (int k = 0; k < W; ++k) {
      float v = to_f32(va.v[k]) * inv_a * (wa != nullptr ? to_f32(vwa.v[k]) : 1.f);
      if (b != nullptr) v += to_f32(vb.v[k]) * inv_b * (wb != nullptr ? to_f32(vwb.v[k]) : 1.f);
      m[k] = v * s;
    }
    if (f != nullptr) {
      if (rows == nullptr) {
        if constexpr (VEC) vf = ld_row8<T>(f + t * f_stride + i); else vf.v[0] = f[t * f_stride + i];
#pragma unroll
        for (int k = 0; k < W; ++k) m[k] += to_f32(vf.v[k]);
      } else {
        float e[W];
#pragma unroll
        for (int k = 0; k < W; ++k) e[k] = 0.f;
        for (int j = 0; j < n_branch; ++j) {        // fixed order: the sum does not depend on where the rows lie
          const float cj = coef[t * n_branch + j];
          const T* fr = f + (int64_t)rows[t * n_branch + j] * f_stride + i;
          if constexpr (VEC) vf = ld_row8<T>(fr); else vf.v[0] = fr[0];
#pragma unroll
          for (int k = 0; k < W; ++k) e[k] += cj * to_f32(vf.v[k]);
        }
#pragma unroll
        for (int k = 0; k < W; ++k) m[k] += e[k];
      }
    }
    if constexpr (VEC) {
      float4* xp = reinterpret_cast<float4*>(x + t * D + i);
      float4 x0 = xp[0], x1 = xp[1];
      x0.x += m[0]; x0.y += m[1]; x0.z += m[2]; x0.w += m[3];
      x1.x += m[4]; x1.y += m[5]; x1.z += m[6]; x1.w += m[7];
      xp[0] = x0; xp[1] = x1;
    } else {
      x[t * D + i] += m[0];
    }
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_scaled_add_group_rmsnorm(float* x_out, void* h_out, const float* x, const void* branch, int64_t branch_stride,
                                   const int32_t* rows, const float* coef, int n_branch, float alpha, const void* weight,
                                   int64_t tokens, int64_t hidden, int groups, float eps, int dtype, void* stream) {
  MI355_REQUIRE(x && weight && (x_out || h_out), MI355_ERR_INVALID, "scaled_add_group_rmsnorm: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0 && groups > 0 && hidden % groups == 0 && groups <= 4096 && hidden <= 32768,
                MI355_ERR_INVALID, "scaled_add_group_rmsnorm: bad shape");
  MI355_REQUIRE((rows == nullptr) == (coef == nullptr) && (rows == nullptr || (branch && n_branch > 0)), MI355_ERR_INVALID,
                "scaled_add_group_rmsnorm: rows, coef and the branch come together");
  if (tokens == 0) return MI355_OK;
  const size_t lds = (size_t)(hidden + groups) * sizeof(float);
  const bool vec8 = hidden % 8 == 0 && aligned16(x) && (branch == nullptr || (branch_stride % 8 == 0 && aligned16(branch)));
  MI355_DISPATCH_DTYPE(dtype, "scaled_add_group_rmsnorm", {
    hipLaunchKernelGGL((scaled_add_group_rmsnorm_kernel<T>), dim3((unsigned)tokens), dim3(256), lds, (hipStream_t)stream, x_out,
                       (T*)h_out, x, (const T*)branch, branch_stride, rows, coef, n_branch, alpha, (const T*)weight, hidden,
                       groups, eps, vec8);
  });
  MI355_CHECK_LAUNCH("scaled_add_group_rmsnorm");
  return MI355_OK;
}

int mi355_rmsnorm_residual_add(float* x, void* h_out, const void* y, int64_t y_stride, const void* weight, int64_t tokens,
                               int64_t hidden, float eps, int dtype, void* stream) {
  return mi355_rmsnorm_residual_add_scaled(x, h_out, y, y_stride, weight, nullptr, 0.f, 1.f, tokens, hidden, eps, dtype, stream);
}

int mi355_rmsnorm_residual_add_scaled(float* x, void* h_out, const void* y, int64_t y_stride, const void* weight,
                                      const void* layer_scale, float offset, float mult, int64_t tokens, int64_t hidden, float eps,
                                      int dtype, void* stream) {
  MI355_REQUIRE(x && y && weight, MI355_ERR_INVALID, "rmsnorm_residual_add: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0 && y_stride >= hidden, MI355_ERR_INVALID, "rmsnorm_residual_add: bad shape");
  if (tokens == 0) return MI355_OK;
  // eight 16-bit features are one 16-byte access; fp32 activations (four to 16 bytes) take the scalar kernel
  const bool vec = dtype != MI355_F32 && hidden % 8 == 0 && y_stride % 8 == 0 && aligned16(x) && aligned16(y) && aligned16(weight) &&
                   (h_out == nullptr || aligned16(h_out)) && (layer_scale == nullptr || aligned16(layer_scale));
  MI355_DISPATCH_DTYPE(dtype, "rmsnorm_residual_add", {
    if (vec)
      hipLaunchKernelGGL((rmsnorm_residual_add_kernel<T, true>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x, (T*)h_out,
                         (const T*)y, y_stride, (const T*)weight, (const T*)layer_scale, offset, mult, hidden, eps);
    else
      hipLaunchKernelGGL((rmsnorm_residual_add_kernel<T, false>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x, (T*)h_out,
                         (const T*)y, y_stride, (const T*)weight, (const T*)layer_scale, offset, mult, hidden, eps);
  });
  MI355_CHECK_LAUNCH("rmsnorm_residual_add");
  return MI355_OK;
}

int mi355_head_norm_rope(void* out, const void* src, const void* weight, const int64_t* positions, const int64_t* loc,
                         const float* inv_freq, int64_t tokens, int heads, int head_dim, int64_t src_token_stride,
                         int64_t src_head_stride, int64_t out_token_stride, int64_t out_head_stride, int64_t out_rows, int rot_dims,
                         int interleaved, float scale, float eps, int dtype, int out_dtype, void* stream) {
  return mi355_head_norm_rope_mag(out, src, weight, positions, loc, inv_freq, tokens, heads, head_dim, src_token_stride,
                                  src_head_stride, out_token_stride, out_head_stride, out_rows, rot_dims, interleaved, scale, eps,
                                  1.0f, dtype, out_dtype, stream);
}

int mi355_head_norm_rope_mag(void* out, const void* src, const void* weight, const int64_t* positions, const int64_t* loc,
                             const float* inv_freq, int64_t tokens, int heads, int head_dim, int64_t src_token_stride,
                             int64_t src_head_stride, int64_t out_token_stride, int64_t out_head_stride, int64_t out_rows,
                             int rot_dims, int interleaved, float scale, float eps, float rot_mag, int dtype, int out_dtype,
                             void* stream) {
  MI355_REQUIRE(out && src && positions, MI355_ERR_INVALID, "head_norm_rope: null pointer");
  MI355_REQUIRE(tokens >= 0 && heads > 0 && head_dim > 0 && head_dim <= 4096 && out_rows >= 0, MI355_ERR_INVALID,
                "head_norm_rope: bad shape");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= head_dim && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq), MI355_ERR_INVALID,
                "head_norm_rope: rot_dims must be even, at most head_dim, and come with frequencies");
  MI355_REQUIRE(out_dtype == dtype || out_dtype == MI355_F32, MI355_ERR_UNSUPPORTED,
                "head_norm_rope: the result is written in the input's type or in fp32");
  if (tokens == 0) return MI355_OK;
  const size_t lds = (size_t)4 * head_dim * sizeof(float);
  const unsigned grid = (unsigned)((tokens * heads + 3) / 4);
  MI355_DISPATCH_DTYPE(dtype, "head_norm_rope", {
    if (out_dtype == dtype) {
      hipLaunchKernelGGL((head_norm_rope_kernel<T, T>), dim3(grid), dim3(256), lds, (hipStream_t)stream, (T*)out, (const T*)src,
                         (const T*)weight, positions, loc, inv_freq, tokens, heads, head_dim, src_token_stride, src_head_stride,
                         out_token_stride, out_head_stride, rot_dims, interleaved, scale, eps, rot_mag);
    } else {
      hipLaunchKernelGGL((head_norm_rope_kernel<T, float>), dim3(grid), dim3(256), lds, (hipStream_t)stream, (float*)out,
                         (const T*)src, (const T*)weight, positions, loc, inv_freq, tokens, heads, head_dim, src_token_stride,
                         src_head_stride, out_token_stride, out_head_stride, rot_dims, interleaved, scale, eps, rot_mag);
    }
  });
  MI355_CHECK_LAUNCH("head_norm_rope");
  return MI355_OK;
}

int mi355_head_rmsnorm_gate(void* out, const float* o, const void* weight, const void* gate, int64_t gate_stride, int64_t tokens,
                            int heads, int value_dim, float eps, int dtype, void* stream) {
  return mi355_head_rmsnorm_gate_act(out, o, weight, gate, gate_stride, tokens, heads, value_dim, eps, 0, dtype, stream);
}

int mi355_head_rmsnorm_gate_act(void* out, const float* o, const void* weight, const void* gate, int64_t gate_stride, int64_t tokens,
                                int heads, int value_dim, float eps, int gate_act, int dtype, void* stream) {
  MI355_REQUIRE(out && o && gate, MI355_ERR_INVALID, "head_rmsnorm_gate: null pointer");
  MI355_REQUIRE(gate_act == 0 || gate_act == 1, MI355_ERR_INVALID, "head_rmsnorm_gate: the gate is silu (0) or sigmoid (1)");
  MI355_REQUIRE(tokens >= 0 && heads > 0 && value_dim > 0 && gate_stride >= (int64_t)heads * value_dim, MI355_ERR_INVALID,
                "head_rmsnorm_gate: bad shape");
  if (tokens == 0) return MI355_OK;
  const unsigned grid = (unsigned)((tokens * heads + 3) / 4);
  MI355_DISPATCH_DTYPE(dtype, "head_rmsnorm_gate", {
    hipLaunchKernelGGL((head_rmsnorm_gate_kernel<T>), dim3(grid), dim3(256), 0, (hipStream_t)stream, (T*)out, o, (const T*)weight,
                       (const T*)gate, gate_stride, tokens, heads, value_dim, eps, gate_act);
  });
  MI355_CHECK_LAUNCH("head_rmsnorm_gate");
  return MI355_OK;
}

int mi355_qkv_norm_rope_write(void* q_out, void* k_cache, void* v_cache, const void* q, const void* k, const void* v,
                              int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, const void* wq, const void* wk,
                              const int64_t* positions, const int64_t* loc, const float* inv_freq, int64_t tokens, int heads,
                              int kv_heads, int head_dim, int v_head_dim, int rot_dims, int interleaved, float eps, float rot_mag,
                              int dtype, void* stream) {
  MI355_REQUIRE(q_out && k_cache && v_cache && q && k && v && wq && wk && positions && loc, MI355_ERR_INVALID,
                "qkv_norm_rope_write: null pointer");
  MI355_REQUIRE(tokens >= 0 && heads > 0 && kv_heads > 0 && head_dim > 0 && head_dim <= 4096 && v_head_dim > 0 && v_head_dim <= 4096,
                MI355_ERR_INVALID, "qkv_norm_rope_write: bad shape");
  MI355_REQUIRE(rot_dims >= 0 && rot_dims <= head_dim && rot_dims % 2 == 0 && (rot_dims == 0 || inv_freq), MI355_ERR_INVALID,
                "qkv_norm_rope_write: rot_dims must be even, at most head_dim, and come with frequencies");
  if (tokens == 0) return MI355_OK;
  const size_t lds = (size_t)4 * std::max(head_dim, v_head_dim) * sizeof(float);
  const unsigned grid = (unsigned)((tokens * (heads + 2 * kv_heads) + 3) / 4);
  MI355_DISPATCH_DTYPE(dtype, "qkv_norm_rope_write", {
    hipLaunchKernelGGL((qkv_norm_rope_write_kernel<T>), dim3(grid), dim3(256), lds, (hipStream_t)stream, (T*)q_out, (T*)k_cache,
                       (T*)v_cache, (const T*)q, (const T*)k, (const T*)v, q_token_stride, k_token_stride, v_token_stride, (const T*)wq,
                       (const T*)wk, positions, loc, inv_freq, tokens, heads, kv_heads, head_dim, v_head_dim, rot_dims, interleaved, eps,
                       rot_mag);
  });
  MI355_CHECK_LAUNCH("qkv_norm_rope_write");
  return MI355_OK;
}

int mi355_gated_group_rmsnorm(void* out, const float* y, const void* gate, int64_t gate_stride, const void* weight, int64_t tokens,
                              int64_t hidden, int groups, float eps, int dtype, void* stream) {
  MI355_REQUIRE(out && y && gate && weight, MI355_ERR_INVALID, "gated_group_rmsnorm: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0 && groups >= 1 && hidden % groups == 0 && gate_stride >= hidden &&
                    tokens * groups < ((int64_t)1 << 31), MI355_ERR_INVALID, "gated_group_rmsnorm: bad shape");
  if (tokens == 0) return MI355_OK;
  MI355_DISPATCH_DTYPE(dtype, "gated_group_rmsnorm", {
    hipLaunchKernelGGL((gated_group_rmsnorm_kernel<T>), dim3((unsigned)(tokens * groups)), dim3(256), 0, (hipStream_t)stream, (T*)out, y,
                       (const T*)gate, gate_stride, (const T*)weight, hidden, groups, eps);
  });
  MI355_CHECK_LAUNCH("gated_group_rmsnorm");
  return MI355_OK;
}

int mi355_gelu_tanh_mul_rows(void* out, const void* gate, int64_t gate_stride, const void* table, int64_t table_rows,
                             int64_t table_stride, int64_t col_off, const int64_t* ids, int64_t rows, int64_t d, int dtype,
                             void* stream) {
  MI355_REQUIRE(out && gate && table && ids, MI355_ERR_INVALID, "gelu_tanh_mul_rows: null pointer");
  MI355_REQUIRE(rows >= 0 && d > 0 && gate_stride >= d && col_off >= 0 && col_off + d <= table_stride && table_rows > 0,
                MI355_ERR_INVALID, "gelu_tanh_mul_rows: bad shape");
  if (rows == 0) return MI355_OK;
  const int grid = (int)std::min<int64_t>((rows * d + 255) / 256, 256 * 16);
  MI355_DISPATCH_DTYPE(dtype, "gelu_tanh_mul_rows", {
    hipLaunchKernelGGL((gelu_tanh_mul_rows_kernel<T>), dim3(grid), dim3(256), 0, (hipStream_t)stream, (T*)out, (const T*)gate,
                       gate_stride, (const T*)table, table_stride, col_off, ids, rows, d);
  });
  MI355_CHECK_LAUNCH("gelu_tanh_mul_rows");
  return MI355_OK;
}

int mi355_offset_rmsnorm(void* h, const float* x, const void* weight, int64_t tokens, int64_t hidden, float eps, float offset,
                         int dtype, void* stream) {
  MI355_REQUIRE(h && x && weight, MI355_ERR_INVALID, "offset_rmsnorm: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0, MI355_ERR_INVALID, "offset_rmsnorm: bad shape");
  if (tokens == 0) return MI355_OK;
  const bool vec = hidden % 8 == 0 && aligned16(x) && aligned16(h) && aligned16(weight);
  MI355_DISPATCH_DTYPE(dtype, "offset_rmsnorm", {
    if (vec)
      hipLaunchKernelGGL((offset_rmsnorm_kernel<T, true>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, (T*)h, x,
                         (const T*)weight, hidden, eps, offset);
    else
      hipLaunchKernelGGL((offset_rmsnorm_kernel<T, false>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, (T*)h, x,
                         (const T*)weight, hidden, eps, offset);
  });
  MI355_CHECK_LAUNCH("offset_rmsnorm");
  return MI355_OK;
}

int mi355_branch_residual_add(float* x, const void* a, int64_t a_stride, const void* wa, const void* b, int64_t b_stride,
                              const void* wb, float s, const void* f, int64_t f_stride, const int32_t* rows, const float* coef,
                              int n_branch, int64_t tokens, int64_t hidden, float eps, int dtype, void* stream) {
  MI355_REQUIRE(x && a, MI355_ERR_INVALID, "branch_residual_add: null pointer");
  MI355_REQUIRE(tokens >= 0 && hidden > 0 && a_stride >= hidden && (b == nullptr || b_stride >= hidden) &&
                    (f == nullptr || f_stride >= hidden), MI355_ERR_INVALID, "branch_residual_add: bad shape");
  MI355_REQUIRE(b != nullptr || wb == nullptr, MI355_ERR_INVALID, "branch_residual_add: a weight without its branch");
  MI355_REQUIRE((rows == nullptr) == (coef == nullptr) && (rows == nullptr || (f && n_branch > 0)), MI355_ERR_INVALID,
                "branch_residual_add: rows, coef and their tensor come together");
  if (tokens == 0) return MI355_OK;
  const bool vec = hidden % 8 == 0 && aligned16(x) && aligned16(a) && a_stride % 8 == 0 && (wa == nullptr || aligned16(wa)) &&
                   (b == nullptr || (aligned16(b) && b_stride % 8 == 0)) && (wb == nullptr || aligned16(wb)) &&
                   (f == nullptr || (aligned16(f) && f_stride % 8 == 0));
  MI355_DISPATCH_DTYPE(dtype, "branch_residual_add", {
    if (vec)
      hipLaunchKernelGGL((branch_residual_add_kernel<T, true>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x,
                         (const T*)a, a_stride, (const T*)wa, (const T*)b, b_stride, (const T*)wb, s, (const T*)f, f_stride, rows, coef,
                         n_branch, hidden, eps);
    else
      hipLaunchKernelGGL((branch_residual_add_kernel<T, false>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, x,
                         (const T*)a, a_stride, (const T*)wa, (const T*)b, b_stride, (const T*)wb, s, (const T*)f, f_stride, rows, coef,
                         n_branch, hidden, eps);
  });
  MI355_CHECK_LAUNCH("branch_residual_add");
  return MI355_OK;
}
