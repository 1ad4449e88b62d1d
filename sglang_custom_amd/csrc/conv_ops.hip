// Short causal convolutions over time, one filter per channel, for sequences that arrive in pieces:
//     y[t][c] = act( (residual ? u[t][c] : 0) + sum_{k < taps} w[c][taps - 1 - k] * u[t - k][c] [+ bias[c]] ),   u = 0 before position 0
// The last taps - 1 inputs of a sequence are its state (fp32 rows [slots, taps - 1, C], row taps - 2 the most recent): a
// step's first tokens read them, and after the step they are replaced by the step's own last inputs.
//   * mi355_causal_conv: every (token, channel) in one launch; up to two filters read the same input (two outputs).  In a
//     step of single tokens (no segments) the same thread also shifts the state, so decode is one launch.
//   * mi355_causal_conv_state_update: the shift for steps with segments, one thread per (sequence, channel), after the
//     convolution has read the old rows.
//   * mi355_activation: out = act(in) over a strided [rows, cols] block (silu, squared relu).
// The sum runs over the taps in a fixed order in fp32 whether an input comes from the step or from the state, so a
// position's result does not depend on how its sequence was cut.
#include "common.cuh"

#include <algorithm>

namespace mi355 {
namespace {

constexpr int CONV_MAX_TAPS = 8;

__device__ __forceinline__ float conv_act(float z, int act) {
  if (act == 1) return z / (1.0f + expf(-z));
  if (act == 2) { const float r = fmaxf(z, 0.f); return r * r; }
  return z;
}

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_kernel(T* __restrict__ y1, T* __restrict__ y2, const T* __restrict__ u,
                                                          int64_t u_stride, const T* __restrict__ w1, const T* __restrict__ w2,
                                                          float* __restrict__ state, const int32_t* __restrict__ req_to_state,
                                                          const int64_t* __restrict__ req_pool_indices,
                                                          const int32_t* __restrict__ tok_req, const int32_t* __restrict__ seg_start,
                                                          const int64_t* __restrict__ positions, int64_t C, int taps, int residual,
                                                          int act, const T* __restrict__ bias) {
  const int64_t t = blockIdx.x;
  const int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = tok_req != nullptr ? tok_req[t] : (int)t;
  const int64_t t0 = seg_start != nullptr ? seg_start[b] : t;
  const int64_t pos = positions[t];
  const int back = (int)(t - t0);                 // tokens of this step before t in its sequence
  float* rows = state + (int64_t)req_to_state[req_pool_indices[b]] * (taps - 1) * C + c;
  float in[CONV_MAX_TAPS];                         // in[k]: the input k tokens back
#pragma unroll
  for (int k = 0; k < CONV_MAX_TAPS; ++k) {
    if (k >= taps) break;
    float v = 0.f;
    if (k <= back) v = to_f32(u[(t - k) * u_stride + c]);
    else if (pos - k >= 0) v = rows[(int64_t)(taps - 1 - (k - back)) * C];
    in[k] = v;
  }
  float a1 = 0.f, a2 = 0.f;
#pragma unroll
  for (int k = CONV_MAX_TAPS - 1; k >= 0; --k) {   // oldest tap first
    if (k >= taps) continue;
    a1 = fmaf(to_f32(w1[c * taps + (taps - 1 - k)]), in[k], a1);
    if (w2 != nullptr) a2 = fmaf(to_f32(w2[c * taps + (taps - 1 - k)]), in[k], a2);
  }
  if (residual) { a1 += in[0]; a2 += in[0]; }
  if (bias != nullptr) a1 += to_f32(bias[c]);
  y1[t * C + c] = from_f32<T>(conv_act(a1, act));
  if (w2 != nullptr) y2[t * C + c] = from_f32<T>(conv_act(a2, act));
  if (tok_req == nullptr) {
    // a step of single tokens: this thread is the only reader and writer of its channel's rows
#pragma unroll
    for (int k = CONV_MAX_TAPS - 2; k >= 0; --k) {
      if (k >= taps - 1) continue;
      rows[(int64_t)(taps - 2 - k) * C] = in[k];
    }
  }
}

// The same for rows of 16-byte channel groups: a thread owns V consecutive channels (V * sizeof(T) = 16) of CONV_TT
// consecutive tokens, so inputs, filters (V * TAPS consecutive elements) and results move as whole vectors, the filters are
// read once per CONV_TT tokens, and a token that follows one of its own sequence takes that token's inputs shifted by one
// instead of reading them again.  TAPS is a template argument so that a filter element's place in its vector is known at
// compile time.
constexpr int CONV_TT = 4;

template <typename T, int V, int TAPS>
__global__ __launch_bounds__(256) void causal_conv_vec_kernel(T* __restrict__ y1, T* __restrict__ y2, const T* __restrict__ u,
                                                              int64_t u_stride, const T* __restrict__ w1, const T* __restrict__ w2,
                                                              float* __restrict__ state, const int32_t* __restrict__ req_to_state,
                                                              const int64_t* __restrict__ req_pool_indices,
                                                              const int32_t* __restrict__ tok_req, const int32_t* __restrict__ seg_start,
                                                              const int64_t* __restrict__ positions, int64_t tokens, int64_t C,
                                                              int residual, int act, const T* __restrict__ bias) {
  const int64_t groups = C / V;
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t tb = idx / groups;
  if (tb * CONV_TT >= tokens) return;
  const int64_t c = (idx - tb * groups) * V;
  float wf[2][V * TAPS];                             // [filter][channel][tap], as stored
#pragma unroll
  for (int f = 0; f < 2; ++f) {
    const T* w = f == 0 ? w1 : w2;
    if (w == nullptr) break;
#pragma unroll
    for (int i = 0; i < TAPS; ++i) {
      const Vec<T, V> x = ldvec<T, V>(w + c * TAPS + i * V);
#pragma unroll
      for (int v = 0; v < V; ++v) wf[f][i * V + v] = to_f32(x.v[v]);
    }
  }
  float bf[V];                                       // the first filter's bias
  if (bias != nullptr) {
    const Vec<T, V> x = ldvec<T, V>(bias + c);
#pragma unroll
    for (int v = 0; v < V; ++v) bf[v] = to_f32(x.v[v]);
  } else {
#pragma unroll
    for (int v = 0; v < V; ++v) bf[v] = 0.f;
  }
  float in[TAPS][V];                                 // in[k]: the input k tokens back
#pragma unroll
  for (int j = 0; j < CONV_TT; ++j) {
    const int64_t t = tb * CONV_TT + j;
    if (t >= tokens) break;
    const int b = tok_req != nullptr ? tok_req[t] : (int)t;
    const int64_t t0 = seg_start != nullptr ? seg_start[b] : t;
    const int64_t pos = positions[t];
    const int back = (int)(t - t0);
    float* rows = state + (int64_t)req_to_state[req_pool_indices[b]] * (TAPS - 1) * C + c;
    if (j > 0 && back >= 1) {
      // the token before is this sequence's and this thread's: its inputs, one further back each
#pragma unroll
      for (int k = TAPS - 1; k >= 1; --k)
#pragma unroll
        for (int v = 0; v < V; ++v) in[k][v] = in[k - 1][v];
      const Vec<T, V> x = ldvec<T, V>(u + t * u_stride + c);
#pragma unroll
      for (int v = 0; v < V; ++v) in[0][v] = to_f32(x.v[v]);
    } else {
#pragma unroll
      for (int k = 0; k < TAPS; ++k) {
        if (k <= back) {
          const Vec<T, V> x = ldvec<T, V>(u + (t - k) * u_stride + c);
#pragma unroll
          for (int v = 0; v < V; ++v) in[k][v] = to_f32(x.v[v]);
        } else if (pos - k >= 0) {
          const float* r = rows + (int64_t)(TAPS - 1 - (k - back)) * C;
#pragma unroll
          for (int v = 0; v < V; v += 4) {
            const float4 q = *reinterpret_cast<const float4*>(r + v);
            in[k][v] = q.x; in[k][v + 1] = q.y; in[k][v + 2] = q.z; in[k][v + 3] = q.w;
          }
        } else {
#pragma unroll
          for (int v = 0; v < V; ++v) in[k][v] = 0.f;
        }
      }
    }
#pragma unroll
    for (int f = 0; f < 2; ++f) {
      if ((f == 0 ? w1 : w2) == nullptr) break;
      Vec<T, V> out;
#pragma unroll
      for (int v = 0; v < V; ++v) {
        float a = 0.f;
#pragma unroll
        for (int k = TAPS - 1; k >= 0; --k) a = fmaf(wf[f][v * TAPS + (TAPS - 1 - k)], in[k][v], a);     // oldest tap first
        if (residual) a += in[0][v];
        if (f == 0) a += bf[v];
        out.v[v] = from_f32<T>(conv_act(a, act));
      }
      stvec<T, V>((f == 0 ? y1 : y2) + t * C + c, out);
    }
    if (tok_req == nullptr) {
      // a step of single tokens: this thread is the only reader and writer of its channels' rows
#pragma unroll
      for (int k = TAPS - 2; k >= 0; --k) {
        float* r = rows + (int64_t)(TAPS - 2 - k) * C;
#pragma unroll
        for (int v = 0; v < V; v += 4) *reinterpret_cast<float4*>(r + v) = make_float4(in[k][v], in[k][v + 1], in[k][v + 2], in[k][v + 3]);
      }
    }
  }
}

template <typename T, int TAPS>
void launch_conv_vec(void* y1, void* y2, const void* u, int64_t u_stride, const void* w1, const void* w2, float* state,
                     const int32_t* req_to_state, const int64_t* req_pool_indices, const int32_t* tok_req, const int32_t* seg_start,
                     const int64_t* positions, int64_t tokens, int64_t channels, int residual, int act, const void* bias, hipStream_t stream) {
  constexpr int V = 16 / sizeof(T);
  const int64_t n = ((tokens + CONV_TT - 1) / CONV_TT) * (channels / V);
  hipLaunchKernelGGL((causal_conv_vec_kernel<T, V, TAPS>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, (T*)y1, (T*)y2,
                     (const T*)u, u_stride, (const T*)w1, (const T*)w2, state, req_to_state, req_pool_indices, tok_req, seg_start,
                     positions, tokens, channels, residual, act, (const T*)bias);
}

template <typename T>
__global__ __launch_bounds__(256) void causal_conv_state_update_kernel(float* __restrict__ state, const T* __restrict__ u,
                                                                       int64_t u_stride, const int32_t* __restrict__ req_to_state,
                                                                       const int64_t* __restrict__ req_pool_indices,
                                                                       const int32_t* __restrict__ seg_start,
                                                                       const int32_t* __restrict__ seg_len,
                                                                       const int64_t* __restrict__ positions, int64_t C, int taps) {
  const int b = blockIdx.y;
  const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int n = seg_len[b];
  if (n <= 0) return;
  const int64_t t0 = seg_start[b];
  const int64_t p0 = positions[t0];
  float* rows = state + (int64_t)req_to_state[req_pool_indices[b]] * (taps - 1) * C + c;
  // the old rows followed by the step's inputs; the new rows are the last taps - 1 of that list.  Row i takes entry
  // n + i >= i + 1, so going up never reads a row already replaced.
  for (int i = 0; i < taps - 1; ++i) {
    const int e = n + i;
    float v;
    if (e < taps - 1) v = (p0 - (taps - 1) + e >= 0) ? rows[(int64_t)e * C] : 0.f;
    else v = to_f32(u[(t0 + e - (taps - 1)) * u_stride + c]);
    rows[(int64_t)i * C] = v;
  }
}

template <typename T>
__global__ __launch_bounds__(256) void activation_kernel(T* __restrict__ out, const T* __restrict__ in, int64_t in_stride,
                                                         int64_t rows, int64_t cols, int act) {
  const int64_t n = rows * cols;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / cols, i = idx - r * cols;
    out[idx] = from_f32<T>(conv_act(to_f32(in[r * in_stride + i]), act));
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_causal_conv(void* y1, void* y2, const void* u, int64_t u_stride, const void* w1, const void* w2, float* state,
                      const int32_t* req_to_state, const int64_t* req_pool_indices, const int32_t* tok_req,
                      const int32_t* seg_start, const int64_t* positions, int64_t tokens, int64_t channels, int taps,
                      int residual, int act, int dtype, void* stream) {
  return mi355_causal_conv_bias(y1, y2, u, u_stride, w1, w2, nullptr, state, req_to_state, req_pool_indices, tok_req, seg_start,
                                positions, tokens, channels, taps, residual, act, dtype, stream);
}

int mi355_causal_conv_bias(void* y1, void* y2, const void* u, int64_t u_stride, const void* w1, const void* w2, const void* bias1,
                           float* state, const int32_t* req_to_state, const int64_t* req_pool_indices, const int32_t* tok_req,
                           const int32_t* seg_start, const int64_t* positions, int64_t tokens, int64_t channels, int taps,
                           int residual, int act, int dtype, void* stream) {
  MI355_REQUIRE(y1 && u && w1 && (state || taps == 1) && req_to_state && req_pool_indices && positions, MI355_ERR_INVALID, "causal_conv: null pointer");
  MI355_REQUIRE((w2 == nullptr) == (y2 == nullptr), MI355_ERR_INVALID, "causal_conv: the second filter comes with its output");
  MI355_REQUIRE((tok_req == nullptr) == (seg_start == nullptr), MI355_ERR_INVALID, "causal_conv: tok_req and seg_start come together");
  MI355_REQUIRE(tokens >= 0 && tokens <= 0x7fffffff && channels > 0 && u_stride >= channels && taps >= 1 && taps <= CONV_MAX_TAPS &&
                    act >= 0 && act <= 2, MI355_ERR_INVALID, "causal_conv: bad shape (1 to %d taps)", CONV_MAX_TAPS);
  if (tokens == 0) return MI355_OK;
  MI355_REQUIRE(channels <= 65535 * 256, MI355_ERR_UNSUPPORTED, "causal_conv: too many channels");
  const int esz = dtype == MI355_F32 ? 4 : 2, vw = 16 / esz;
  const bool vec = channels % vw == 0 && u_stride % vw == 0 && aligned16(u) && aligned16(y1) && aligned16(w1) &&
                   (y2 == nullptr || (aligned16(y2) && aligned16(w2))) && (taps == 1 || aligned16(state)) && channels % 4 == 0 &&
                   (bias1 == nullptr || aligned16(bias1)) &&
                   tokens * (channels / vw) < ((int64_t)1 << 31) * 256;
  if (vec) {
#define MI355_CONV_TAPS(N)                                                                                                    \
  case N:                                                                                                                     \
    MI355_DISPATCH_DTYPE(dtype, "causal_conv", {                                                                              \
      launch_conv_vec<T, N>(y1, y2, u, u_stride, w1, w2, state, req_to_state, req_pool_indices, tok_req, seg_start, positions,   \
                            tokens, channels, residual, act, bias1, (hipStream_t)stream);                                     \
    });                                                                                                                       \
    break;
    switch (taps) {
      MI355_CONV_TAPS(1) MI355_CONV_TAPS(2) MI355_CONV_TAPS(3) MI355_CONV_TAPS(4) MI355_CONV_TAPS(5) MI355_CONV_TAPS(6)
      MI355_CONV_TAPS(7) MI355_CONV_TAPS(8)
      default: break;
    }
#undef MI355_CONV_TAPS
    MI355_CHECK_LAUNCH("causal_conv");
    return MI355_OK;
  }
  const dim3 grid((unsigned)tokens, (unsigned)cdiv(channels, 256));
  MI355_DISPATCH_DTYPE(dtype, "causal_conv", {
    hipLaunchKernelGGL((causal_conv_kernel<T>), grid, dim3(256), 0, (hipStream_t)stream, (T*)y1, (T*)y2, (const T*)u, u_stride,
                       (const T*)w1, (const T*)w2, state, req_to_state, req_pool_indices, tok_req, seg_start, positions, channels,
                       taps, residual, act, (const T*)bias1);
  });
  MI355_CHECK_LAUNCH("causal_conv");
  return MI355_OK;
}

int mi355_causal_conv_state_update(float* state, const void* u, int64_t u_stride, const int32_t* req_to_state,
                                   const int64_t* req_pool_indices, const int32_t* seg_start, const int32_t* seg_len,
                                   const int64_t* positions, int64_t batch, int64_t channels, int taps, int dtype, void* stream) {
  MI355_REQUIRE((state || taps == 1) && u && req_to_state && req_pool_indices && seg_start && seg_len && positions, MI355_ERR_INVALID,
                "causal_conv_state_update: null pointer");
  MI355_REQUIRE(batch >= 0 && batch <= 65535 && channels > 0 && u_stride >= channels && taps >= 1 && taps <= CONV_MAX_TAPS,
                MI355_ERR_INVALID, "causal_conv_state_update: bad shape");
  if (batch == 0 || taps == 1) return MI355_OK;
  const dim3 grid((unsigned)cdiv(channels, 256), (unsigned)batch);
  MI355_DISPATCH_DTYPE(dtype, "causal_conv_state_update", {
    hipLaunchKernelGGL((causal_conv_state_update_kernel<T>), grid, dim3(256), 0, (hipStream_t)stream, state, (const T*)u, u_stride,
                       req_to_state, req_pool_indices, seg_start, seg_len, positions, channels, taps);
  });
  MI355_CHECK_LAUNCH("causal_conv_state_update");
  return MI355_OK;
}

int mi355_activation(void* out, const void* in, int64_t in_stride, int64_t rows, int64_t cols, int act, int dtype, void* stream) {
  MI355_REQUIRE(out && in, MI355_ERR_INVALID, "activation: null pointer");
  MI355_REQUIRE(rows >= 0 && cols > 0 && in_stride >= cols && (act == 1 || act == 2), MI355_ERR_INVALID, "activation: bad shape or kind");
  if (rows == 0) return MI355_OK;
  const int grid = (int)std::min<int64_t>((rows * cols + 255) / 256, 256 * 16);
  MI355_DISPATCH_DTYPE(dtype, "activation", {
    hipLaunchKernelGGL((activation_kernel<T>), dim3(grid), dim3(256), 0, (hipStream_t)stream, (T*)out, (const T*)in, in_stride, rows,
                       cols, act);
  });
  MI355_CHECK_LAUNCH("activation");
  return MI355_OK;
}
