// Mixture of experts without a trip to the host:
//   * mi355_moe_route_grouped: sigmoid scores, grouped top-k selection on corrected scores, normalised weights (one wave
//     per token, fp32),
//   * mi355_moe_align: the (token, choice) pairs sorted by expert into blocks of `block` rows that belong to one expert
//     each (padding rows marked -1), with the block -> expert table and the number of blocks used, all on the device,
//   * mi355_moe_grouped_linear: out[p] = act(W[expert of p's block] . in[row(p)]) over those blocks; rows are gathered
//     through the sorted list (first GEMM) or taken in place (second GEMM); blocks past the used count exit at once.
//     16-bit dtypes with K a multiple of 8 run on the matrix cores, reading both operands' fragments straight from
//     global memory (a weight row and an input row are both contiguous along K, which is the fragment's direction);
//     everything else (fp32: exact) on the vector ALU through LDS tiles.
#include "common.cuh"

#include <algorithm>
#include <type_traits>

namespace mi355 {
namespace {

constexpr int MOE_BLOCK = 64;

__device__ __forceinline__ float moe_gelu_erf(float z) { return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f)); }

// One wave per token; sm per wave: choice[E] | score[E] | group[G]
__global__ __launch_bounds__(256) void moe_route_grouped_kernel(int32_t* __restrict__ ids, float* __restrict__ weights,
                                                                const float* __restrict__ logits,
                                                                const float* __restrict__ correction, int64_t tokens, int E,
                                                                int top, int n_groups, int keep, float scale, int score_fn,
                                                                int group_best, int renorm) {
  extern __shared__ float sm[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t t = (int64_t)blockIdx.x * 4 + wv;
  float* choice = sm + (int64_t)wv * (2 * E + n_groups);
  float* score = choice + E;
  float* gsc = score + E;
  const bool valid = t < tokens;
  const int per = E / n_groups;
  if (valid) {
    float mx = 0.f, inv = 1.f;
    if (score_fn == 1) {
      // softmax over all experts
      mx = -INFINITY;
      for (int e = lane; e < E; e += 64) mx = fmaxf(mx, logits[t * E + e]);
      mx = wave_max(mx);
      float sum = 0.f;
      for (int e = lane; e < E; e += 64) sum += expf(logits[t * E + e] - mx);
      inv = 1.0f / wave_sum(sum);
    }
    for (int e = lane; e < E; e += 64) {
      const float s = score_fn == 1 ? expf(logits[t * E + e] - mx) * inv : 1.0f / (1.0f + expf(-logits[t * E + e]));
      score[e] = s;
      choice[e] = s + (correction != nullptr ? correction[e] : 0.f);
    }
  }
  __syncthreads();
  if (valid) {
    for (int g = lane; g < n_groups; g += 64) {
      float m1 = -INFINITY, m2 = -INFINITY;
      for (int i = 0; i < per; ++i) {
        const float c = choice[g * per + i];
        if (c > m1) {
          m2 = m1;
          m1 = c;
        } else if (c > m2) {
          m2 = c;
        }
      }
      gsc[g] = (per > 1 && group_best >= 2) ? m1 + m2 : m1;
    }
  }
  __syncthreads();
  if (valid) {
    // group g stays if fewer than `keep` groups come before it (larger score, or equal score and smaller index)
    for (int g = lane; g < n_groups; g += 64) {
      const float mine = gsc[g];
      int before = 0;
      for (int o = 0; o < n_groups; ++o) before += (gsc[o] > mine || (gsc[o] == mine && o < g)) ? 1 : 0;
      if (before >= keep)
        for (int i = 0; i < per; ++i) choice[g * per + i] = -INFINITY;
    }
  }
  __syncthreads();
  if (!valid) return;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float c = choice[e];
      if (c > best || (c == best && e < bi)) {
        best = c;
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (bi >= E) bi = 0;            // nothing left to choose from (NaN scores): stay inside the table
    if ((bi & 63) == lane) choice[bi] = -INFINITY;     // the owner of that entry retires it; it alone reads it again
    const float s = score[bi];
    total += s;
    if (lane == 0) {
      ids[t * top + k] = bi;
      weights[t * top + k] = s;
    }
  }
  if (lane == 0) {
    const float inv = renorm ? scale / (total + 1e-20f) : scale;
    for (int k = 0; k < top; ++k) weights[t * top + k] *= inv;
  }
}

// One workgroup.  src_row must hold `padded` entries, tile_expert padded / block.
__global__ __launch_bounds__(1024) void moe_align_kernel(int32_t* __restrict__ src_row, int32_t* __restrict__ rows,
                                                         int32_t* __restrict__ tile_expert, int32_t* __restrict__ n_tiles,
                                                         const int32_t* __restrict__ ids, int64_t pairs, int top, int E, int block,
                                                         int64_t padded) {
  extern __shared__ int smi[];
  int* count = smi;            // [E]
  int* start = smi + E;        // [E + 1]
  for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
  for (int64_t p = threadIdx.x; p < padded; p += blockDim.x) src_row[p] = -1;
  __syncthreads();
  for (int64_t i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      const int nb = (count[e] + block - 1) / block;
      for (int b = 0; b < nb; ++b) tile_expert[at / block + b] = e;
      at += nb * block;
      count[e] = 0;              // becomes the cursor
    }
    start[E] = at;
    *n_tiles = at / block;
  }
  __syncthreads();
  for (int64_t i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int e = ids[i];
    if (e < 0 || e >= E) {
      rows[i] = 0;
      continue;
    }
    const int p = start[e] + atomicAdd(&count[e], 1);
    src_row[p] = (int)(i / top);
    rows[i] = p;
  }
}

// Vector ALU, any type and shape: 64 x 64 output tile, K in steps of 16 through LDS, 4 x 4 outputs per thread.
template <typename T>
__global__ __launch_bounds__(256) void moe_grouped_linear_valu_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                                      int64_t in_stride, const T* __restrict__ w,
                                                                      const int32_t* __restrict__ src_row,
                                                                      const int32_t* __restrict__ tile_expert,
                                                                      const int32_t* __restrict__ n_tiles, int gather, int gelu,
                                                                      int N, int K) {
  const int tile = blockIdx.y;
  if (tile >= *n_tiles) return;
  __shared__ float As[16][MOE_BLOCK + 4];
  __shared__ float Ws[16][64 + 4];
  __shared__ int rowsrc[MOE_BLOCK];
  const int e = tile_expert[tile];
  const int n0 = blockIdx.x * 64;
  const int tid = threadIdx.x;
  if (tid < MOE_BLOCK) {
    const int s = src_row[tile * MOE_BLOCK + tid];
    rowsrc[tid] = s < 0 ? -1 : (gather ? s : tile * MOE_BLOCK + tid);
  }
  __syncthreads();
  const T* we = w + (int64_t)e * N * K;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  const int tr = tid >> 4, tc = tid & 15;       // rows tr * 4.., columns tc * 4..
  for (int k0 = 0; k0 < K; k0 += 16) {
    for (int x = tid; x < 64 * 16; x += 256) {
      const int r = x >> 4, kk = x & 15;
      const int src = rowsrc[r];
      As[kk][r] = (src >= 0 && k0 + kk < K) ? to_f32(in[(int64_t)src * in_stride + k0 + kk]) : 0.f;
      Ws[kk][r] = (n0 + r < N && k0 + kk < K) ? to_f32(we[(int64_t)(n0 + r) * K + k0 + kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][tr * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = Ws[kk][tc * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = tr * 4 + i;
    const bool live = rowsrc[r] >= 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tc * 4 + j;
      if (n >= N) continue;
      float y = live ? acc[i][j] : 0.f;
      if (gelu) y = moe_gelu_erf(y);
      out[(int64_t)(tile * MOE_BLOCK + r) * N + n] = from_f32<T>(y);
    }
  }
}

// Matrix cores, 16-bit types, K % 8 == 0: 64 x 64 output tile, wave (wm, wn) owns its 32 x 32 quarter as 2 x 2 MFMA
// 16x16x32 tiles.  Lane l reads A[row l & 15][k0 + 8 (l >> 4) ..+7] and W[n l & 15][the same k]: 16 contiguous bytes each.
template <typename T>
__global__ __launch_bounds__(256) void moe_grouped_linear_mfma_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                                      int64_t in_stride, const T* __restrict__ w,
                                                                      const int32_t* __restrict__ src_row,
                                                                      const int32_t* __restrict__ tile_expert,
                                                                      const int32_t* __restrict__ n_tiles, int gather, int gelu,
                                                                      int N, int K) {
  const int tile = blockIdx.y;
  if (tile >= *n_tiles) return;
  using Frag = typename Mfma<T>::frag;
  const int e = tile_expert[tile];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int wm = wv >> 1, wn = wv & 1;
  const int n0 = blockIdx.x * 64 + wn * 32;
  const int i = lane & 15, kq = lane >> 4;
  const T* we = w + (int64_t)e * N * K;
  // every load is unconditional: padding rows and columns past N read row 0 (their products are never stored), the K
  // tail is zeroed by a select
  const T* arow[2];
  const T* brow[2];
#pragma unroll
  for (int x = 0; x < 2; ++x) {
    const int p = tile * MOE_BLOCK + wm * 32 + x * 16 + i;
    const int s = src_row[p];
    arow[x] = in + (int64_t)(s < 0 ? 0 : (gather ? s : p)) * in_stride;
    const int n = n0 + x * 16 + i;
    brow[x] = we + (int64_t)(n < N ? n : 0) * K;
  }
  f32x4 acc[2][2];
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int y = 0; y < 2; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};
  const Frag zero = {};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in_k = k0 + 8 * kq < K;
    const int k = in_k ? k0 + 8 * kq : 0;
    Frag af[2], bf[2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
      const Frag av = *reinterpret_cast<const Frag*>(arow[x] + k);
      af[x] = in_k ? av : zero;
      bf[x] = *reinterpret_cast<const Frag*>(brow[x] + k);
    }
#pragma unroll
    for (int x = 0; x < 2; ++x)
#pragma unroll
      for (int y = 0; y < 2; ++y) acc[x][y] = Mfma<T>::run(af[x], bf[y], acc[x][y]);
  }
#pragma unroll
  for (int x = 0; x < 2; ++x)
#pragma unroll
    for (int y = 0; y < 2; ++y) {
      const int n = n0 + y * 16 + (lane & 15);
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int p = tile * MOE_BLOCK + wm * 32 + x * 16 + 4 * (lane >> 4) + r;
        float v = src_row[p] >= 0 ? acc[x][y][r] : 0.f;
        if (gelu) v = moe_gelu_erf(v);
        out[(int64_t)p * N + n] = from_f32<T>(v);
      }
    }
}


// Matrix cores through LDS for prefill-sized steps: 128 x 128 output tile (one block of 128 sorted rows of one expert), K in
// tiles of 64, wave (wm, wn) owns a 64 x 64 quarter as 4 x 4 MFMA 16x16x32 tiles.  The next K tile's rows travel from
// global memory into registers while the current one is multiplied and are stored to LDS after it; LDS rows are padded by
// 16 bytes so that the 16-byte fragment reads of 16 consecutive rows fall into different banks.
// one 16-byte load, spelled as a vector of four dwords so that it cannot be taken apart
typedef unsigned moe_u32x4 __attribute__((ext_vector_type(4)));
template <typename T> __device__ __forceinline__ Vec<T, 8> ld16(const T* p) {
  return __builtin_bit_cast(Vec<T, 8>, *reinterpret_cast<const moe_u32x4*>(p));
}

constexpr int MOE_WIDE = 128;
constexpr int MOE_WK = 64;
constexpr int MOE_WLD = MOE_WK + 8;

template <typename T>
__global__ __launch_bounds__(256) void moe_grouped_linear_wide_kernel(T* __restrict__ out, const T* __restrict__ in,
                                                                      int64_t in_stride, const T* __restrict__ w,
                                                                      const int32_t* __restrict__ src_row,
                                                                      const int32_t* __restrict__ tile_expert,
                                                                      const int32_t* __restrict__ n_tiles, int gather, int gelu,
                                                                      int N, int K) {
  const int tile = blockIdx.y;
  if (tile >= *n_tiles) return;
  using Frag = typename Mfma<T>::frag;
  __shared__ __attribute__((aligned(16))) T As[MOE_WIDE * MOE_WLD];
  __shared__ __attribute__((aligned(16))) T Bs[MOE_WIDE * MOE_WLD];
  __shared__ int rowsrc[MOE_WIDE];
  const int e = tile_expert[tile];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int wm = wv >> 1, wn = wv & 1;
  const int li = lane & 15, lg = lane >> 4;
  const int n0 = blockIdx.x * MOE_WIDE;
  if (tid < MOE_WIDE) {
    const int sr = src_row[tile * MOE_WIDE + tid];
    rowsrc[tid] = sr < 0 ? -1 : (gather ? sr : tile * MOE_WIDE + tid);
  }
  __syncthreads();
  const T* we = w + (int64_t)e * N * K;
  // staging: chunk c = tid + 256 u (u < 4) is row c / 8, 16-byte piece c % 8 of the 64-wide K tile.  Every load is
  // unconditional (a load under a branch is waited for at the branch's end, one latency per load): padding rows and
  // columns past N read row 0 -- their products are never stored -- and only the K tail is zeroed, by a select.
  const T* aptr[4];
  const T* bptr[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int c = tid + 256 * u, r = c >> 3, piece = c & 7;
    const int sr = rowsrc[r];
    aptr[u] = in + (int64_t)(sr < 0 ? 0 : sr) * in_stride + piece * 8;
    bptr[u] = we + (int64_t)(n0 + r < N ? n0 + r : 0) * K + piece * 8;
  }
  Vec<T, 8> zero8;
#pragma unroll
  for (int x = 0; x < 8; ++x) zero8.v[x] = from_f32<T>(0.f);
  Vec<T, 8> areg[4], breg[4];
  const bool k_tail = K % MOE_WK != 0;
  auto request = [&](int k0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int piece = (tid + 256 * u) & 7;
      const bool in_k = !k_tail || k0 + piece * 8 < K;
      const int kk = in_k ? k0 : 0;
      const Vec<T, 8> av = ld16<T>(aptr[u] + kk), bv = ld16<T>(bptr[u] + kk);
      areg[u] = in_k ? av : zero8;
      breg[u] = bv;
    }
  };
  f32x4 acc[4][4];
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int y = 0; y < 4; ++y) acc[x][y] = f32x4{0.f, 0.f, 0.f, 0.f};
  request(0);
  for (int k0 = 0; k0 < K; k0 += MOE_WK) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = tid + 256 * u, r = c >> 3, piece = c & 7;
      lds_store16(As + r * MOE_WLD + piece * 8, areg[u]);
      lds_store16(Bs + r * MOE_WLD + piece * 8, breg[u]);
    }
    __syncthreads();
    if (k0 + MOE_WK < K) request(k0 + MOE_WK);
#pragma unroll
    for (int kk = 0; kk < MOE_WK; kk += 32) {
      Frag af[4], bf[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        af[x] = lds_load16<Frag>(As + (wm * 64 + x * 16 + li) * MOE_WLD + kk + 8 * lg);
        bf[x] = lds_load16<Frag>(Bs + (wn * 64 + x * 16 + li) * MOE_WLD + kk + 8 * lg);
      }
#pragma unroll
      for (int x = 0; x < 4; ++x)
#pragma unroll
        for (int y = 0; y < 4; ++y) acc[x][y] = Mfma<T>::run(af[x], bf[y], acc[x][y]);
    }
  }
#pragma unroll
  for (int x = 0; x < 4; ++x)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = wm * 64 + x * 16 + 4 * lg + r;
      const bool live = rowsrc[row] >= 0;
      T* dst = out + (int64_t)(tile * MOE_WIDE + row) * N;
#pragma unroll
      for (int y = 0; y < 4; ++y) {
        const int n = n0 + wn * 64 + y * 16 + li;
        if (n >= N) continue;
        float v = live ? acc[x][y][r] : 0.f;
        if (gelu) v = moe_gelu_erf(v);
        dst[n] = from_f32<T>(v);
      }
    }
}

// Exact fp32 logits of few rows against a small table: out[t][n] = x[t] . w[n].  One workgroup per row: the row is staged
// in LDS once, wave v takes table rows v, v + 4, ..., four at a time so that sixteen loads are in flight per lane; meant for
// decode-sized steps, where a tiled GEMM with so few columns would occupy a handful of CUs.
__global__ __launch_bounds__(256) void moe_router_logits_kernel(float* __restrict__ out, const float* __restrict__ x,
                                                                const float* __restrict__ w, int N, int K) {
  extern __shared__ __attribute__((aligned(16))) float smx[];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t t = blockIdx.x;
  for (int k = threadIdx.x; k < K; k += 256) smx[k] = x[t * K + k];
  __syncthreads();
  const bool vec = (K & 3) == 0 && aligned16(w);
  for (int nb = wv; nb < N; nb += 16) {        // this wave's rows nb, nb + 4, nb + 8, nb + 12
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (vec) {
      for (int k = 4 * lane; k < K; k += 256) {
        const float4 xv = *reinterpret_cast<const float4*>(smx + k);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int n = min(nb + 4 * j, N - 1);   // rows past the table read its last row; their sums are dropped
          const float4 wv4 = *reinterpret_cast<const float4*>(w + (int64_t)n * K + k);
          acc[j] = fmaf(xv.x, wv4.x, fmaf(xv.y, wv4.y, fmaf(xv.z, wv4.z, fmaf(xv.w, wv4.w, acc[j]))));
        }
      }
    } else {
      for (int k = lane; k < K; k += 64) {
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = fmaf(smx[k], w[(int64_t)min(nb + 4 * j, N - 1) * K + k], acc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float sum = wave_sum(acc[j]);
      if (lane == 0 && nb + 4 * j < N) out[t * N + nb + 4 * j] = sum;
    }
  }
}

template <typename T>
int launch_grouped(void* out, const void* in, int64_t in_stride, const void* w, const int32_t* src_row, const int32_t* tile_expert,
                   const int32_t* n_tiles, int gather, int gelu, int N, int K, int64_t max_tiles, bool mfma, int block,
                   hipStream_t stream) {
  const dim3 grid((unsigned)cdiv(N, block), (unsigned)max_tiles);
  if constexpr (!std::is_same<T, float>::value) {
    if (mfma && block == MOE_WIDE) {
      hipLaunchKernelGGL((moe_grouped_linear_wide_kernel<T>), grid, dim3(256), 0, stream, (T*)out, (const T*)in, in_stride,
                         (const T*)w, src_row, tile_expert, n_tiles, gather, gelu, N, K);
      return MI355_OK;
    }
    if (mfma) {
      hipLaunchKernelGGL((moe_grouped_linear_mfma_kernel<T>), grid, dim3(256), 0, stream, (T*)out, (const T*)in, in_stride,
                         (const T*)w, src_row, tile_expert, n_tiles, gather, gelu, N, K);
      return MI355_OK;
    }
  }
  hipLaunchKernelGGL((moe_grouped_linear_valu_kernel<T>), grid, dim3(256), 0, stream, (T*)out, (const T*)in, in_stride,
                     (const T*)w, src_row, tile_expert, n_tiles, gather, gelu, N, K);
  return MI355_OK;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_moe_route_grouped(int32_t* ids, float* weights, const float* logits, const float* correction, int64_t tokens,
                            int num_experts, int top, int n_groups, int keep_groups, float scale, void* stream) {
  MI355_REQUIRE(correction, MI355_ERR_INVALID, "moe_route_grouped: null pointer");
  return mi355_moe_route_scores(ids, weights, logits, correction, tokens, num_experts, top, n_groups, keep_groups, scale, 0, 2, 1,
                                stream);
}

int mi355_moe_route_scores(int32_t* ids, float* weights, const float* logits, const float* correction, int64_t tokens,
                           int num_experts, int top, int n_groups, int keep_groups, float scale, int score_fn, int group_best,
                           int renorm, void* stream) {
  MI355_REQUIRE(ids && weights && logits, MI355_ERR_INVALID, "moe_route_grouped: null pointer");
  MI355_REQUIRE((score_fn == 0 || score_fn == 1) && (group_best == 1 || group_best == 2), MI355_ERR_INVALID,
                "moe_route_grouped: scores are sigmoid (0) or softmax (1), a group counts its best 1 or 2");
  MI355_REQUIRE(tokens >= 0 && num_experts > 0 && n_groups > 0 && num_experts % n_groups == 0 && keep_groups >= 1 &&
                    keep_groups <= n_groups && top >= 1 && top <= num_experts / n_groups * keep_groups,
                MI355_ERR_INVALID, "moe_route_grouped: bad shape");
  MI355_REQUIRE(num_experts <= 2048, MI355_ERR_UNSUPPORTED, "moe_route_grouped: %d experts above 2048", num_experts);
  if (tokens == 0) return MI355_OK;
  const size_t lds = (size_t)4 * (2 * num_experts + n_groups) * sizeof(float);
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((unsigned)((tokens + 3) / 4)), dim3(256), lds, (hipStream_t)stream, ids,
                     weights, logits, correction, tokens, num_experts, top, n_groups, keep_groups, scale, score_fn, group_best, renorm);
  MI355_CHECK_LAUNCH("moe_route_grouped");
  return MI355_OK;
}

constexpr int MOE_TILED = 256;     // rows of a block of the prefill projection kernel (gemm_tiled.hip)

int mi355_moe_block_rows(int wide) { return wide >= 2 ? MOE_TILED : wide == 1 ? MOE_WIDE : MOE_BLOCK; }

int mi355_moe_router_logits(float* out, const float* x, const float* weight, int64_t rows, int n, int k, void* stream) {
  MI355_REQUIRE(out && x && weight, MI355_ERR_INVALID, "moe_router_logits: null pointer");
  MI355_REQUIRE(rows >= 0 && n > 0 && k > 0 && k <= 16384, MI355_ERR_INVALID, "moe_router_logits: bad shape");
  if (rows == 0) return MI355_OK;
  hipLaunchKernelGGL(moe_router_logits_kernel, dim3((unsigned)rows), dim3(256), (size_t)k * sizeof(float), (hipStream_t)stream, out,
                     x, weight, n, k);
  MI355_CHECK_LAUNCH("moe_router_logits");
  return MI355_OK;
}

int mi355_moe_align(int32_t* src_row, int32_t* rows, int32_t* tile_expert, int32_t* n_tiles, const int32_t* ids, int64_t tokens,
                    int top, int num_experts, int block, int64_t padded, void* stream) {
  MI355_REQUIRE(block == MOE_BLOCK || block == MOE_WIDE || block == MOE_TILED, MI355_ERR_INVALID, "moe_align: blocks of %d, %d or %d rows",
                MOE_BLOCK, MOE_WIDE, MOE_TILED);
  MI355_REQUIRE(src_row && rows && tile_expert && n_tiles && ids, MI355_ERR_INVALID, "moe_align: null pointer");
  MI355_REQUIRE(tokens >= 0 && top > 0 && num_experts > 0 && num_experts <= 4096, MI355_ERR_INVALID, "moe_align: bad shape");
  MI355_REQUIRE(padded % block == 0 && padded >= tokens * top + (int64_t)std::min<int64_t>(num_experts, tokens * top) * (block - 1),
                MI355_ERR_INVALID, "moe_align: %lld padded rows cannot hold %lld pairs of %d experts", (long long)padded,
                (long long)(tokens * top), num_experts);
  const size_t lds = (size_t)(2 * num_experts + 1) * sizeof(int);
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), lds, (hipStream_t)stream, src_row, rows, tile_expert, n_tiles, ids,
                     tokens * top, top, num_experts, block, padded);
  MI355_CHECK_LAUNCH("moe_align");
  return MI355_OK;
}

int mi355_moe_grouped_linear(void* out, const void* in, int64_t in_stride, const void* weight, const int32_t* src_row,
                             const int32_t* tile_expert, const int32_t* n_tiles, int gather, int gelu, int64_t padded, int block,
                             int n, int k, int dtype, void* stream) {
  MI355_REQUIRE(out && in && weight && src_row && tile_expert && n_tiles, MI355_ERR_INVALID, "moe_grouped_linear: null pointer");
  if (block == MOE_TILED)
    return mi355_moe_grouped_linear_tiled(out, in, in_stride, weight, gather ? src_row : nullptr, tile_expert, n_tiles, gelu ? 1 : 0,
                                          padded, n, k, dtype, stream);
  MI355_REQUIRE(block == MOE_BLOCK || block == MOE_WIDE, MI355_ERR_INVALID, "moe_grouped_linear: blocks of %d or %d rows", MOE_BLOCK,
                MOE_WIDE);
  MI355_REQUIRE(padded >= 0 && padded % block == 0 && n > 0 && k > 0 && in_stride >= k && padded / block <= 65535,
                MI355_ERR_INVALID, "moe_grouped_linear: bad shape");
  if (padded == 0) return MI355_OK;
  const bool mfma = dtype != MI355_F32 && k % 8 == 0 && in_stride % 8 == 0 && aligned16(in) && aligned16(weight);
  MI355_REQUIRE(block == MOE_BLOCK || mfma, MI355_ERR_UNSUPPORTED,
                "moe_grouped_linear: blocks of %d rows are for 16-bit operands with 16-byte rows", MOE_WIDE);
  int rc = MI355_OK;
  MI355_DISPATCH_DTYPE(dtype, "moe_grouped_linear", {
    rc = launch_grouped<T>(out, in, in_stride, weight, src_row, tile_expert, n_tiles, gather, gelu, n, k, padded / block, mfma,
                           block, (hipStream_t)stream);
  });
  if (rc != MI355_OK) return rc;
  MI355_CHECK_LAUNCH("moe_grouped_linear");
  return MI355_OK;
}
