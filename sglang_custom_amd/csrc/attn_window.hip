// Softmax attention over a sliding window with an optional sink in the denominator, grouped key heads, no rotation:
//     s_j = (q[t, h] . K[j, g]) * scale               for keys j with 0 <= pos(t) - j < window   (window <= 0: every j <= pos)
//     out[t, h] = sum_j exp(s_j) V[j, g] / (exp(sink_h) + sum_j exp(s_j)),        g = h / (H / G)
// over per-layer key / value buffers [slots, G, d] / [slots, G, dv] reached through the request table.  sink null: no such
// term; a sink of 0 adds one to the denominator.  Scores, weights and sums are fp32.
//
// A workgroup takes one run of consecutive tokens of one sequence, one kv head and the query heads that share it as rows of
// one tile, walks the key tiles that any of its rows can see (from the window's lower edge of the run's first token to the
// run's last token) and keeps the running (max, sum) pair per row, started at (sink, 1) -- or (-huge, 0) without a sink.
//   * 16-bit dtypes, d a multiple of 32 and dv of 16: matrix cores, 64 rows per workgroup (S = Q K^T on 16x16x32 MFMA from
//     LDS rows, the weights through LDS in the activation dtype, P V with V read by columns; a row's rescale factor travels
//     through LDS from the wave that owns the row's scores to the waves that own its result columns),
//   * everything else (fp32, odd widths): vector ALU, 16 rows per workgroup, all fp32.
// Prefill portions, decode steps and mixed batches are the same launch, told apart only by the list of runs.  A launch of
// single tokens (a decode step) may cut each token's keys into num_splits ranges: every range leaves its unnormalised sum,
// running maximum and running sum in fp32 scratch (the sink belongs to the first range), and a second launch merges them.
//
// Averaged blocks (pool > 0, window > 0): beside the window's tokens, token i sees one key / value row for every block b of
// `pool` positions whose last position precedes its window, b pool + pool - 1 <= i - window; the rows are the means of the
// block's cached keys and values, kept in pooled buffers at row slot(b pool + pool - 1) / pool_div (mi355_pool_kv_blocks
// writes them when a block's last token enters the cache).  The walk then starts with the tiles of the pooled rows that the
// run's last token sees, masked per row, and goes on with the window's tiles; blocks and tokens share the running (max, sum).
// A gate per head (head_gate, logits) multiplies head h's result by its sigmoid.
#include "common.cuh"

#include <algorithm>
#include <type_traits>

namespace mi355 {
namespace {

constexpr int WA_ROWS = 16;
constexpr int WA_KT = 32;
constexpr float WA_NEG = -1.0e30f;

struct WaArgs {
  void* out;
  const void* q;
  const void* k_cache;
  const void* v_cache;
  const int32_t* req_to_token;
  const int64_t* req_pool_indices;
  const int32_t* tok_req;
  const int64_t* positions;
  const int32_t* blocks;
  const float* sink;
  const void* pooled_k;
  const void* pooled_v;
  const void* gate;        // [token][head] logits of the result's gate, or null
  int64_t gate_token_stride;
  int pool, pool_div;
  float* partial;          // num_splits > 1: [split][token][head][dv + 2] = unnormalised result | running max | running sum
  int64_t q_token_stride, q_head_stride, out_token_stride, out_head_stride, req_to_token_stride, tokens;
  int heads, kv_heads, d, dv, heads_per_tile, window, num_splits;
  float scale;
};

// 16 lanes that hold one row (a DPP row): max and sum over them, every lane gets the result.  Lane exchanges inside quads,
// then across the halves of a half row, then across the row's halves.
template <int CTRL> __device__ __forceinline__ float wa_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float row16_max(float x) {
  x = fmaxf(x, wa_dpp<0xB1>(x));      // quad_perm [1,0,3,2]
  x = fmaxf(x, wa_dpp<0x4E>(x));      // quad_perm [2,3,0,1]
  x = fmaxf(x, wa_dpp<0x141>(x));     // row_half_mirror
  return fmaxf(x, wa_dpp<0x140>(x));  // row_mirror
}
__device__ __forceinline__ float row16_sum(float x) {
  x += wa_dpp<0xB1>(x);
  x += wa_dpp<0x4E>(x);
  x += wa_dpp<0x141>(x);
  return x + wa_dpp<0x140>(x);
}

__device__ __forceinline__ float wa_sigmoid(float z) { return 1.0f / (1.0f + expf(-z)); }

// Vector-ALU kernel.  sm: Qs [16][d] | Ks [KT][d + 1] | Vs [KT][dv] | Ps [16][KT]
template <typename T>
__global__ __launch_bounds__(256) void window_attention_valu_kernel(WaArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int d = a.d, dv = a.dv;
  float* Qs = sm;
  float* Ks = Qs + WA_ROWS * d;
  float* Vs = Ks + WA_KT * (d + 1);
  float* Ps = Vs + WA_KT * dv;
  __shared__ int row_pos[WA_ROWS];
  const int rep = a.heads / a.kv_heads;
  const int chunks = (rep + a.heads_per_tile - 1) / a.heads_per_tile;
  const int g = blockIdx.y / chunks, hc = blockIdx.y - g * chunks;
  const unsigned bx = gridDim.x - 1 - blockIdx.x;
  const int64_t t0 = a.blocks != nullptr ? a.blocks[2 * bx] : bx;
  const int nt = a.blocks != nullptr ? a.blocks[2 * bx + 1] : 1;
  const int b = a.tok_req != nullptr ? a.tok_req[t0] : (int)t0;
  const int32_t* table = a.req_to_token + a.req_pool_indices[b] * a.req_to_token_stride;
  const int h0 = g * rep + hc * a.heads_per_tile;
  const int nh = min(a.heads_per_tile, rep - hc * a.heads_per_tile);
  const int tid = threadIdx.x;
  const T* q = (const T*)a.q;
  for (int e = tid; e < WA_ROWS * d; e += 256) {
    const int r = e / d, i = e - r * d;
    const int tl = r / a.heads_per_tile, hl = r - tl * a.heads_per_tile;
    Qs[e] = (tl < nt && hl < nh) ? to_f32(q[(t0 + tl) * a.q_token_stride + (int64_t)(h0 + hl) * a.q_head_stride + i]) : 0.f;
  }
  if (tid < WA_ROWS) {
    const int tl = tid / a.heads_per_tile, hl = tid - tl * a.heads_per_tile;
    row_pos[tid] = (tl < nt && hl < nh) ? (int)a.positions[t0 + tl] : -1;
  }
  const int first = (int)a.positions[t0];
  const int last = first + nt - 1;                      // the run's tokens are consecutive
  const int lowest = a.window > 0 ? max(0, first - a.window + 1) : 0;
  const int split = blockIdx.z;
  const int all_lo = lowest / WA_KT, all_hi = last / WA_KT + 1;
  // pooled rows that the run's last token sees come first on the walk: ptiles tiles of them, then the window's tiles
  const int nb_run = (a.pool > 0 && a.window > 0 && last - a.window + 1 >= a.pool) ? (last - a.window + 1) / a.pool : 0;
  const int ptiles = (nb_run + WA_KT - 1) / WA_KT;
  const int ntiles = ptiles + all_hi - all_lo;
  const int per = (ntiles + a.num_splits - 1) / a.num_splits;
  const int tile_lo = split * per, tile_hi = min(ntiles, tile_lo + per);
  const int r = tid >> 4, cx = tid & 15;
  const int hl_r = r % a.heads_per_tile;
  float run_m = WA_NEG, run_l = 0.f;
  if (a.sink != nullptr && split == 0) { run_m = a.sink[h0 + min(hl_r, nh - 1)]; run_l = 1.f; }
  float acc[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) acc[m] = 0.f;
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const bool ptile = tile < ptiles;
    const int j0 = (ptile ? tile : all_lo + tile - ptiles) * WA_KT;
    const T* kc = (const T*)(ptile ? a.pooled_k : a.k_cache);
    const T* vc = (const T*)(ptile ? a.pooled_v : a.v_cache);
    __syncthreads();
    for (int e = tid; e < WA_KT * (d + dv); e += 256) {
      const bool isk = e < WA_KT * d;
      const int e2 = isk ? e : e - WA_KT * d;
      const int w = isk ? d : dv;
      const int kk = e2 / w, i = e2 - kk * w;
      const int j = j0 + kk;
      float val = 0.f;
      if (ptile ? j < nb_run : (j >= lowest && j <= last)) {
        const int64_t row = ptile ? table[j * a.pool + a.pool - 1] / a.pool_div : table[j];
        val = to_f32((isk ? kc : vc)[(row * a.kv_heads + g) * w + i]);
      }
      if (isk) Ks[kk * (d + 1) + i] = val;
      else Vs[e2] = val;
    }
    __syncthreads();
    const int rp = row_pos[r];
    float sc[WA_KT / 16];
    float tmax = WA_NEG;
#pragma unroll
    for (int u = 0; u < WA_KT / 16; ++u) {
      const int kk = cx + 16 * u;
      float s = 0.f;
      for (int i = 0; i < d; ++i) s = fmaf(Qs[r * d + i], Ks[kk * (d + 1) + i], s);
      const int j = j0 + kk;
      const bool seen = ptile ? (rp >= 0 && j * a.pool + a.pool - 1 <= rp - a.window) : (j <= rp && (a.window <= 0 || rp - j < a.window));
      sc[u] = seen ? s * a.scale : WA_NEG;
      tmax = fmaxf(tmax, sc[u]);
    }
    tmax = row16_max(tmax);
    const float new_m = fmaxf(run_m, tmax);
    const float alpha = expf(run_m - new_m);          // 1 when nothing changed, also for rows that have seen nothing yet
    float psum = 0.f;
#pragma unroll
    for (int u = 0; u < WA_KT / 16; ++u) {
      const float p = sc[u] > 0.5f * WA_NEG ? expf(sc[u] - new_m) : 0.f;
      Ps[r * WA_KT + cx + 16 * u] = p;
      psum += p;
    }
    psum = row16_sum(psum);
    run_l = run_l * alpha + psum;
    run_m = new_m;
    __syncthreads();
#pragma unroll
    for (int m = 0; m < 16; ++m) acc[m] *= alpha;
    for (int kk = 0; kk < WA_KT; ++kk) {
      const float p = Ps[r * WA_KT + kk];
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        const int c = cx + 16 * m;
        if (c < dv) acc[m] = fmaf(p, Vs[kk * dv + c], acc[m]);
      }
    }
  }
  const int tl = r / a.heads_per_tile, hl = r - tl * a.heads_per_tile;
  if (tl < nt && hl < nh) {
    if (a.num_splits > 1) {
      float* part = a.partial + (((int64_t)split * a.tokens + t0 + tl) * a.heads + h0 + hl) * (dv + 2);
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        const int c = cx + 16 * m;
        if (c < dv) part[c] = acc[m];
      }
      if (cx == 0) { part[dv] = run_m; part[dv + 1] = run_l; }
      return;
    }
    float inv = run_l > 0.f ? 1.0f / run_l : 0.f;
    if (a.gate != nullptr) inv *= wa_sigmoid(to_f32(((const T*)a.gate)[(t0 + tl) * a.gate_token_stride + h0 + hl]));
#pragma unroll
    for (int m = 0; m < 16; ++m) {
      const int c = cx + 16 * m;
      if (c >= dv) continue;
      ((T*)a.out)[(t0 + tl) * a.out_token_stride + (int64_t)(h0 + hl) * a.out_head_stride + c] = from_f32<T>(acc[m] * inv);
    }
  }
}

// out[t, h] = sum_s acc_s e^(m_s - M) / sum_s l_s e^(m_s - M), M = max_s m_s, over the key ranges in order.  One wave per
// (token, head).
template <typename T>
__global__ __launch_bounds__(256) void window_attention_merge_kernel(T* __restrict__ out, const float* __restrict__ partial,
                                                                     int64_t tokens, int heads, int dv, int num_splits,
                                                                     int64_t out_token_stride, int64_t out_head_stride,
                                                                     const T* __restrict__ gate, int64_t gate_token_stride) {
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int64_t idx = (int64_t)blockIdx.x * 4 + wv;
  if (idx >= tokens * heads) return;
  const int64_t t = idx / heads;
  const int h = (int)(idx - t * heads);
  const int64_t stride = tokens * heads * (int64_t)(dv + 2);
  const float* p0 = partial + idx * (dv + 2);
  float M = WA_NEG;
  for (int k = 0; k < num_splits; ++k) M = fmaxf(M, p0[k * stride + dv]);
  float L = 0.f;
  for (int k = 0; k < num_splits; ++k) L += p0[k * stride + dv + 1] * expf(p0[k * stride + dv] - M);
  float inv = L > 0.f ? 1.0f / L : 0.f;
  if (gate != nullptr) inv *= wa_sigmoid(to_f32(gate[t * gate_token_stride + h]));
  for (int c = lane; c < dv; c += 64) {
    float s = 0.f;
    for (int k = 0; k < num_splits; ++k) s += p0[k * stride + c] * expf(p0[k * stride + dv] - M);
    out[t * out_token_stride + (int64_t)h * out_head_stride + c] = from_f32<T>(s * inv);
  }
}

// Matrix-core kernel for 16-bit dtypes, d % 32 == 0, dv % 16 == 0.  Four waves, 64 (token, head) rows.  Per key tile of 32:
//   S: wave w computes its 16 rows x 32 keys with 2 * d / 32 MFMA 16x16x32 (A = Q rows, B = K rows from LDS), masks, updates
//      its rows' running (max, sum), leaves P in LDS as T and each row's rescale factor in LDS as fp32;
//   O: wave w owns CT 16-column tiles of the result for ALL row tiles: it rescales them by the rows' factors and adds P V,
//      one MFMA 16x16x32 per (row tile, column tile), each V fragment read (transposed) once per workgroup.
// The next tile's K and V rows are requested from global memory into registers before the current tile's products and
// stored to LDS after them.
// sm: Qs [64][d + 8] | Ks [32][d + 8] | Vs [32][dv + 8] | Ps [64][32 + 8]   (all T)
constexpr int WAM_ROWS = 64;
constexpr int WAM_MAXC = 4;      // 16-byte chunks of a K (V) tile per thread: d (dv) up to 256

template <typename T, int CT>
__global__ __launch_bounds__(256) void window_attention_mfma_kernel(WaArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smraw[];
  const int d = a.d, dv = a.dv;
  const int qld = d + 8, vld = dv + 8, pld = WA_KT + 8;
  T* Qs = reinterpret_cast<T*>(smraw);
  T* Ks = Qs + WAM_ROWS * qld;
  T* Vs = Ks + WA_KT * qld;
  T* Ps = Vs + WA_KT * vld;
  __shared__ int row_pos[WAM_ROWS];
  __shared__ float row_alpha[WAM_ROWS], row_l[WAM_ROWS], row_m[WAM_ROWS];
  const int rep = a.heads / a.kv_heads;
  const int HR = a.heads_per_tile;
  const int chunks = (rep + HR - 1) / HR;
  const int g = blockIdx.y / chunks, hc = blockIdx.y - g * chunks;
  const unsigned bx = gridDim.x - 1 - blockIdx.x;
  const int64_t t0 = a.blocks != nullptr ? a.blocks[2 * bx] : bx;
  const int nt = a.blocks != nullptr ? a.blocks[2 * bx + 1] : 1;
  const int b = a.tok_req != nullptr ? a.tok_req[t0] : (int)t0;
  const int32_t* table = a.req_to_token + a.req_pool_indices[b] * a.req_to_token_stride;
  const int h0 = g * rep + hc * HR;
  const int nh = min(HR, rep - hc * HR);
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const T* q = (const T*)a.q;
  const int dch = d / 8, vch = dv / 8;           // 16-byte chunks per row
  const int live_rows = nt * HR;                 // rows at or past this hold no (token, head)
  for (int e = tid; e < WAM_ROWS * dch; e += 256) {
    const int r = e / dch, ch = e - r * dch;
    const int tl = r / HR, hl = r - tl * HR;
    Vec<T, 8> val;
    if (tl < nt && hl < nh) {
      val = ldvec<T, 8>(q + (t0 + tl) * a.q_token_stride + (int64_t)(h0 + hl) * a.q_head_stride + ch * 8);
    } else {
#pragma unroll
      for (int x = 0; x < 8; ++x) val.v[x] = from_f32<T>(0.f);
    }
    lds_store16(Qs + r * qld + ch * 8, val);
  }
  if (tid < WAM_ROWS) {
    const int tl = tid / HR, hl = tid - tl * HR;
    row_pos[tid] = (tl < nt && hl < nh) ? (int)a.positions[t0 + tl] : -1;
  }
  const int first = (int)a.positions[t0];
  const int last = first + nt - 1;
  const int lowest = a.window > 0 ? max(0, first - a.window + 1) : 0;
  const int split = blockIdx.z;
  const int all_lo = lowest / WA_KT, all_hi = last / WA_KT + 1;
  // pooled rows that the run's last token sees come first on the walk: ptiles tiles of them, then the window's tiles
  const int nb_run = (a.pool > 0 && a.window > 0 && last - a.window + 1 >= a.pool) ? (last - a.window + 1) / a.pool : 0;
  const int ptiles = (nb_run + WA_KT - 1) / WA_KT;
  const int ntiles = ptiles + all_hi - all_lo;
  const int per = (ntiles + a.num_splits - 1) / a.num_splits;
  const int tile_lo = split * per, tile_hi = min(ntiles, tile_lo + per);
  const int nblk = dv / 16;
  // this lane's four score rows: 16 wv + 4 lg + x
  float run_m[4], run_l[4];
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const int r = 16 * wv + 4 * lg + x;
    const int hl = r % HR;
    if (a.sink != nullptr && split == 0) { run_m[x] = a.sink[h0 + min(hl, nh - 1)]; run_l[x] = 1.f; }
    else { run_m[x] = WA_NEG; run_l[x] = 0.f; }
  }
  f32x4 acc[4][CT];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int c = 0; c < CT; ++c) acc[rt][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  using Frag = typename Mfma<T>::frag;
  Vec<T, 8> kreg[WAM_MAXC], vreg[WAM_MAXC];
  int64_t ksrc[WAM_MAXC], vsrc[WAM_MAXC];
  // every load is unconditional: chunk numbers past the tile's last one are clamped (and never stored), keys outside
  // [0, last] (pooled rows past the last one the run sees) are clamped to a valid row (and masked below)
  auto load_slots = [&](int tile) {
    const bool ptile = tile < ptiles;
    const int j0 = (ptile ? tile : all_lo + tile - ptiles) * WA_KT;
    kc = (const T*)(ptile ? a.pooled_k : a.k_cache);
    vc = (const T*)(ptile ? a.pooled_v : a.v_cache);
#pragma unroll
    for (int u = 0; u < WAM_MAXC; ++u) {
      const int ek = min(tid + 256 * u, WA_KT * dch - 1), ev = min(tid + 256 * u, WA_KT * vch - 1);
      const int kk = ek / dch, kv = ev / vch;
      const int64_t rk = ptile ? table[min(j0 + kk, nb_run - 1) * a.pool + a.pool - 1] / a.pool_div : table[min(j0 + kk, last)];
      const int64_t rv = ptile ? table[min(j0 + kv, nb_run - 1) * a.pool + a.pool - 1] / a.pool_div : table[min(j0 + kv, last)];
      ksrc[u] = (rk * a.kv_heads + g) * d + (ek - kk * dch) * 8;
      vsrc[u] = (rv * a.kv_heads + g) * dv + (ev - kv * vch) * 8;
    }
  };
  auto request = [&]() {
#pragma unroll
    for (int u = 0; u < WAM_MAXC; ++u) {
      kreg[u] = ldvec<T, 8>(kc + ksrc[u]);
      vreg[u] = ldvec<T, 8>(vc + vsrc[u]);
    }
  };
  if (tile_lo < tile_hi) {
    load_slots(tile_lo);
    request();
    load_slots(min(tile_lo + 1, tile_hi - 1));
  }
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const bool ptile = tile < ptiles;
    const int j0 = (ptile ? tile : all_lo + tile - ptiles) * WA_KT;
    __syncthreads();                             // the last tile's readers are done (and, the first time, Qs is written)
#pragma unroll
    for (int u = 0; u < WAM_MAXC; ++u) {
      const int e = tid + 256 * u;
      if (e < WA_KT * dch) {
        const int kk = e / dch, ch = e - kk * dch;
        lds_store16(Ks + kk * qld + ch * 8, kreg[u]);
      }
      if (e < WA_KT * vch) {
        const int kk = e / vch, ch = e - kk * vch;
        lds_store16(Vs + kk * vld + ch * 8, vreg[u]);
      }
    }
    __syncthreads();
    if (tile + 1 < tile_hi) {                    // in flight during this tile's products
      request();
      load_slots(min(tile + 2, tile_hi - 1));
    }
    if (16 * wv < live_rows) {
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
      for (int c = 0; c < d; c += 32) {
        const Frag af = lds_load16<Frag>(Qs + (16 * wv + li) * qld + c + 8 * lg);
        const Frag b0 = lds_load16<Frag>(Ks + li * qld + c + 8 * lg);
        const Frag b1 = lds_load16<Frag>(Ks + (16 + li) * qld + c + 8 * lg);
        s0 = Mfma<T>::run(af, b0, s0);
        s1 = Mfma<T>::run(af, b1, s1);
      }
      // result lane: rows 16 wv + 4 lg + x, key columns li (s0) and 16 + li (s1); a row's 32 scores sit in 16 lanes
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int r = 16 * wv + 4 * lg + x;
        const int rp = row_pos[r];
        const int ja = j0 + li, jb = j0 + 16 + li;
        const bool va = ptile ? (rp >= 0 && ja * a.pool + a.pool - 1 <= rp - a.window) : (ja <= rp && (a.window <= 0 || rp - ja < a.window));
        const bool vb = ptile ? (rp >= 0 && jb * a.pool + a.pool - 1 <= rp - a.window) : (jb <= rp && (a.window <= 0 || rp - jb < a.window));
        const float sa = va ? s0[x] * a.scale : WA_NEG, sb = vb ? s1[x] * a.scale : WA_NEG;
        const float new_m = fmaxf(run_m[x], row16_max(fmaxf(sa, sb)));
        const float alpha = __expf(run_m[x] - new_m);
        const float pa = va ? __expf(sa - new_m) : 0.f, pb = vb ? __expf(sb - new_m) : 0.f;
        run_l[x] = run_l[x] * alpha + row16_sum(pa + pb);
        run_m[x] = new_m;
        lds_store2(Ps + r * pld + li, from_f32<T>(pa));
        lds_store2(Ps + r * pld + 16 + li, from_f32<T>(pb));
        if (li == 0) row_alpha[r] = alpha;
      }
    } else if (lane < 16) {
      row_alpha[16 * wv + lane] = 1.f;
    }
    __syncthreads();
    {
      const T* vrow = Vs + (8 * lg + (li >> 2)) * vld + 4 * (li & 3) + 16 * CT * wv;
      typename TrRead<T>::v4 lo[CT], hi[CT];
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        if (CT * wv + c < nblk) {
          lo[c] = TrRead<T>::run(vrow + 16 * c);
          hi[c] = TrRead<T>::run(vrow + 4 * vld + 16 * c);
        }
      }
#pragma unroll
      for (int rt = 0; rt < 4; ++rt) {
        if (16 * rt < live_rows) {
          const Frag pa = lds_load16<Frag>(Ps + (16 * rt + li) * pld + 8 * lg);
          float al[4];
#pragma unroll
          for (int x = 0; x < 4; ++x) al[x] = row_alpha[16 * rt + 4 * lg + x];
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            if (CT * wv + c < nblk) {
#pragma unroll
              for (int x = 0; x < 4; ++x) acc[rt][c][x] *= al[x];
              typename TrRead<T>::v4 both[2] = {lo[c], hi[c]};
              acc[rt][c] = Mfma<T>::run(pa, __builtin_bit_cast(Frag, both), acc[rt][c]);
            }
          }
        }
      }
    }
  }
  __syncthreads();
  if (li == 0) {
#pragma unroll
    for (int x = 0; x < 4; ++x) { row_l[16 * wv + 4 * lg + x] = run_l[x]; row_m[16 * wv + 4 * lg + x] = run_m[x]; }
  }
  __syncthreads();
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      if (CT * wv + c >= nblk) continue;
      const int col = 16 * (CT * wv + c) + li;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int r = 16 * rt + 4 * lg + x;
        const int tl = r / HR, hl = r - tl * HR;
        if (tl >= nt || hl >= nh) continue;
        if (a.num_splits > 1) {
          float* part = a.partial + (((int64_t)split * a.tokens + t0 + tl) * a.heads + h0 + hl) * (dv + 2);
          part[col] = acc[rt][c][x];
          if (col == 0) { part[dv] = row_m[r]; part[dv + 1] = row_l[r]; }
          continue;
        }
        const float l = row_l[r];
        float o = l > 0.f ? acc[rt][c][x] / l : 0.f;
        if (a.gate != nullptr) o *= wa_sigmoid(to_f32(((const T*)a.gate)[(t0 + tl) * a.gate_token_stride + h0 + hl]));
        ((T*)a.out)[(t0 + tl) * a.out_token_stride + (int64_t)(h0 + hl) * a.out_head_stride + col] = from_f32<T>(o);
      }
    }
  }
}

// One workgroup per token of the step; only a token whose position ends a block of `pool` does anything: it averages the
// block's cached rows into the pooled buffers' row for the block.  A row is kw key features followed (in another buffer) by
// vw value features, taken V at a time (16 bytes when the shapes allow, else one); the workgroup's threads form R lanes of
// rows x C columns of such vectors, lane r sums rows r, r + R, ... in fp32, the lanes' sums meet in LDS in lane order, one
// multiplication by 1 / pool.  The order of the additions depends on the shapes alone, never on how a prompt was cut.
template <typename T, int V>
__global__ __launch_bounds__(256) void pool_kv_blocks_kernel(T* __restrict__ pk, T* __restrict__ pv, const T* __restrict__ kc,
                                                             const T* __restrict__ vc, const int32_t* __restrict__ req_to_token,
                                                             const int64_t* __restrict__ req_pool_indices,
                                                             const int32_t* __restrict__ tok_req,
                                                             const int64_t* __restrict__ positions, int64_t req_to_token_stride,
                                                             int kw, int vw, int pool, int pool_div) {
  __shared__ float part[256 * V];
  const int64_t t = blockIdx.x;
  const int pos = (int)positions[t];
  if ((pos + 1) % pool != 0) return;
  const int b = tok_req != nullptr ? tok_req[t] : (int)t;
  const int32_t* table = req_to_token + req_pool_indices[b] * req_to_token_stride + (pos - pool + 1);
  const int64_t dst = table[pool - 1] / pool_div;
  const float inv = 1.0f / (float)pool;
  const int nk = kw / V, nv = (kw + vw) / V;           // vectors per row: keys first, then values
  const int C = min(nv, 256);                          // columns handled at a time
  int R = 256 / C;                                     // lanes of rows
  R = min(R, pool);
  const int tid = threadIdx.x;
  const int col = tid % C, lane = tid / C;
  for (int c0 = 0; c0 < nv; c0 += C) {
    const int c = c0 + col;
    const bool live = lane < R && c < nv;
    const bool isk = c < nk;
    const T* src = isk ? kc : vc;
    const int w = isk ? kw : vw;
    const int off = (isk ? c : c - nk) * V;
    float acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = 0.f;
    if (live) {
      int j = lane;
      for (; j + 3 * R < pool; j += 4 * R) {           // four rows in flight
        const Vec<T, V> a0 = ldvec<T, V>(src + (int64_t)table[j] * w + off);
        const Vec<T, V> a1 = ldvec<T, V>(src + (int64_t)table[j + R] * w + off);
        const Vec<T, V> a2 = ldvec<T, V>(src + (int64_t)table[j + 2 * R] * w + off);
        const Vec<T, V> a3 = ldvec<T, V>(src + (int64_t)table[j + 3 * R] * w + off);
#pragma unroll
        for (int k = 0; k < V; ++k) acc[k] = ((acc[k] + to_f32(a0.v[k])) + to_f32(a1.v[k])) + (to_f32(a2.v[k]) + to_f32(a3.v[k]));
      }
      for (; j < pool; j += R) {
        const Vec<T, V> a0 = ldvec<T, V>(src + (int64_t)table[j] * w + off);
#pragma unroll
        for (int k = 0; k < V; ++k) acc[k] += to_f32(a0.v[k]);
      }
    }
    __syncthreads();                                   // the last pass's readers are done
    if (live) {
#pragma unroll
      for (int k = 0; k < V; ++k) part[(lane * C + col) * V + k] = acc[k];
    }
    __syncthreads();
    if (live && lane == 0) {
      Vec<T, V> out;
#pragma unroll
      for (int k = 0; k < V; ++k) {
        float sum = part[col * V + k];
        for (int r = 1; r < R; ++r) sum += part[(r * C + col) * V + k];
        out.v[k] = from_f32<T>(sum * inv);
      }
      stvec<T, V>((isk ? pk : pv) + dst * w + off, out);
    }
  }
}

inline bool wa_mfma_shape(int dtype, int d, int dv) {
  return dtype != MI355_F32 && d % 32 == 0 && dv % 16 == 0 && d <= 32 * WAM_MAXC * 2 && dv <= 32 * WAM_MAXC * 2;
}

template <typename T> int launch_window(const WaArgs& a, dim3 grid, bool mfma, hipStream_t stream) {
  if constexpr (!std::is_same<T, float>::value) {
    if (mfma) {
      const size_t lds = ((size_t)(WAM_ROWS + WA_KT) * (a.d + 8) + (size_t)WA_KT * (a.dv + 8) + WAM_ROWS * (WA_KT + 8)) * sizeof(T);
      const int nblk = a.dv / 16;
#define MI355_WA_LAUNCH(CT)                                                                                                    \
  do {                                                                                                                         \
    if (lds > 64 * 1024) {                                                                                                     \
      hipError_t e = hipFuncSetAttribute((const void*)window_attention_mfma_kernel<T, CT>,                                     \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                \
      MI355_REQUIRE(e == hipSuccess, MI355_ERR_LAUNCH, "window_attention: %zu bytes of LDS refused", lds);                     \
    }                                                                                                                          \
    hipLaunchKernelGGL((window_attention_mfma_kernel<T, CT>), grid, dim3(256), lds, stream, a);                                \
  } while (0)
      if (nblk <= 4) MI355_WA_LAUNCH(1);
      else if (nblk <= 8) MI355_WA_LAUNCH(2);
      else MI355_WA_LAUNCH(4);
#undef MI355_WA_LAUNCH
      return MI355_OK;
    }
  }
  const size_t lds = ((size_t)WA_ROWS * a.d + (size_t)WA_KT * (a.d + 1) + (size_t)WA_KT * a.dv + WA_ROWS * WA_KT) * sizeof(float);
  if (lds > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)window_attention_valu_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    MI355_REQUIRE(e == hipSuccess, MI355_ERR_LAUNCH, "window_attention: %zu bytes of LDS refused", lds);
  }
  hipLaunchKernelGGL((window_attention_valu_kernel<T>), grid, dim3(256), lds, stream, a);
  return MI355_OK;
}

inline int wa_heads_per_tile(int heads, int kv_heads, int rows) { return std::min(heads / kv_heads, rows); }

}  // namespace
}  // namespace mi355

using namespace mi355;

int mi355_window_attention_block_tokens(int heads, int kv_heads, int head_dim, int v_head_dim, int dtype) {
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads) return 0;
  const int rows = wa_mfma_shape(dtype, head_dim, v_head_dim) ? WAM_ROWS : WA_ROWS;
  return std::max(1, rows / wa_heads_per_tile(heads, kv_heads, rows));
}

int mi355_window_attention(void* out, const void* q, const void* k_cache, const void* v_cache, const int32_t* req_to_token,
                           const int64_t* req_pool_indices, const int32_t* tok_req, const int64_t* positions,
                           const int32_t* blocks, int64_t num_blocks, const float* sink, int64_t q_token_stride,
                           int64_t q_head_stride, int64_t out_token_stride, int64_t out_head_stride, int64_t req_to_token_stride,
                           int heads, int kv_heads, int head_dim, int v_head_dim, int window, float scale, int num_splits,
                           float* split_scratch, int64_t tokens, int max_run, int dtype, void* stream) {
  return mi355_window_attention_pooled(out, q, k_cache, v_cache, nullptr, nullptr, req_to_token, req_pool_indices, tok_req, positions,
                                       blocks, num_blocks, sink, nullptr, 0, q_token_stride, q_head_stride, out_token_stride,
                                       out_head_stride, req_to_token_stride, heads, kv_heads, head_dim, v_head_dim, window, 0, 1,
                                       scale, num_splits, split_scratch, tokens, max_run, dtype, stream);
}

int mi355_window_attention_pooled(void* out, const void* q, const void* k_cache, const void* v_cache, const void* pooled_k,
                                  const void* pooled_v, const int32_t* req_to_token, const int64_t* req_pool_indices,
                                  const int32_t* tok_req, const int64_t* positions, const int32_t* blocks, int64_t num_blocks,
                                  const float* sink, const void* head_gate, int64_t gate_token_stride, int64_t q_token_stride,
                                  int64_t q_head_stride, int64_t out_token_stride, int64_t out_head_stride,
                                  int64_t req_to_token_stride, int heads, int kv_heads, int head_dim, int v_head_dim, int window,
                                  int pool, int pool_div, float scale, int num_splits, float* split_scratch, int64_t tokens,
                                  int max_run, int dtype, void* stream) {
  MI355_REQUIRE(pool >= 0 && pool_div >= 1 && (pool == 0 || (pooled_k && pooled_v && window > 0)), MI355_ERR_INVALID,
                "window_attention: averaged blocks need their buffers and a window");
  MI355_REQUIRE(head_gate == nullptr || gate_token_stride >= heads, MI355_ERR_INVALID, "window_attention: bad gate stride");
  MI355_REQUIRE(num_splits >= 1 && num_splits <= 64 && (num_splits == 1 || (split_scratch && blocks == nullptr)), MI355_ERR_INVALID,
                "window_attention: key splits serve launches of one token per run and need scratch");
  MI355_REQUIRE(out && q && k_cache && v_cache && req_to_token && req_pool_indices && positions, MI355_ERR_INVALID,
                "window_attention: null pointer");
  MI355_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && head_dim > 0 && v_head_dim > 0 && tokens >= 0 &&
                    num_blocks >= 0, MI355_ERR_INVALID, "window_attention: bad shape");
  MI355_REQUIRE(head_dim <= 512 && v_head_dim <= 256, MI355_ERR_UNSUPPORTED, "window_attention: head width %d / %d not served",
                head_dim, v_head_dim);
  MI355_REQUIRE(blocks != nullptr || num_blocks == tokens, MI355_ERR_INVALID, "window_attention: without runs, one block per token");
  if (num_blocks == 0) return MI355_OK;
  WaArgs a;
  a.out = out; a.q = q; a.k_cache = k_cache; a.v_cache = v_cache; a.req_to_token = req_to_token;
  a.req_pool_indices = req_pool_indices; a.tok_req = tok_req; a.positions = positions; a.blocks = blocks; a.sink = sink;
  a.pooled_k = pooled_k; a.pooled_v = pooled_v; a.gate = head_gate; a.gate_token_stride = gate_token_stride; a.pool = pool;
  a.pool_div = pool_div;
  a.q_token_stride = q_token_stride; a.q_head_stride = q_head_stride; a.out_token_stride = out_token_stride;
  a.out_head_stride = out_head_stride; a.req_to_token_stride = req_to_token_stride; a.tokens = tokens; a.heads = heads;
  // the matrix-core kernel needs 16-byte rows everywhere; a caller whose q is laid out otherwise gets the vector-ALU kernel,
  // whose runs are shorter: max_run says how long the caller's runs may be, and a launch that cannot take them is refused
  const bool mfma = wa_mfma_shape(dtype, head_dim, v_head_dim) && q_token_stride % 8 == 0 && q_head_stride % 8 == 0 &&
                    aligned16(q) && aligned16(k_cache) && aligned16(v_cache) && (pool == 0 || (aligned16(pooled_k) && aligned16(pooled_v)));
  const int rows = mfma ? WAM_ROWS : WA_ROWS;
  a.kv_heads = kv_heads; a.d = head_dim; a.dv = v_head_dim; a.heads_per_tile = wa_heads_per_tile(heads, kv_heads, rows);
  a.window = window; a.scale = scale; a.num_splits = num_splits; a.partial = split_scratch;
  const int tokens_per_tile = std::max(1, rows / a.heads_per_tile);
  MI355_REQUIRE(max_run >= 1 && max_run <= tokens_per_tile, MI355_ERR_UNSUPPORTED,
                "window_attention: runs of up to %d tokens, this launch takes %d", max_run, tokens_per_tile);
  const int rep = heads / kv_heads;
  const int chunks = (rep + a.heads_per_tile - 1) / a.heads_per_tile;
  const dim3 grid((unsigned)num_blocks, (unsigned)(kv_heads * chunks), (unsigned)num_splits);
  MI355_REQUIRE(kv_heads * chunks <= 65535, MI355_ERR_UNSUPPORTED, "window_attention: too many heads");
  int rc = MI355_OK;
  MI355_DISPATCH_DTYPE(dtype, "window_attention", { rc = launch_window<T>(a, grid, mfma, (hipStream_t)stream); });
  if (rc != MI355_OK) return rc;
  MI355_CHECK_LAUNCH("window_attention");
  if (num_splits > 1) {
    const unsigned g2 = (unsigned)((tokens * heads + 3) / 4);
    MI355_DISPATCH_DTYPE(dtype, "window_attention", {
      hipLaunchKernelGGL((window_attention_merge_kernel<T>), dim3(g2), dim3(256), 0, (hipStream_t)stream, (T*)out, split_scratch, tokens,
                         heads, v_head_dim, num_splits, out_token_stride, out_head_stride, (const T*)head_gate, gate_token_stride);
    });
    MI355_CHECK_LAUNCH("window_attention(merge)");
  }
  return MI355_OK;
}

int mi355_pool_kv_blocks(void* pooled_k, void* pooled_v, const void* k_cache, const void* v_cache, const int32_t* req_to_token,
                         const int64_t* req_pool_indices, const int32_t* tok_req, const int64_t* positions, int64_t tokens,
                         int64_t req_to_token_stride, int kv_heads, int head_dim, int v_head_dim, int pool, int pool_div, int dtype,
                         void* stream) {
  MI355_REQUIRE(pooled_k && pooled_v && k_cache && v_cache && req_to_token && req_pool_indices && positions, MI355_ERR_INVALID,
                "pool_kv_blocks: null pointer");
  MI355_REQUIRE(tokens >= 0 && tokens <= 0x7fffffff && kv_heads > 0 && head_dim > 0 && v_head_dim > 0 && pool >= 1 && pool_div >= 1,
                MI355_ERR_INVALID, "pool_kv_blocks: bad shape");
  if (tokens == 0) return MI355_OK;
  const int kw = kv_heads * head_dim, vw = kv_heads * v_head_dim;
  const int vecw = dtype == MI355_F32 ? 4 : 8;
  const bool vec = kw % vecw == 0 && vw % vecw == 0 && aligned16(pooled_k) && aligned16(pooled_v) && aligned16(k_cache) && aligned16(v_cache);
  MI355_DISPATCH_DTYPE(dtype, "pool_kv_blocks", {
    constexpr int V = 16 / sizeof(T);
    if (vec)
      hipLaunchKernelGGL((pool_kv_blocks_kernel<T, V>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, (T*)pooled_k,
                         (T*)pooled_v, (const T*)k_cache, (const T*)v_cache, req_to_token, req_pool_indices, tok_req, positions,
                         req_to_token_stride, kw, vw, pool, pool_div);
    else
      hipLaunchKernelGGL((pool_kv_blocks_kernel<T, 1>), dim3((unsigned)tokens), dim3(256), 0, (hipStream_t)stream, (T*)pooled_k,
                         (T*)pooled_v, (const T*)k_cache, (const T*)v_cache, req_to_token, req_pool_indices, tok_req, positions,
                         req_to_token_stride, kw, vw, pool, pool_div);
  });
  MI355_CHECK_LAUNCH("pool_kv_blocks");
  return MI355_OK;
}
