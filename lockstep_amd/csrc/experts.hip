// A feed-forward of many small experts of which each token uses a few (routing on the device, no
// word of it read by the host):
//
//   z[t]        = router logits of token t (float, computed by the caller's matrix product) + bias
//   chosen(t)   = the `top` experts with the largest z[t] (the lower index wins a tie), in that order
//   w[t, k]     = softmax over the chosen logits alone
//   expert e    : y = act(W_gate[e] x, W_up[e] x),  out = W_down[e] y
//                 act(g, u) = g' sigmoid(alpha g') (u' + shift),  g' = min(g, limit),  u' = clamp(u, -limit, limit)
//                 (an infinite limit, alpha 1 and shift 0: the plain gated unit silu(g) u)
//   P[k][t]     = w[t, k] * expert chosen(t)[k] (x[t])        (float; the caller adds the slices in order)
//
// (1) route: a wave a token picks the experts and their weights.  (2) group: the (token, choice) pairs
// are put in the order of their experts (a stable counting sort: a wave an expert counts its pairs by
// ballots, then places them; one workgroup does (1) and (2) for a step of few tokens), and every
// expert's pairs are cut into tiles of ROWS rows; the tile list has a fixed capacity that depends on the sizes only, unused
// tiles are marked.  (3) the gate and up products of every tile with the activation as epilogue; (4)
// the down products, scaled and scattered to P.  Products use the 16x16 MFMA atom with the weight
// rows as first operand (a lane ends with four consecutive output columns of one row); a row's
// contraction is one chain over ascending K from zero, so its bits do not depend on the tile it is in
// or on what else is in the step.  A weight fragment is loaded once and multiplied with all RT row
// tiles of a wave.

#include "common.h"

namespace ls {

constexpr int kMaxTop = 16;

__device__ __forceinline__ float sigmoid_e(float x) { return 1.0f / (1.0f + expf(-x)); }

// ---------------------------------------------------------------------------
// (1) A wave a token.  Lane l holds the logits of experts l, l + 64, ...; a pick is the best of every lane's
// best (the larger value, then the lower index), found by exchanges across the wave; lane k < top keeps the
// k-th pick.  expert [T][top] int, weight [T][top] float.
// ---------------------------------------------------------------------------
constexpr int kMaxPerLane = 8;   // experts a lane holds: up to 512 experts

// scoring 0: the weights are the softmax over the chosen logits; 1: each chosen expert weighs the sigmoid of its own
// logit, and nothing is renormalised (the sigmoid grows with the logit, so the largest logits are the largest scores).
__device__ __forceinline__ void pick_top(const float* __restrict__ row, const float* __restrict__ bias, int E, int top,
                                         int lane, int* __restrict__ picked, float* __restrict__ share, int scoring) {
  float mine[kMaxPerLane];
#pragma unroll
  for (int m = 0; m < kMaxPerLane; ++m) {
    const int e = lane + 64 * m;
    mine[m] = e < E ? row[e] + (bias ? bias[e] : 0.f) : 0.f;
  }
  unsigned taken = 0;
  int my_pick = 0;
  float my_value = 0.f, first = 0.f;
  for (int k = 0; k < top; ++k) {
    float best_v = 0.f;
    int best = 0x7fffffff;
#pragma unroll
    for (int m = 0; m < kMaxPerLane; ++m) {
      const int e = lane + 64 * m;
      if (e < E && !((taken >> m) & 1u) && (best == 0x7fffffff || mine[m] > best_v)) {
        best_v = mine[m];
        best = e;
      }
    }
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) {
      const float other_v = __shfl_xor(best_v, step, kWave);
      const int other = __shfl_xor(best, step, kWave);
      const bool take = other != 0x7fffffff && (best == 0x7fffffff || other_v > best_v || (other_v == best_v && other < best));
      best_v = take ? other_v : best_v;
      best = take ? other : best;
    }
    if ((best & 63) == lane) taken |= 1u << (best >> 6);
    if (k == 0) first = best_v;
    if (lane == k) {
      my_pick = best;
      my_value = best_v;
    }
  }
  const float ex = lane < top ? expf(my_value - first) : 0.f;   // (the first pick is the largest)
  const float sum = wave_sum(ex);
  if (lane < top) {
    picked[lane] = my_pick;
    share[lane] = scoring == 1 ? sigmoid_e(my_value) : ex / sum;
  }
}

// The experts of a token come from a table instead of a router: row token_id of table [vocab][top] names them (its
// entries differ), and every one weighs 1 / top.
__global__ __launch_bounds__(256) void route_table_kernel(const int* __restrict__ token_ids, const int* __restrict__ table,
                                                          int n_tokens, int top, int* __restrict__ expert,
                                                          float* __restrict__ weight) {
  const long pair = (long)blockIdx.x * 256 + threadIdx.x;
  if (pair >= (long)n_tokens * top) return;
  expert[pair] = table[(long)token_ids[pair / top] * top + pair % top];
  weight[pair] = 1.0f / (float)top;
}

__global__ __launch_bounds__(256) void route_topk_kernel(const float* __restrict__ z, long ldz,
                                                         const float* __restrict__ bias, int n_tokens, int E, int top,
                                                         int* __restrict__ expert, float* __restrict__ weight, int scoring) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= n_tokens) return;
  pick_top(z + (long)t * ldz, bias, E, top, threadIdx.x & 63, expert + (long)t * top, weight + (long)t * top, scoring);
}

// ---------------------------------------------------------------------------
// (2) order [P]: the pairs (token * top + choice) sorted by expert, stable.  tiles [cap][4]: expert (-1: unused),
// first place in order, rows, 0.  A wave an expert: it counts its pairs by ballots, adds up the counts of the
// experts before it, writes its tiles and places its pairs.  Many pairs: two launches of a wave an expert
// (count; place).  Few: one workgroup that also picks the experts, with the picks and counts in LDS.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int count_pairs(const int* expert, int P, int e, int lane) {
  int n = 0;
  for (int p0 = 0; p0 < P; p0 += 256) {   // (four loads requested together)
    int got[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) got[u] = p0 + 64 * u + lane < P ? expert[p0 + 64 * u + lane] : -1;
#pragma unroll
    for (int u = 0; u < 4; ++u) n += __popcll(__ballot(got[u] == e));
  }
  return n;
}

__device__ __forceinline__ void place_pairs(const int* expert, const int* counts, int P, int E, int e, int lane,
                                            int rows_a_tile, int* __restrict__ order, int* __restrict__ tiles, int cap) {
  int base = 0, tile = 0;
  for (int j0 = 0; j0 < e; j0 += 64) {   // (sums of whole numbers: any order)
    const int c = j0 + lane < e ? counts[j0 + lane] : 0;
    int b = c, t = (c + rows_a_tile - 1) / rows_a_tile;
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) {
      b += __shfl_xor(b, step, kWave);
      t += __shfl_xor(t, step, kWave);
    }
    base += b;
    tile += t;
  }
  const int n = counts[e];
  for (int i = lane; i * rows_a_tile < n; i += 64) {
    if (tile + i < cap) {
      tiles[4 * (tile + i)] = e;
      tiles[4 * (tile + i) + 1] = base + i * rows_a_tile;
      tiles[4 * (tile + i) + 2] = min(rows_a_tile, n - i * rows_a_tile);
      tiles[4 * (tile + i) + 3] = 0;
    }
  }
  if (e == E - 1) {
    const int used = tile + (n + rows_a_tile - 1) / rows_a_tile;
    for (int i = used + lane; i < cap; i += 64) {
      tiles[4 * i] = -1;
      tiles[4 * i + 1] = tiles[4 * i + 2] = tiles[4 * i + 3] = 0;
    }
  }
  int at = base;
  for (int p0 = 0; p0 < P; p0 += 256) {
    int got[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) got[u] = p0 + 64 * u + lane < P ? expert[p0 + 64 * u + lane] : -1;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool mine = got[u] == e;
      const unsigned long long votes = __ballot(mine);
      if (mine) order[at + __popcll(votes & ((1ull << lane) - 1ull))] = p0 + 64 * u + lane;
      at += __popcll(votes);
    }
  }
}

__global__ __launch_bounds__(64) void route_count_kernel(const int* __restrict__ expert, int P, int* __restrict__ counts) {
  const int n = count_pairs(expert, P, blockIdx.x, threadIdx.x);
  if (threadIdx.x == 0) counts[blockIdx.x] = n;
}

__global__ __launch_bounds__(64) void route_place_kernel(const int* __restrict__ expert, const int* __restrict__ counts,
                                                         int P, int E, int rows_a_tile, int* __restrict__ order,
                                                         int* __restrict__ tiles, int cap) {
  place_pairs(expert, counts, P, E, blockIdx.x, threadIdx.x, rows_a_tile, order, tiles, cap);
}

constexpr int kSmallPairs = 512, kSmallExperts = 512;   // what the one-workgroup kernel keeps in LDS

__global__ __launch_bounds__(1024) void route_small_kernel(const float* __restrict__ z, long ldz,
                                                           const float* __restrict__ bias, int n_tokens, int E, int top,
                                                           int rows_a_tile, int* __restrict__ expert,
                                                           float* __restrict__ weight, int* __restrict__ order,
                                                           int* __restrict__ tiles, int cap,
                                                           const int* __restrict__ token_ids, const int* __restrict__ table,
                                                           int scoring) {
  __shared__ int picks_s[kSmallPairs];
  __shared__ float share_s[16][kMaxTop];
  __shared__ int counts_s[kSmallExperts];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int P = n_tokens * top;
  if (table) {   // the picks are looked up, not chosen
    for (int pair = threadIdx.x; pair < P; pair += 1024) {
      const int e = table[(long)token_ids[pair / top] * top + pair % top];
      picks_s[pair] = e;
      expert[pair] = e;
      weight[pair] = 1.0f / (float)top;
    }
  }
  for (int t = w; t < n_tokens && !table; t += 16) {
    pick_top(z + (long)t * ldz, bias, E, top, lane, picks_s + t * top, share_s[w], scoring);
    if (lane < top) {
      expert[(long)t * top + lane] = picks_s[t * top + lane];
      weight[(long)t * top + lane] = share_s[w][lane];
    }
  }
  __syncthreads();
  for (int e = w; e < E; e += 16) {
    const int n = count_pairs(picks_s, P, e, lane);
    if (lane == 0) counts_s[e] = n;
  }
  __syncthreads();
  for (int e = w; e < E; e += 16) place_pairs(picks_s, counts_s, P, E, e, lane, rows_a_tile, order, tiles, cap);
}

// ---------------------------------------------------------------------------
// (3) act [P][ldy] (T) = act(x[token] W_gate[e]^T, x[token] W_up[e]^T) for the pairs of every tile, in the
// order of `order`.  w_gate, w_up [E][F][K].  A workgroup: one tile, four waves with 16 columns of F each.
// ---------------------------------------------------------------------------
template <typename T, int RT, int KS>
__global__ __launch_bounds__(256) void experts_gate_up_kernel(const T* __restrict__ x, long ldx,
                                                              const T* __restrict__ w_gate, const T* __restrict__ w_up,
                                                              int F, int K, int top, const int* __restrict__ order,
                                                              const int* __restrict__ tiles, float limit, float alpha, float shift,
                                                              const float* __restrict__ in_weight, T* __restrict__ act, long ldy) {
  // in_weight (or null): a pair's routing weight multiplies the expert's input, w * x, so both products are scaled
  // by it before the gated unit (the down product then adds the expert's output as it is)
  constexpr int VEC = Atom<T>::VEC, KC = Atom<T>::KCHUNK;
  const int e = tiles[4 * blockIdx.x];
  if (e < 0) return;
  const int first = tiles[4 * blockIdx.x + 1], rows = tiles[4 * blockIdx.x + 2];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4;
  // KS 1: the four waves take 16 columns each.  KS 4 (few rows): they take a quarter of K each for the same 16
  // columns, so that all of a wave's operands are on their way at once, and their sums are added in wave order.
  const int col0 = KS == 1 ? (blockIdx.y * 4 + w) * 16 : blockIdx.y * 16;
  if (col0 >= F) return;
  const bool w_ok = col0 + l16 < F;
  const T* g_row = w_gate + ((long)e * F + (w_ok ? col0 + l16 : 0)) * K;
  const T* u_row = w_up + ((long)e * F + (w_ok ? col0 + l16 : 0)) * K;
  const T* x_row[RT];
  bool x_ok[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    x_ok[r] = 16 * r + l16 < rows;
    const int pair = x_ok[r] ? order[first + 16 * r + l16] : 0;
    x_row[r] = x + (long)(pair / top) * ldx;
  }
  f32x4 acc_g[RT], acc_u[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc_g[r] = acc_u[r] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool aligned = K % VEC == 0;
  // the operands of U chunks are requested together, then multiplied in ascending order
  constexpr int U = RT == 1 ? 8 : 4;
  const int k_each = KS == 1 ? K : (K + KC * KS - 1) / (KC * KS) * KC;
  const int k_lo = KS == 1 ? 0 : w * k_each, k_hi = KS == 1 ? K : min(K, k_lo + k_each);
  for (int k0 = k_lo; k0 < k_hi; k0 += U * KC) {
    typename Atom<T>::vec_t a_g[U], a_u[U], b[U][RT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * KC + VEC * quad;
      a_g[u] = load_vec<T>(g_row, 0, k, k_hi, 0, w_ok, aligned);
      a_u[u] = load_vec<T>(u_row, 0, k, k_hi, 0, w_ok, aligned);
#pragma unroll
      for (int r = 0; r < RT; ++r) b[u][r] = load_vec<T>(x_row[r], 0, k, k_hi, 0, x_ok[r], aligned);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        Atom<T>::mma(acc_g[r], a_g[u], b[u][r]);
        Atom<T>::mma(acc_u[r], a_u[u], b[u][r]);
      }
  }
  if constexpr (KS > 1) {
    __shared__ f32x4 sums_s[KS][2][RT][64];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      sums_s[w][0][r][lane] = acc_g[r];
      sums_s[w][1][r][lane] = acc_u[r];
    }
    __syncthreads();
    if (w != 0) return;
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int o = 1; o < KS; ++o)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc_g[r][i] = acc_g[r][i] + sums_s[o][0][r][lane][i];
          acc_u[r][i] = acc_u[r][i] + sums_s[o][1][r][lane][i];
        }
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (!x_ok[r]) continue;
    T* dst = act + (long)(first + 16 * r + l16) * ldy;
    const float wt = in_weight ? in_weight[order[first + 16 * r + l16]] : 1.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = col0 + 4 * quad + i;
      if (c < F) {
        const float g = fminf(acc_g[r][i] * wt, limit);
        const float u = fminf(fmaxf(acc_u[r][i] * wt, -limit), limit);
        dst[c] = from_f32<T>((g * sigmoid_e(alpha * g)) * (u + shift));
      }
    }
  }
}

// ---------------------------------------------------------------------------
// (4) P[choice][token][:] = weight[pair] * (act[place] W_down[e]^T).  w_down [E][N][F]; P [top][n_tokens][N] float.
// ---------------------------------------------------------------------------
template <typename T, int RT, int KS>
__global__ __launch_bounds__(256) void experts_down_kernel(const T* __restrict__ act, long ldy,
                                                           const T* __restrict__ w_down, int N, int F, int top,
                                                           int n_tokens, const int* __restrict__ order,
                                                           const int* __restrict__ tiles,
                                                           const float* __restrict__ weight, float* __restrict__ P) {
  constexpr int VEC = Atom<T>::VEC, KC = Atom<T>::KCHUNK;
  const int e = tiles[4 * blockIdx.x];
  if (e < 0) return;
  const int first = tiles[4 * blockIdx.x + 1], rows = tiles[4 * blockIdx.x + 2];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4;
  const int col0 = KS == 1 ? (blockIdx.y * 4 + w) * 16 : blockIdx.y * 16;
  if (col0 >= N) return;
  const bool w_ok = col0 + l16 < N;
  const T* d_row = w_down + ((long)e * N + (w_ok ? col0 + l16 : 0)) * F;
  const T* y_row[RT];
  bool y_ok[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    y_ok[r] = 16 * r + l16 < rows;
    y_row[r] = act + (long)(first + (y_ok[r] ? 16 * r + l16 : 0)) * ldy;
  }
  f32x4 acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool aligned = F % VEC == 0 && ldy % VEC == 0;
  constexpr int U = RT == 1 ? 8 : 4;
  const int k_each = KS == 1 ? F : (F + KC * KS - 1) / (KC * KS) * KC;
  const int k_lo = KS == 1 ? 0 : w * k_each, k_hi = KS == 1 ? F : min(F, k_lo + k_each);
  for (int k0 = k_lo; k0 < k_hi; k0 += U * KC) {
    typename Atom<T>::vec_t a[U], b[U][RT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * KC + VEC * quad;
      a[u] = load_vec<T>(d_row, 0, k, k_hi, 0, w_ok, aligned);
#pragma unroll
      for (int r = 0; r < RT; ++r) b[u][r] = load_vec<T>(y_row[r], 0, k, k_hi, 0, y_ok[r], aligned);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RT; ++r) Atom<T>::mma(acc[r], a[u], b[u][r]);
  }
  if constexpr (KS > 1) {
    __shared__ f32x4 sums_s[KS][RT][64];
#pragma unroll
    for (int r = 0; r < RT; ++r) sums_s[w][r][lane] = acc[r];
    __syncthreads();
    if (w != 0) return;
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int o = 1; o < KS; ++o)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[r][i] = acc[r][i] + sums_s[o][r][lane][i];
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (!y_ok[r]) continue;
    const int pair = order[first + 16 * r + l16];
    const float share = weight ? weight[pair] : 1.0f;
    float* dst = P + ((long)(pair % top) * n_tokens + pair / top) * N;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = col0 + 4 * quad + i;
      if (c < N) dst[c] = share * acc[r][i];
    }
  }
}

// ---------------------------------------------------------------------------
// The same two products for tiles of 64 rows (many tokens an expert), both operands staged through LDS: a
// workgroup takes 64 rows x 64 columns, its four waves 32 x 32 each.  A stage is 128 bytes of K for every row of
// the operands (two chunks of the atom), copied from global memory into registers while the stage before it is
// multiplied, then written to the other of two LDS buffers; rows of an LDS tile are 144 bytes apart, which
// spreads the sixteen rows of a fragment read over all banks.  A row's contraction is still one chain over
// ascending chunks from zero: the same bits as the kernels above give without a cut of K.  NB: weight matrices
// that share the rows (gate and up: 2; down: 1).
// ---------------------------------------------------------------------------
constexpr int kStageBytes = 128, kLdsRow = kStageBytes + 16;

template <typename T, int NB>
struct TiledProduct {
  typedef typename Atom<T>::vec_t vec_t;
  static constexpr int VEC = Atom<T>::VEC;
  static constexpr int kStageK = kStageBytes / (int)sizeof(T);
  vec_t staged[1 + NB][2];
  f32x4 acc[NB][2][2];

  // a_row / b_row: where this thread's two pieces of a stage come from (null: zeros), for rows tid/8 and tid/8 + 32
  __device__ __forceinline__ void request(const T* const (&a_row)[2], const T* const (&b_row)[NB][2], int k0, int K) {
    const int seg = threadIdx.x & 7;
    const int k = k0 + seg * VEC;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      staged[0][j] = (a_row[j] && k < K) ? *reinterpret_cast<const vec_t*>(a_row[j] + k) : Atom<T>::zero();
#pragma unroll
      for (int m = 0; m < NB; ++m)
        staged[1 + m][j] = (b_row[m][j] && k < K) ? *reinterpret_cast<const vec_t*>(b_row[m][j] + k) : Atom<T>::zero();
    }
  }
  __device__ __forceinline__ void store(char* lds) {
    const int row = threadIdx.x >> 3, seg = threadIdx.x & 7;
#pragma unroll
    for (int m = 0; m < 1 + NB; ++m)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        *reinterpret_cast<vec_t*>(lds + ((m * 64) + row + 32 * j) * kLdsRow + seg * 16) = staged[m][j];
  }
  __device__ __forceinline__ void multiply(const char* lds) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int l16 = lane & 15, quad = lane >> 4, wr = w >> 1, wc = w & 1;
#pragma unroll
    for (int c = 0; c < kStageBytes / 64; ++c) {
      vec_t a[2], b[NB][2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        a[t] = *reinterpret_cast<const vec_t*>(lds + (wr * 32 + t * 16 + l16) * kLdsRow + c * 64 + quad * 16);
#pragma unroll
        for (int m = 0; m < NB; ++m)
          b[m][t] = *reinterpret_cast<const vec_t*>(lds + ((1 + m) * 64 + wc * 32 + t * 16 + l16) * kLdsRow + c * 64 + quad * 16);
      }
#pragma unroll
      for (int m = 0; m < NB; ++m)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
          for (int ct = 0; ct < 2; ++ct) Atom<T>::mma(acc[m][rt][ct], b[m][ct], a[rt]);
    }
  }
  __device__ __forceinline__ void run(const T* const (&a_row)[2], const T* const (&b_row)[NB][2], int K, char* lds) {
#pragma unroll
    for (int m = 0; m < NB; ++m)
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) acc[m][rt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int kBuffer = (1 + NB) * 64 * kLdsRow;
    const int stages = (K + kStageK - 1) / kStageK;
    request(a_row, b_row, 0, K);
    store(lds);
    __syncthreads();
    for (int s = 0; s < stages; ++s) {
      if (s + 1 < stages) request(a_row, b_row, (s + 1) * kStageK, K);
      multiply(lds + (s & 1) * kBuffer);
      if (s + 1 < stages) store(lds + ((s + 1) & 1) * kBuffer);
      __syncthreads();
    }
  }
};

template <typename T>
__global__ __launch_bounds__(256) void experts_gate_up_tiled_kernel(const T* __restrict__ x, long ldx,
                                                                    const T* __restrict__ w_gate,
                                                                    const T* __restrict__ w_up, int F, int K, int top,
                                                                    const int* __restrict__ order,
                                                                    const int* __restrict__ tiles, float limit, float alpha,
                                                                    float shift, const float* __restrict__ in_weight,
                                                                    T* __restrict__ act, long ldy) {
  __shared__ __attribute__((aligned(16))) char lds[2 * 3 * 64 * kLdsRow];
  const int e = tiles[4 * blockIdx.x];
  if (e < 0) return;
  const int first = tiles[4 * blockIdx.x + 1], rows = tiles[4 * blockIdx.x + 2];
  const int col0 = blockIdx.y * 64;
  const T* a_row[2];
  const T* b_row[2][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int r = (threadIdx.x >> 3) + 32 * j;
    a_row[j] = r < rows ? x + (long)(order[first + r] / top) * ldx : nullptr;
    b_row[0][j] = col0 + r < F ? w_gate + ((long)e * F + col0 + r) * K : nullptr;
    b_row[1][j] = col0 + r < F ? w_up + ((long)e * F + col0 + r) * K : nullptr;
  }
  TiledProduct<T, 2> product;
  product.run(a_row, b_row, K, lds);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4, wr = w >> 1, wc = w & 1;
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int r = wr * 32 + rt * 16 + l16;
    if (r >= rows) continue;
    T* dst = act + (long)(first + r) * ldy;
    const float wt = in_weight ? in_weight[order[first + r]] : 1.0f;
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = col0 + wc * 32 + ct * 16 + 4 * quad + i;
        if (c < F) {
          const float g = fminf(product.acc[0][rt][ct][i] * wt, limit);
          const float u = fminf(fmaxf(product.acc[1][rt][ct][i] * wt, -limit), limit);
          dst[c] = from_f32<T>((g * sigmoid_e(alpha * g)) * (u + shift));
        }
      }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void experts_down_tiled_kernel(const T* __restrict__ act, long ldy,
                                                                 const T* __restrict__ w_down, int N, int F, int top,
                                                                 int n_tokens, const int* __restrict__ order,
                                                                 const int* __restrict__ tiles,
                                                                 const float* __restrict__ weight, float* __restrict__ P) {
  __shared__ __attribute__((aligned(16))) char lds[2 * 2 * 64 * kLdsRow];
  const int e = tiles[4 * blockIdx.x];
  if (e < 0) return;
  const int first = tiles[4 * blockIdx.x + 1], rows = tiles[4 * blockIdx.x + 2];
  const int col0 = blockIdx.y * 64;
  const T* a_row[2];
  const T* b_row[1][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int r = (threadIdx.x >> 3) + 32 * j;
    a_row[j] = r < rows ? act + (long)(first + r) * ldy : nullptr;
    b_row[0][j] = col0 + r < N ? w_down + ((long)e * N + col0 + r) * F : nullptr;
  }
  TiledProduct<T, 1> product;
  product.run(a_row, b_row, F, lds);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4, wr = w >> 1, wc = w & 1;
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const int r = wr * 32 + rt * 16 + l16;
    if (r >= rows) continue;
    const int pair = order[first + r];
    const float share = weight ? weight[pair] : 1.0f;
    float* dst = P + ((long)(pair % top) * n_tokens + pair / top) * N;
#pragma unroll
    for (int ct = 0; ct < 2; ++ct)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = col0 + wc * 32 + ct * 16 + 4 * quad + i;
        if (c < N) dst[c] = share * product.acc[0][rt][ct][i];
      }
  }
}

}  // namespace ls

LS_DEFINE_ERROR_API

using namespace ls;

extern "C" int ls_experts_max_top() { return kMaxTop; }

// Tiles that the pairs of n_tokens tokens can need at most, with rows_a_tile rows each.
extern "C" int ls_experts_tile_capacity(int n_tokens, int E, int top, int rows_a_tile) {
  const long pairs = (long)n_tokens * top;
  return (int)(pairs / rows_a_tile + (pairs < E ? pairs : E));
}

// z [n_tokens][ldz] float router logits, bias [E] or null -> expert, weight [n_tokens][top]; order [n_tokens * top];
// tiles [cap][4]; counts: scratch of E ints.  rows_a_tile 16, 32 or 64.
extern "C" int ls_experts_route(const float* z, long ldz, const float* bias, int n_tokens, int E, int top,
                                int rows_a_tile, int* expert, float* weight, int* order, int* tiles, int cap,
                                int* counts, int scoring, void* stream) {
  LS_REQUIRE(scoring == 0 || scoring == 1, "experts_route: scoring %d (0: softmax over the chosen, 1: sigmoid)", scoring);
  LS_REQUIRE(n_tokens > 0 && E > 0 && top > 0 && top <= E && top <= kMaxTop && ldz >= E,
             "experts_route: %d tokens, %d experts, %d chosen (at most %d)", n_tokens, E, top, kMaxTop);
  LS_REQUIRE(rows_a_tile == 16 || rows_a_tile == 32 || rows_a_tile == 64, "experts_route: tiles of %d rows", rows_a_tile);
  LS_REQUIRE(z && expert && weight && order && tiles && counts, "experts_route: null operand");
  LS_REQUIRE(cap >= ls_experts_tile_capacity(n_tokens, E, top, rows_a_tile), "experts_route: %d tiles are too few", cap);
  LS_REQUIRE(E <= 64 * kMaxPerLane, "experts_route: %d experts, the routing kernel takes %d", E, 64 * kMaxPerLane);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int P = n_tokens * top;
  if (P <= kSmallPairs && E <= kSmallExperts) {
    hipLaunchKernelGGL(route_small_kernel, dim3(1), dim3(1024), 0, s, z, ldz, bias, n_tokens, E, top, rows_a_tile,
                       expert, weight, order, tiles, cap, (const int*)nullptr, (const int*)nullptr, scoring);
  } else {
    hipLaunchKernelGGL(route_topk_kernel, dim3((n_tokens + 3) / 4), dim3(256), 0, s, z, ldz, bias, n_tokens, E, top,
                       expert, weight, scoring);
    hipLaunchKernelGGL(route_count_kernel, dim3(E), dim3(64), 0, s, expert, P, counts);
    hipLaunchKernelGGL(route_place_kernel, dim3(E), dim3(64), 0, s, expert, counts, P, E, rows_a_tile, order, tiles, cap);
  }
  return check_launch("experts_route");
}

// The same grouping for experts that a table names: token_ids [n_tokens], table [vocab][top] with entries in [0, E).
extern "C" int ls_experts_route_table(const int* token_ids, const int* table, int n_tokens, int E, int top,
                                      int rows_a_tile, int* expert, float* weight, int* order, int* tiles, int cap,
                                      int* counts, void* stream) {
  LS_REQUIRE(n_tokens > 0 && E > 0 && top > 0 && top <= E, "experts_route_table: %d tokens, %d experts, %d a token", n_tokens, E, top);
  LS_REQUIRE(rows_a_tile == 16 || rows_a_tile == 32 || rows_a_tile == 64, "experts_route_table: tiles of %d rows", rows_a_tile);
  LS_REQUIRE(token_ids && table && expert && weight && order && tiles && counts, "experts_route_table: null operand");
  LS_REQUIRE(cap >= ls_experts_tile_capacity(n_tokens, E, top, rows_a_tile), "experts_route_table: %d tiles are too few", cap);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int P = n_tokens * top;
  if (P <= kSmallPairs && E <= kSmallExperts) {
    hipLaunchKernelGGL(route_small_kernel, dim3(1), dim3(1024), 0, s, (const float*)nullptr, 0L, (const float*)nullptr,
                       n_tokens, E, top, rows_a_tile, expert, weight, order, tiles, cap, token_ids, table, 0);
  } else {
    hipLaunchKernelGGL(route_table_kernel, dim3((P + 255) / 256), dim3(256), 0, s, token_ids, table, n_tokens, top, expert,
                       weight);
    hipLaunchKernelGGL(route_count_kernel, dim3(E), dim3(64), 0, s, expert, P, counts);
    hipLaunchKernelGGL(route_place_kernel, dim3(E), dim3(64), 0, s, expert, counts, P, E, rows_a_tile, order, tiles, cap);
  }
  return check_launch("experts_route_table");
}

// x [n_tokens][ldx]; w_gate, w_up [E][F][K]; w_down [E][N][F]; act: scratch [n_tokens * top][ldy] of the compute
// dtype; P [top][n_tokens][N] float.
extern "C" int ls_experts_apply(int dtype, const void* x, long ldx, const void* w_gate, const void* w_up,
                                const void* w_down, int n_tokens, int E, int top, int K, int F, int N,
                                int rows_a_tile, const int* order, const int* tiles, int cap, const float* weight,
                                float limit, float alpha, float shift, void* act, long ldy, float* P, int weigh_input,
                                void* stream) {
  // weigh_input: the routing weight multiplies the expert's input instead of its output
  const float* in_weight = weigh_input ? weight : nullptr;
  const float* out_weight = weigh_input ? nullptr : weight;
  LS_REQUIRE(n_tokens > 0 && E > 0 && top > 0 && K > 0 && F > 0 && N > 0 && ldx >= K && ldy >= F, "experts_apply: bad sizes");
  LS_REQUIRE(rows_a_tile == 16 || rows_a_tile == 32 || rows_a_tile == 64, "experts_apply: tiles of %d rows", rows_a_tile);
  LS_REQUIRE(x && w_gate && w_up && w_down && order && tiles && weight && act && P && cap > 0, "experts_apply: null operand");
  LS_REQUIRE(limit > 0.f, "experts_apply: the limit must be positive");
  LS_REQUIRE(dtype == kF32 || dtype == kBF16, "experts_apply: unknown dtype %d", dtype);
  const int vec = dtype == kF32 ? 4 : 8;
  LS_REQUIRE(reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(act) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(w_gate) % 16 == 0 && reinterpret_cast<uintptr_t>(w_up) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(w_down) % 16 == 0 && (K % vec != 0 || ldx % vec == 0),
             "experts_apply: operands must be 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // tiles of 16 rows (few tokens an expert): a workgroup takes 16 columns and cuts K over its waves
  const int cols = rows_a_tile == 16 ? 16 : 64;
  const dim3 grid_up(cap, (F + cols - 1) / cols), grid_down(cap, (N + cols - 1) / cols);
#define LS_EXPERTS(T_, RT_, KS_)                                                                                      \
  do {                                                                                                                \
    hipLaunchKernelGGL((experts_gate_up_kernel<T_, RT_, KS_>), grid_up, dim3(256), 0, s, (const T_*)x, ldx,           \
                       (const T_*)w_gate, (const T_*)w_up, F, K, top, order, tiles, limit, alpha, shift, in_weight,   \
                       (T_*)act, ldy);                                                                                \
    hipLaunchKernelGGL((experts_down_kernel<T_, RT_, KS_>), grid_down, dim3(256), 0, s, (const T_*)act, ldy,          \
                       (const T_*)w_down, N, F, top, n_tokens, order, tiles, out_weight, P);                          \
  } while (0)
  // tiles of 64 rows go through LDS where every row of every operand starts on a 16-byte boundary
  const bool staged = rows_a_tile == 64 && K % vec == 0 && F % vec == 0 && ldx % vec == 0 && ldy % vec == 0;
#define LS_EXPERTS_STAGED(T_)                                                                                         \
  do {                                                                                                                \
    hipLaunchKernelGGL(experts_gate_up_tiled_kernel<T_>, grid_up, dim3(256), 0, s, (const T_*)x, ldx,                 \
                       (const T_*)w_gate, (const T_*)w_up, F, K, top, order, tiles, limit, alpha, shift, in_weight,   \
                       (T_*)act, ldy);                                                                                \
    hipLaunchKernelGGL(experts_down_tiled_kernel<T_>, grid_down, dim3(256), 0, s, (const T_*)act, ldy,                \
                       (const T_*)w_down, N, F, top, n_tokens, order, tiles, out_weight, P);                          \
  } while (0)
#define LS_EXPERTS_BY_ROWS(T_)                 \
  switch (rows_a_tile) {                       \
    case 16: LS_EXPERTS(T_, 1, 4); break;      \
    case 32: LS_EXPERTS(T_, 2, 1); break;      \
    default:                                   \
      if (staged)                              \
        LS_EXPERTS_STAGED(T_);                 \
      else                                     \
        LS_EXPERTS(T_, 4, 1);                  \
      break;                                   \
  }
  if (dtype == kF32) {
    LS_EXPERTS_BY_ROWS(float)
  } else {
    LS_EXPERTS_BY_ROWS(bf16_t)
  }
#undef LS_EXPERTS_BY_ROWS
#undef LS_EXPERTS_STAGED
#undef LS_EXPERTS
  return check_launch("experts_apply");
}
