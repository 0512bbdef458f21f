// More kernels of the mixers library: a residual stream of several copies that every sublayer reads
// as one weighted sum and writes back through a small mixing matrix (with the norm of the next reader
// fused in), the passes around attention over a cached latent (norms of the latents, rotation of the
// shared key part, queries brought into the latent's space by a product a head), and the gated delta
// rule with its short convolutions.
//
// Everything here is computed in float whatever the compute dtype T is: T is the type of what a
// matrix product reads next (and of the cache).  Per-row reductions have an order fixed by the row's
// sizes alone; the recurrence walks a request's tokens in order, so nothing depends on how the
// request was cut into steps or on what else is in the batch.

#include "common.h"
#include "mixers_api.h"

namespace ls {

struct SeqMeta {  // one per sequence of the step (all int32), as the step's upload lays it out
  int q_off;      // first packed row
  int q_len;      // rows in this step
  int q_start;    // absolute position of the first row
  int kv_len;     // q_start + q_len
  int table_row;  // row of the block table, and the request's state slot
  int reserved[3];
};

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// The four wave sums of a workgroup of 256 threads added in wave order; every thread gets the total.
__device__ __forceinline__ float block_sum4(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  return ((scratch[0] + scratch[1]) + scratch[2]) + scratch[3];
}

// ---------------------------------------------------------------------------
// A residual stream of n copies X [rows][n][W] (float).  One launch does, for a row, either or both of
//   write:  y = P[0][row] + P[1][row] + ... (slices ascending, from +0: the sublayer's output, left as slice sums);
//           X'_t = sum_s mix[s][t] X_s + gain[t] y      for all t at once from the old copies
//   read:   u = sum_t take[t] X'_t   (take == null: the plain sum of the copies)
//           out = u / sqrt(mean(u^2) + eps) * weight     (T)
// Thread t of 256 owns the elements 1024 c + 4 t + {0..3}, c ascending; the sum of squares adds them in that order, then
// a butterfly over the wave and the wave sums in wave order.  `row` = rows[r] when a row list is given.
// ---------------------------------------------------------------------------
constexpr int kMaxStreams = 8;
constexpr int kStreamChunks = 12;  // a row of up to 1024 * kStreamChunks elements keeps what it read in LDS

__device__ __forceinline__ f32x4 load4(const float* __restrict__ p, int e, int W, bool vec_ok) {
  if (vec_ok) return *reinterpret_cast<const f32x4*>(p + e);
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (e + i < W) v[i] = p[e + i];
  return v;
}

// (N, the number of copies, is a template parameter: every copy's load stands in straight-line code, so all of a
// thread's loads are on their way before the first is used)
template <typename T, int N>
__global__ __launch_bounds__(256) void streams_step_kernel(float* __restrict__ X, long ldx, int W,
                                                           const float* __restrict__ P, int slices, long p_stride,
                                                           const float* __restrict__ mix, const float* __restrict__ gain,
                                                           const float* __restrict__ take, const float* __restrict__ weight,
                                                           float eps, T* __restrict__ out, long ld_out,
                                                           const int* __restrict__ rows) {
  __shared__ float mix_s[N * N], gain_s[N], take_s[N], scratch[4];
  const int r_out = blockIdx.x;
  const long row = rows ? rows[r_out] : r_out;
  if (threadIdx.x < N * N) mix_s[threadIdx.x] = P ? mix[threadIdx.x] : 0.f;
  if (threadIdx.x < N) {
    gain_s[threadIdx.x] = P ? gain[threadIdx.x] : 0.f;
    take_s[threadIdx.x] = take ? take[threadIdx.x] : 1.0f;
  }
  __syncthreads();
  float* x = X + row * ldx;
  // rows of whole vectors of four: a copy's elements and a slice's move as 16 bytes
  const bool vec_ok = W % 4 == 0 && ldx % 4 == 0;
  extern __shared__ float u_s[];   // what the row's read gave, until the row's sum of squares is known (a thread's own elements)
  float part = 0.f;
  constexpr int BATCH = 8;         // slice sums requested together
#pragma unroll 1
  for (int e = 4 * (int)threadIdx.x; e < W; e += 1024) {
    f32x4 copy[N];
#pragma unroll
    for (int s = 0; s < N; ++s) copy[s] = load4(x + (long)s * W, e, W, vec_ok);
    if (P) {
      const float* p = P + row * W;
      f32x4 y = {0.f, 0.f, 0.f, 0.f};
      for (int s0 = 0; s0 < slices; s0 += BATCH) {
        f32x4 got[BATCH];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) got[u] = load4(p + (long)min(s0 + u, slices - 1) * p_stride, e, W, vec_ok);   // (clamped: no branch between the loads)
#pragma unroll
        for (int u = 0; u < BATCH; ++u)
          if (s0 + u < slices) y = y + got[u];
      }
      f32x4 fresh[N];
#pragma unroll
      for (int t = 0; t < N; ++t) {
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s2 = 0; s2 < N; ++s2) v = v + mix_s[s2 * N + t] * copy[s2];
        fresh[t] = v + gain_s[t] * y;
      }
#pragma unroll
      for (int t = 0; t < N; ++t) {
        copy[t] = fresh[t];
        if (vec_ok) {
          *reinterpret_cast<f32x4*>(x + (long)t * W + e) = fresh[t];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (e + i < W) x[(long)t * W + e + i] = fresh[t][i];
        }
      }
    }
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < N; ++t) sum = sum + take_s[t] * copy[t];
    if (out) *reinterpret_cast<f32x4*>(u_s + e) = sum;
#pragma unroll
    for (int i = 0; i < 4; ++i) part = part + sum[i] * sum[i];   // (elements beyond W are zeros)
  }
  if (!out) return;
  const float scale = 1.0f / sqrtf(block_sum4(part, scratch) / (float)W + eps);
#pragma unroll 1
  for (int e0 = 4 * (int)threadIdx.x; e0 < W; e0 += 1024) {
    const f32x4 u = *reinterpret_cast<const f32x4*>(u_s + e0);
    if (vec_ok) {
      const f32x4 w = *reinterpret_cast<const f32x4*>(weight + e0);
      T* dst = out + (long)r_out * ld_out + e0;
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[i] = from_f32<T>((u[i] * scale) * w[i]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (e0 + i < W) out[(long)r_out * ld_out + e0 + i] = from_f32<T>((u[i] * scale) * weight[e0 + i]);
    }
  }
}

// ---------------------------------------------------------------------------
// Post pass of the down projections of attention over a latent: raw [T][ld] float = a (QR) | c (CR) | r (RD), the
// last two absent for a layer that reads another layer's latent (has_kv == 0).
//   a -> a / sqrt(mean(a^2) + eps) * a_weight            -> a_out [T][QR] (T)
//   c -> c / sqrt(mean(c^2) + eps) * c_weight            -> key pages [page][0][slot][0 .. CR) and value pages
//                                                           [page][0][0 .. CR)[slot]: the latent is key and value
//   r -> rotated in neighbouring pairs (2i, 2i + 1) on its first `rot` dimensions at the token's position
//                                                        -> key pages [page][0][slot][CR .. CR + RD), zeros up to Dp
// One workgroup a token; the sums of squares as in streams_step_kernel.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_post_kernel(
    const float* __restrict__ raw, long ld, int QR, int CR, int RD, int Dp, int has_kv, const float* __restrict__ a_weight,
    const float* __restrict__ c_weight, float eps, const float* __restrict__ cos_table, const float* __restrict__ sin_table,
    int rot, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, const SeqMeta* __restrict__ seqs,
    const int* __restrict__ table, int table_stride, T* __restrict__ a_out, long lda, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int page_size) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const float* row = raw + (long)t * ld;
  {
    const float part = row_sumsq_part(row, QR, threadIdx.x, false);
    const float scale = 1.0f / sqrtf(block_sum4(part, scratch) / (float)QR + eps);
    for (int e = threadIdx.x; e < QR; e += 256) a_out[(long)t * lda + e] = from_f32<T>((row[e] * scale) * a_weight[e]);
  }
  if (!has_kv) return;
  const int pos = tok_pos[t];
  const int page = table[(long)seqs[tok_seq[t]].table_row * table_stride + pos / page_size];
  const int slot = pos % page_size;
  const float part = row_sumsq_part(row + QR, CR, threadIdx.x, false);
  const float scale = 1.0f / sqrtf(block_sum4(part, scratch) / (float)CR + eps);
  if (page < 0) return;
  T* key = k_pages + ((long)page * page_size + slot) * Dp;
  T* value = v_pages + (long)page * CR * page_size + slot;
  for (int e = threadIdx.x; e < CR; e += 256) {
    const T c = from_f32<T>((row[QR + e] * scale) * c_weight[e]);
    key[e] = c;
    value[(long)e * page_size] = c;
  }
  const float* r = row + QR + CR;
  const int half = rot >> 1;
  for (int i = threadIdx.x; i < Dp - CR; i += 256) {
    float v = 0.f;
    if (i < RD) {
      v = r[i];
      if (i < rot) {
        const float other = r[i ^ 1], c = cos_table[(long)pos * half + (i >> 1)], s = sin_table[(long)pos * half + (i >> 1)];
        v = (i & 1) ? v * c + other * s : v * c - other * s;
      }
    }
    key[CR + i] = from_f32<T>(v);
  }
}

// ---------------------------------------------------------------------------
// Post pass of the up projection of the queries: qf [T][ld] float holds, head by head, D plain dimensions and RD
// rotated ones.  The plain ones go to plain_out [T][H*D] (T), the operand of the product that brings them into the
// latent's space; the rotated ones are rotated (neighbouring pairs, first `rot` dimensions) and written where the
// attention kernel reads them, behind the CR latent dimensions of a query head of Dp elements (zeros up to Dp).
// One thread an element.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_query_kernel(const float* __restrict__ qf, long ld, int n_tokens, int H, int D,
                                                           int RD, int CR, int Dp, const float* __restrict__ cos_table,
                                                           const float* __restrict__ sin_table, int rot,
                                                           const int* __restrict__ tok_pos, T* __restrict__ plain_out,
                                                           long ldp, T* __restrict__ q_out, long ldq) {
  const int tail = Dp - CR, each = D + tail;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)n_tokens * H * each) return;
  const int i = (int)(idx % each), head = (int)((idx / each) % H), t = (int)(idx / ((long)each * H));
  const float* src = qf + (long)t * ld + (long)head * (D + RD);
  if (i < D) {
    plain_out[(long)t * ldp + head * D + i] = from_f32<T>(src[i]);
    return;
  }
  const int j = i - D;
  float v = 0.f;
  if (j < RD) {
    v = src[D + j];
    if (j < rot) {
      const int half = rot >> 1;
      const long pos = tok_pos[t];
      const float other = src[D + (j ^ 1)], c = cos_table[pos * half + (j >> 1)], s = sin_table[pos * half + (j >> 1)];
      v = (j & 1) ? v * c + other * s : v * c - other * s;
    }
  }
  q_out[(long)t * ldq + (long)head * Dp + CR + j] = from_f32<T>(v);
}

// ---------------------------------------------------------------------------
// A product a head: out[t][head * o_stride + n] = sum_k w[head][n][k] x[t][head * x_stride + k], w [H][N][K].
// A workgroup: 16 * RT rows of one head, four waves with 16 columns each.  The 16x16 MFMA atom with the weight rows
// as first operand; a row's contraction is one chain over ascending K from zero.
// ---------------------------------------------------------------------------
template <typename T, int RT>
__global__ __launch_bounds__(256) void heads_product_kernel(const T* __restrict__ x, long ldx, int x_stride,
                                                            const T* __restrict__ w, int N, int K, int n_rows,
                                                            T* __restrict__ out, long ldo, int o_stride, int x_aligned) {
  constexpr int VEC = Atom<T>::VEC, KC = Atom<T>::KCHUNK;
  const int head = blockIdx.y;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4;
  const int col0 = (blockIdx.z * 4 + wv) * 16;
  if (col0 >= N) return;
  const bool w_ok = col0 + l16 < N;
  const T* w_row = w + ((long)head * N + (w_ok ? col0 + l16 : 0)) * K;
  const int row0 = blockIdx.x * 16 * RT;
  const T* x_row[RT];
  bool x_ok[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    x_ok[r] = row0 + 16 * r + l16 < n_rows;
    x_row[r] = x + (long)(x_ok[r] ? row0 + 16 * r + l16 : 0) * ldx + (long)head * x_stride;
  }
  f32x4 acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};
  const bool w_aligned = K % VEC == 0;
  constexpr int U = 4;
  for (int k0 = 0; k0 < K; k0 += U * KC) {
    typename Atom<T>::vec_t a[U], b[U][RT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = k0 + u * KC + VEC * quad;
      a[u] = load_vec<T>(w_row, 0, k, K, 0, w_ok, w_aligned);
#pragma unroll
      for (int r = 0; r < RT; ++r) b[u][r] = load_vec<T>(x_row[r], 0, k, K, 0, x_ok[r], x_aligned != 0);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int r = 0; r < RT; ++r) Atom<T>::mma(acc[r], a[u], b[u][r]);
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (!x_ok[r]) continue;
    T* dst = out + (long)(row0 + 16 * r + l16) * ldo + (long)head * o_stride;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = col0 + 4 * quad + i;
      if (c < N) dst[c] = from_f32<T>(acc[r][i]);
    }
  }
}

// ---------------------------------------------------------------------------
// The gated delta rule.  raw [T][ld] float holds the projections q (G heads of D) | k (G of D) | v (H of DV) |
// b (H) | a (H) | whatever follows.  Per request a state of floats: S [H][D][DV], then the last M - 1 inputs of the
// short convolutions [M - 1][C], C = 2 G D + H DV channels, oldest first, zeros before the start.
//
// (1) delta_prep: a wave a (token, unit).  Units: the G query heads, the G key heads, the H value heads, and one for
//     the gates.  A channel's convolution y = sum_m taps[c][m] in(p - (M - 1) + m) (m ascending) takes the inputs of
//     this step from raw and those before it from the state; then silu; queries and keys become unit vectors
//     x / sqrt(sum x^2 + unit_eps) (lane i adds the squares of the elements i, i + 64, ... ascending, then a
//     butterfly), the query also times D^(-1/2).  Gates of head h: beta = sigmoid(b_h),
//     decay = exp(-exp(A_log_h) softplus(a_h + dt_bias_h)).
//     qk [T][2 G][dp] (queries, then keys; zeros beyond D), vv [T][H * DV], gates [T][H][2].
// (2) delta_rule: a wave a (request, head, 64 / L columns of the state); L neighbouring lanes share a column, lane
//     part p of them keeps the rows p * R + {0 .. R-1}.  Per token, in order:
//       kS = decay * sum_r S[r] k[r];  u = beta (v - kS);  S[r] = decay S[r] + k[r] u;  o = sum_r S[r] q[r]
//     (the sums: a lane's rows in four interleaved chains of fused multiply-adds, then the lanes of a column by moves inside their row of sixteen; the
//     decay multiplies the sum of the old state with the key, which is the decayed state's sum up to rounding).
//     A token's operands are requested eight (four) tokens before it is worked on.
// (3) delta_conv_state: the last M - 1 inputs of every channel become the state of the next step.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void delta_prep_kernel(
    const float* __restrict__ raw, long ld, int n_tokens, int G, int H, int D, int DV, int dp, int M,
    const float* __restrict__ taps, const float* __restrict__ a_log, const float* __restrict__ dt_bias, float unit_eps,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, const SeqMeta* __restrict__ seqs,
    const float* __restrict__ state, long state_stride, long conv_at, float* __restrict__ qk, float* __restrict__ vv,
    float* __restrict__ gates, const float* __restrict__ chan, long ldc, float* __restrict__ decays) {
  // (with a decay a key channel, chan [T][ldc] holds its H * D logits and dt_bias has as many entries: a unit a head
  // then forms the head's beta and its row of decays, decays [T][H][dp], ones beyond D)
  const int units = 2 * G + H + (chan ? H : 1);
  const long id = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (id >= (long)n_tokens * units) return;
  const int t = (int)(id / units), unit = (int)(id % units), lane = threadIdx.x & 63;
  const float* row = raw + (long)t * ld;
  const int C = 2 * G * D + H * DV;
  if (chan && unit >= 2 * G + H) {
    const int h = unit - (2 * G + H);
    if (lane < 2) gates[((long)t * H + h) * 2 + lane] = lane == 0 ? sigmoid_f(row[C + h]) : 1.0f;
    const float rate = expf(a_log[h]);
    for (int r = lane; r < dp; r += 64)
      decays[((long)t * H + h) * dp + r] =
          r < D ? expf(-rate * softplus_f(chan[(long)t * ldc + h * D + r] + dt_bias[h * D + r])) : 1.0f;
    return;
  }
  if (unit == units - 1) {
    for (int h = lane; h < H; h += 64) {
      gates[((long)t * H + h) * 2] = sigmoid_f(row[C + h]);
      gates[((long)t * H + h) * 2 + 1] = expf(-expf(a_log[h]) * softplus_f(row[C + H + h] + dt_bias[h]));
    }
    return;
  }
  const SeqMeta m = seqs[tok_seq[t]];
  const int pos = tok_pos[t];
  const float* old = state + (long)m.table_row * state_stride + conv_at;
  const bool is_v = unit >= 2 * G;
  const int size = is_v ? DV : D;
  const int c0 = is_v ? 2 * G * D + (unit - 2 * G) * DV : unit * D;
  // channel c at this token: convolution over the last M inputs, then silu.  An input's address is chosen (this
  // step's rows, or the state), then loaded: no branch stands between the loads of the taps.
  auto channel = [&](int c) LS_INLINED {
    float y = 0.f;
    for (int a = 0; a < M; ++a) {
      const int p = pos - (M - 1) + a;
      const float* src = p >= m.q_start ? raw + (long)(m.q_off + p - m.q_start) * ld + c
                                        : old + (long)(p - m.q_start + M - 1) * C + c;
      y = y + taps[(long)c * M + a] * *src;
    }
    return silu_f(y);
  };
  if (is_v) {
    for (int i = lane; i < size; i += 64) vv[(long)t * H * DV + (c0 - 2 * G * D) + i] = channel(c0 + i);
    return;
  }
  // a head of up to 256 elements: a lane keeps its up to four in registers between the sum and the scaling
  float mine[4];
  float part = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + 64 * j;
    mine[j] = i < size ? channel(c0 + i) : 0.f;
    part = part + mine[j] * mine[j];
  }
  float scale = 1.0f / sqrtf(wave_sum(part) + unit_eps);
  if (unit < G) scale = scale * (1.0f / sqrtf((float)D));
  float* dst = qk + ((long)t * 2 * G + unit) * dp;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + 64 * j;
    if (i < dp) dst[i] = mine[j] * scale;
  }
}

// Sum over the L (4, 8 or 16) neighbouring lanes that share a column, by data-parallel moves inside a row of sixteen
// lanes (no LDS): pairs, pairs of pairs, then the mirror image of the half row and of the row.  After every step
// the lanes that were added hold the same value, so all L lanes end with the same bits.
template <int L>
__device__ __forceinline__ float lanes_sum(float v) {
  v = v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));  // lanes 1 0 3 2
  v = v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));  // lanes 2 3 0 1
  if constexpr (L >= 8) v = v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x141, 0xF, 0xF, true));  // 7 - i
  if constexpr (L >= 16) v = v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x140, 0xF, 0xF, true));  // 15 - i
  return v;
}

// R rows a lane, L lanes a column (R * L rows, the head size rounded up), 64 / L columns a wave.  CH: the decay is a
// number a row of the state (decays [T][H][dp]) instead of one a head: S[r] <- g[r] S[r] first, then the rule as stated.
template <int R, int L, bool CH>
__global__ __launch_bounds__(64) void delta_rule_kernel(const float* __restrict__ qk, const float* __restrict__ vv,
                                                        const float* __restrict__ gates, const float* __restrict__ decays,
                                                        int G, int H, int D, int DV,
                                                        const SeqMeta* __restrict__ seqs, float* __restrict__ state,
                                                        long state_stride, float* __restrict__ out, long ldo) {
  constexpr int dp = L * R, COLS = 64 / L;
  const int seq = blockIdx.x / H, head = blockIdx.x % H;
  const SeqMeta m = seqs[seq];
  if (m.q_len <= 0) return;
  const int lane = threadIdx.x, lc = lane / L, part = lane % L;
  const int col = blockIdx.y * COLS + lc;
  const bool col_ok = col < DV;
  const int row0 = part * R;
  const int kh = head / (H / G);
  float* mine = state + (long)m.table_row * state_stride + (long)head * D * DV;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) S[r] = (row0 + r < D && col_ok) ? mine[(long)(row0 + r) * DV + col] : 0.f;
  struct Operands {
    f32x4 q[R / 4], k[R / 4], g[CH ? R / 4 : 1];
    float v, gate;   // gate: beta in the even lanes, the decay in the odd ones
  };
  // Pointers to the operands of the token that is requested next; they move on by a token after every request and
  // stay on the request's last token (no index arithmetic and no branch between the requests).  beta and the decay
  // are fetched by the lanes (even: beta, odd: decay) and handed round inside the quad: a load whose address is
  // the same in every lane would go through the scalar cache, whose loads return in any order, so that a wait for
  // one of them waits for all, also for those of the tokens ahead.
  const float* q_at = qk + ((long)m.q_off * 2 * G + kh) * dp + row0;
  const float* k_at = q_at + (long)G * dp;
  const float* v_at = vv + (long)m.q_off * H * DV + head * DV + (col_ok ? col : 0);
  const float* g_at = gates + ((long)m.q_off * H + head) * 2 + (lane & 1);
  const float* d_at = CH ? decays + ((long)m.q_off * H + head) * dp + row0 : nullptr;
  int left = m.q_len - 1;   // tokens behind the one the pointers stand on
  auto fetch = [&]() LS_INLINED {
    Operands x;
#pragma unroll
    for (int j = 0; j < R / 4; ++j) {
      x.q[j] = *reinterpret_cast<const f32x4*>(q_at + 4 * j);
      x.k[j] = *reinterpret_cast<const f32x4*>(k_at + 4 * j);
      if constexpr (CH) x.g[j] = *reinterpret_cast<const f32x4*>(d_at + 4 * j);
    }
    x.v = *v_at;
    x.gate = *g_at;
    const long step = left > 0 ? 1 : 0;
    left -= (int)step;
    q_at += step * 2 * G * dp;
    k_at += step * 2 * G * dp;
    v_at += step * H * DV;
    g_at += step * H * 2;
    if constexpr (CH) d_at += step * H * dp;
    return x;
  };
  // the operands of the token DEPTH tokens on are requested before a token is worked on (a ring of registers)
  constexpr int DEPTH = (R <= 8 && !CH) ? 8 : 4;
  Operands ring[DEPTH];
#pragma unroll
  for (int j = 0; j < DEPTH; ++j) ring[j] = fetch();
  for (int i0 = 0; i0 < m.q_len; i0 += DEPTH) {
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      const int i = i0 + j;
      if (i >= m.q_len) break;
      const Operands now = ring[j];
      ring[j] = fetch();
      const float beta = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(now.gate), 0x00, 0xF, 0xF, true));   // lane 0 of the quad
      const float decay = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(now.gate), 0x55, 0xF, 0xF, true));  // lane 1
      // a lane's rows in four interleaved chains (rows r, r + 4, ... of each), added as (0 + 1) + (2 + 3)
      float ks4[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (CH) {
#pragma unroll
        for (int r = 0; r < R; ++r) S[r] = S[r] * now.g[r >> 2][r & 3];
      }
#pragma unroll
      for (int r = 0; r < R; ++r) ks4[r & 3] = fmaf(S[r], now.k[r >> 2][r & 3], ks4[r & 3]);
      const float ks = lanes_sum<L>((ks4[0] + ks4[1]) + (ks4[2] + ks4[3])) * (CH ? 1.0f : decay);
      const float u = beta * (now.v - ks);
      float o4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < R; ++r) {
        S[r] = fmaf(now.k[r >> 2][r & 3], u, CH ? S[r] : decay * S[r]);
        o4[r & 3] = fmaf(S[r], now.q[r >> 2][r & 3], o4[r & 3]);
      }
      const float o = lanes_sum<L>((o4[0] + o4[1]) + (o4[2] + o4[3]));
      if (part == 0 && col_ok) out[(long)(m.q_off + i) * ldo + head * DV + col] = o;
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (row0 + r < D && col_ok) mine[(long)(row0 + r) * DV + col] = S[r];
}

__global__ __launch_bounds__(256) void delta_conv_state_kernel(const float* __restrict__ raw, long ld, int C, int M,
                                                               const SeqMeta* __restrict__ seqs, float* __restrict__ state,
                                                               long state_stride, long conv_at) {
  const SeqMeta m = seqs[blockIdx.x];
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (m.q_len <= 0 || c >= C) return;
  float* kept = state + (long)m.table_row * state_stride + conv_at;
  // place a holds the input at position kv_len - (M - 1) + a: one of this step's, or one the state already holds
  // further on (read before the ascending walk overwrites it)
  for (int a = 0; a < M - 1; ++a) {
    const int p = m.kv_len - (M - 1) + a;
    kept[(long)a * C + c] = p >= m.q_start ? raw[(long)(m.q_off + p - m.q_start) * ld + c]
                                           : kept[(long)(p - m.q_start + M - 1) * C + c];
  }
}

}  // namespace ls

using namespace ls;

extern "C" int ls_streams_max() { return kMaxStreams; }
extern "C" int ls_streams_max_width() { return 1024 * kStreamChunks; }

extern "C" int ls_streams_step(int dtype, float* X, long ldx, int n, int width, const float* P, int slices, int p_rows,
                               const float* mix, const float* gain, const float* take, const float* weight, float eps,
                               void* out, long ld_out, const int* rows, int n_rows, void* stream) {
  LS_REQUIRE(n_rows > 0 && n > 0 && n <= kMaxStreams && width > 0 && width <= 1024 * kStreamChunks && ldx >= (long)n * width,
             "streams_step: %d copies of %d elements (at most %d of %d)", n, width, kMaxStreams, 1024 * kStreamChunks);
  LS_REQUIRE(X && (P || out), "streams_step: nothing to do");
  LS_REQUIRE(!P || (slices > 0 && p_rows > 0 && mix && gain), "streams_step: a write needs slices, mix and gain");
  LS_REQUIRE(!out || (weight && ld_out >= width && eps > 0.f), "streams_step: a read needs a weight and eps");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long p_stride = (long)p_rows * width;
  LS_REQUIRE(dtype == kF32 || dtype == kBF16, "streams_step: unknown dtype %d", dtype);
  const size_t lds = out ? (size_t)((width + 3) / 4) * 16 : 0;
#define LS_STREAMS(N_)                                                                                               \
  case N_:                                                                                                           \
    if (dtype == kF32)                                                                                               \
      hipLaunchKernelGGL((streams_step_kernel<float, N_>), dim3(n_rows), dim3(256), lds, s, X, ldx, width, P, slices, \
                         p_stride, mix, gain, take, weight, eps, (float*)out, ld_out, rows);                         \
    else                                                                                                             \
      hipLaunchKernelGGL((streams_step_kernel<bf16_t, N_>), dim3(n_rows), dim3(256), lds, s, X, ldx, width, P, slices, \
                         p_stride, mix, gain, take, weight, eps, (bf16_t*)out, ld_out, rows);                        \
    break;
  switch (n) {
    LS_STREAMS(1) LS_STREAMS(2) LS_STREAMS(3) LS_STREAMS(4) LS_STREAMS(5) LS_STREAMS(6) LS_STREAMS(7) LS_STREAMS(8)
  }
#undef LS_STREAMS
  return check_launch("streams_step");
}

extern "C" int ls_latent_post(int dtype, const float* raw, long ld, int n_tokens, int QR, int CR, int RD, int Dp,
                              int has_kv, const float* a_weight, const float* c_weight, float eps, const float* cos_table,
                              const float* sin_table, int rot, int table_positions, int max_pos, const int* tok_seq,
                              const int* tok_pos, const void* seqs, const int* table, int table_stride, void* a_out,
                              long lda, void* k_pages, void* v_pages, int page_size, void* stream) {
  LS_REQUIRE(n_tokens > 0 && QR > 0 && raw && a_out && a_weight && lda >= QR && eps > 0.f, "latent_post: bad query latent");
  LS_REQUIRE(ld >= QR + (has_kv ? CR + RD : 0), "latent_post: rows of %ld floats are too short", ld);
  if (has_kv) {
    LS_REQUIRE(CR > 0 && RD >= 0 && Dp >= CR + RD && c_weight && k_pages && v_pages && table && seqs && tok_seq && tok_pos &&
                   page_size > 0 && table_stride > 0,
               "latent_post: bad key/value latent");
    LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= RD, "latent_post: %d rotated dimensions of %d", rot, RD);
    LS_REQUIRE(rot == 0 || (cos_table && sin_table && max_pos < table_positions),
               "latent_post: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
    LS_REQUIRE(max_pos / page_size < table_stride, "latent_post: position %d is beyond the block table", max_pos);
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define LS_LATENT_POST(T_)                                                                                            \
  hipLaunchKernelGGL(latent_post_kernel<T_>, dim3(n_tokens), dim3(256), 0, s, raw, ld, QR, CR, RD, Dp, has_kv, a_weight, \
                     c_weight, eps, cos_table, sin_table, rot, tok_seq, tok_pos, (const SeqMeta*)seqs, table,         \
                     table_stride, (T_*)a_out, lda, (T_*)k_pages, (T_*)v_pages, page_size)
  if (dtype == kF32)
    LS_LATENT_POST(float);
  else if (dtype == kBF16)
    LS_LATENT_POST(bf16_t);
  else
    return fail("latent_post: unknown dtype %d", dtype);
#undef LS_LATENT_POST
  return check_launch("latent_post");
}

extern "C" int ls_latent_query(int dtype, const float* qf, long ld, int n_tokens, int H, int D, int RD, int CR, int Dp,
                               const float* cos_table, const float* sin_table, int rot, int table_positions, int max_pos,
                               const int* tok_pos, void* plain_out, long ldp, void* q_out, long ldq, void* stream) {
  LS_REQUIRE(n_tokens > 0 && H > 0 && D > 0 && RD >= 0 && CR > 0 && Dp >= CR + RD, "latent_query: bad sizes");
  LS_REQUIRE(qf && plain_out && q_out && tok_pos && ld >= (long)H * (D + RD) && ldp >= (long)H * D && ldq >= (long)H * Dp,
             "latent_query: bad operands");
  LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= RD, "latent_query: %d rotated dimensions of %d", rot, RD);
  LS_REQUIRE(rot == 0 || (cos_table && sin_table && max_pos < table_positions),
             "latent_query: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long total = (long)n_tokens * H * (D + Dp - CR);
  const unsigned blocks = (unsigned)((total + 255) / 256);
#define LS_LATENT_QUERY(T_)                                                                                          \
  hipLaunchKernelGGL(latent_query_kernel<T_>, dim3(blocks), dim3(256), 0, s, qf, ld, n_tokens, H, D, RD, CR, Dp,     \
                     cos_table, sin_table, rot, tok_pos, (T_*)plain_out, ldp, (T_*)q_out, ldq)
  if (dtype == kF32)
    LS_LATENT_QUERY(float);
  else if (dtype == kBF16)
    LS_LATENT_QUERY(bf16_t);
  else
    return fail("latent_query: unknown dtype %d", dtype);
#undef LS_LATENT_QUERY
  return check_launch("latent_query");
}

extern "C" int ls_heads_product(int dtype, const void* x, long ldx, int x_stride, const void* w, int H, int N, int K,
                                int n_rows, void* out, long ldo, int o_stride, void* stream) {
  LS_REQUIRE(n_rows > 0 && H > 0 && N > 0 && K > 0 && x && w && out, "heads_product: bad sizes");
  LS_REQUIRE(x_stride >= 0 && o_stride >= 0 && ldx >= (long)(H - 1) * x_stride + K && ldo >= (long)(H - 1) * o_stride + N,
             "heads_product: the heads do not fit the rows");
  LS_REQUIRE(dtype == kF32 || dtype == kBF16, "heads_product: unknown dtype %d", dtype);
  const int vec = dtype == kF32 ? 4 : 8;
  LS_REQUIRE(reinterpret_cast<uintptr_t>(w) % 16 == 0, "heads_product: the weights must be 16-byte aligned");
  const int x_aligned = reinterpret_cast<uintptr_t>(x) % 16 == 0 && ldx % vec == 0 && x_stride % vec == 0 && K % vec == 0;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool many = n_rows > 64;
  const int rows_a_block = many ? 64 : 16;
  const dim3 grid((n_rows + rows_a_block - 1) / rows_a_block, H, (N + 63) / 64);
#define LS_HEADS(T_, RT_)                                                                                            \
  hipLaunchKernelGGL((heads_product_kernel<T_, RT_>), grid, dim3(256), 0, s, (const T_*)x, ldx, x_stride, (const T_*)w, N, \
                     K, n_rows, (T_*)out, ldo, o_stride, x_aligned)
  if (dtype == kF32) {
    if (many) LS_HEADS(float, 4); else LS_HEADS(float, 1);
  } else {
    if (many) LS_HEADS(bf16_t, 4); else LS_HEADS(bf16_t, 1);
  }
#undef LS_HEADS
  return check_launch("heads_product");
}

extern "C" int ls_delta_max_dim() { return 256; }

// The rows of a head's queries and keys in the scratch buffer: the head size rounded up to what the lanes of the
// recurrence hold (16, 32, 64, 128 or 256).
extern "C" int ls_delta_padded_dim(int D) {
  int dp = 16;
  while (dp < D) dp *= 2;
  return dp;
}

// Floats of scratch that ls_delta_rule needs: qk, vv and gates.
extern "C" long ls_delta_scratch_floats(int n_tokens, int G, int H, int D, int DV) {
  return (long)n_tokens * (2L * G * ls_delta_padded_dim(D) + (long)H * DV + 2L * H);
}
// ... and with a decay a key channel (chan given): the decays as well.
extern "C" long ls_delta_scratch_floats_channel(int n_tokens, int G, int H, int D, int DV) {
  return ls_delta_scratch_floats(n_tokens, G, H, D, DV) + (long)n_tokens * H * ls_delta_padded_dim(D);
}

extern "C" int ls_delta_rule(const float* raw, long ld, int n_tokens, int G, int H, int D, int DV, int M,
                             const float* taps, const float* a_log, const float* dt_bias, float unit_eps,
                             const int* tok_seq, const int* tok_pos, const void* seqs, int n_seqs, float* state,
                             long state_stride, float* scratch, float* out, long ldo, const float* chan, long ldc,
                             void* stream) {
  // chan [T][ldc] (or null): the logits of a decay a head and key channel, H * D a token; dt_bias then has H * D
  // entries, raw needs no `a` columns, and the scratch is that of ls_delta_scratch_floats_channel.
  LS_REQUIRE(!chan || ldc >= (long)H * D, "delta_rule: the channel decays' rows are too short");
  LS_REQUIRE(n_tokens > 0 && n_seqs > 0 && G > 0 && H > 0 && H % G == 0 && D > 0 && D <= 256 && DV > 0 && M >= 1,
             "delta_rule: bad sizes (%d key heads, %d heads, keys of %d, values of %d, %d taps)", G, H, D, DV, M);
  const long C = 2L * G * D + (long)H * DV;
  const long conv_at = (long)H * D * DV;
  LS_REQUIRE(ld >= C + (chan ? 1L : 2L) * H && state_stride >= conv_at + (long)(M - 1) * C && ldo >= (long)H * DV,
             "delta_rule: rows or state are too short");
  LS_REQUIRE(raw && taps && a_log && dt_bias && tok_seq && tok_pos && seqs && state && scratch && out,
             "delta_rule: null operand");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(scratch) % 16 == 0, "delta_rule: the scratch must be 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int dp = ls_delta_padded_dim(D);
  float* qk = scratch;
  float* vv = qk + (long)n_tokens * 2 * G * dp;
  float* gates = vv + (long)n_tokens * H * DV;
  float* decays = chan ? gates + (long)n_tokens * H * 2 : nullptr;
  const long units = (long)n_tokens * (2 * G + H + (chan ? H : 1));
  hipLaunchKernelGGL(delta_prep_kernel, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, s, raw, ld, n_tokens, G, H, D, DV,
                     dp, M, taps, a_log, dt_bias, unit_eps, tok_seq, tok_pos, (const SeqMeta*)seqs, state, state_stride,
                     conv_at, qk, vv, gates, chan, ldc, decays);
#define LS_DELTA(R_, L_)                                                                                              \
  do {                                                                                                                \
    if (chan)                                                                                                         \
      hipLaunchKernelGGL((delta_rule_kernel<R_, L_, true>), dim3(n_seqs * H, (DV * L_ + 63) / 64), dim3(64), 0, s, qk, vv, \
                         gates, decays, G, H, D, DV, (const SeqMeta*)seqs, state, state_stride, out, ldo);            \
    else                                                                                                              \
      hipLaunchKernelGGL((delta_rule_kernel<R_, L_, false>), dim3(n_seqs * H, (DV * L_ + 63) / 64), dim3(64), 0, s, qk, vv, \
                         gates, decays, G, H, D, DV, (const SeqMeta*)seqs, state, state_stride, out, ldo);            \
  } while (0)
  switch (dp) {
    case 16: LS_DELTA(4, 4); break;
    case 32: LS_DELTA(8, 4); break;
    case 64: LS_DELTA(8, 8); break;
    case 128: LS_DELTA(8, 16); break;
    default: LS_DELTA(16, 16); break;
  }
#undef LS_DELTA
  if (M > 1)
    hipLaunchKernelGGL(delta_conv_state_kernel, dim3(n_seqs, (unsigned)((C + 255) / 256)), dim3(256), 0, s, raw, ld, (int)C,
                       M, (const SeqMeta*)seqs, state, state_stride, conv_at);
  return check_launch("delta_rule");
}
