// Kernels of the mixers, norms and activations beyond the softmax-attention decoder: Dynamic Tanh
// norm (with the deferred residual addition), the clamped gated unit, the soft cap of the logits,
// the post pass of an attention projection with biases, partial rotation, value mixing and cache
// write for keys and values of different sizes (and its sibling with a norm over the whole projection,
// rotation of neighbouring pairs and keys that are the values), the linear recurrence with per-row decay and write
// gates (HGRN2, retention), and the per-head RMS norm with an optional weight and gate.
//
// Everything here is computed in float whatever the compute dtype T is: T is the type of what a
// matrix product reads next (and of the cache).  Per-row reductions have an order fixed by the
// row's sizes alone; the recurrence walks a request's tokens in order, so nothing depends on how
// the request was cut into steps or on what else is in the batch.

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

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x * sigmoidf_(x); }

// ---------------------------------------------------------------------------
// Dynamic Tanh norm of rows of the float residual stream, elementwise:
//   h[row] += P[0][row] + P[1][row] + ...   (when P is given; slices ascending, from +0)
//   out[r] = tanh(alpha * h[row]) * w + b
// `row` = rows[r] when a row list is given.  alpha is one float on the device.
// out == nullptr: the addition only.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void dyt_kernel(float* __restrict__ h, const float* __restrict__ P, int slices,
                                                  long p_stride, const float* __restrict__ weight,
                                                  const float* __restrict__ bias, const float* __restrict__ alpha,
                                                  T* __restrict__ out, const int* __restrict__ rows, int width,
                                                  long ldh, long ld_out) {
  const int r_out = blockIdx.x;
  const long row = rows ? rows[r_out] : r_out;
  float* src = h + row * ldh;
  const float a = out ? alpha[0] : 0.f;
  // one element a thread (blockIdx.y walks the row): the slice sums of an element are requested together
  const int e = blockIdx.y * 256 + threadIdx.x;
  if (e >= width) return;
  float v = src[e];
  if (P) {
    const float* p = P + row * width + e;
    float sum = 0.f;
    int s = 0;
    for (; s + 4 <= slices; s += 4) {
      const float p0 = p[s * p_stride], p1 = p[(s + 1) * p_stride], p2 = p[(s + 2) * p_stride], p3 = p[(s + 3) * p_stride];
      sum = (((sum + p0) + p1) + p2) + p3;
    }
    for (; s < slices; ++s) sum = sum + p[s * p_stride];
    v = v + sum;
    src[e] = v;
  }
  if (out) out[(long)r_out * ld_out + e] = from_f32<T>(tanhf(a * v) * weight[e] + bias[e]);
}

// ---------------------------------------------------------------------------
// Clamped gated unit on float rows x [rows][2 * width] (gates, then ups):
//   g = min(gate, limit); u = clamp(up, -limit, limit); out = g * sigmoid(alpha * g) * (u + 1)
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void glu_clamped_kernel(const float* __restrict__ x, long ldx, T* __restrict__ out,
                                                          long ldo, int rows, int width, float limit, float alpha) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * width) return;
  const long r = idx / width;
  const int c = (int)(idx % width);
  const float g = fminf(x[r * ldx + c], limit);
  const float u = fminf(fmaxf(x[r * ldx + width + c], -limit), limit);
  out[r * ldo + c] = from_f32<T>((g * sigmoidf_(alpha * g)) * (u + 1.0f));
}

// Soft cap in place: x = cap * tanh(x / cap).
__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long ld, int rows, int width, float cap) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * width) return;
  float* at = x + (idx / width) * ld + idx % width;
  *at = cap * tanhf(*at / cap);
}

// ---------------------------------------------------------------------------
// Rotation of element i of a head (rot leading dimensions, pair (i, i + rot/2)) at a position.
// `own` and `other` are the element and its partner; cos/sin tables [positions][rot/2].
// ---------------------------------------------------------------------------
__device__ __forceinline__ float rotate_element(float own, float other, int i, int rot, const float* cos_row,
                                                const float* sin_row) {
  const int half = rot >> 1;
  if (i < half) return own * cos_row[i] - other * sin_row[i];
  return own * cos_row[i - half] + other * sin_row[i - half];
}

// ---------------------------------------------------------------------------
// Post pass of an attention projection raw [T][ld] float = q (H heads of D) | k (G of D) | v (G of DV):
//   biases added; q and k rotated on their first `rot` dimensions at the token's position;
//   q -> q_out [T][H*D] (T);  k -> key pages [page][G][slot][D];
//   v -> value pages [page][G][DV][slot], after value mixing:
//     mode 1: v is also kept in v_first [T][G*DV] (float) for the layers that follow;
//     mode 2: v = (1 - lambda) v + lambda v_first[t], lambda one float on the device.
// One thread per element.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void talk_qkv_kernel(
    const float* __restrict__ raw, long ld, int n_tokens, int H, int G, int D, int DV, const float* __restrict__ bias,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot, const int* __restrict__ tok_seq,
    const int* __restrict__ tok_pos, const SeqMeta* __restrict__ seqs, const int* __restrict__ table, int table_stride,
    T* __restrict__ q_out, long ldq, T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int vmix_mode,
    const float* __restrict__ vmix, float* __restrict__ v_first, long ldv) {
  const int width = H * D + G * D + G * DV;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)n_tokens * width) return;
  const int t = (int)(idx / width);
  const int e = (int)(idx % width);
  const float* row = raw + (long)t * ld;
  const int pos = tok_pos[t];
  float own = row[e] + (bias ? bias[e] : 0.f);
  const int qk = (H + G) * D;
  if (e < qk) {
    const int i = e % D;
    if (i < rot) {
      const int half = rot >> 1;
      const int pe = i < half ? e + half : e - half;
      const float other = row[pe] + (bias ? bias[pe] : 0.f);
      own = rotate_element(own, other, i, rot, cos_table + (long)pos * half, sin_table + (long)pos * half);
    }
    if (e < H * D) {
      q_out[(long)t * ldq + e] = from_f32<T>(own);
      return;
    }
  }
  const int table_row = seqs[tok_seq[t]].table_row;
  const int page = table[(long)table_row * table_stride + pos / page_size];
  const int slot = pos % page_size;
  if (e < qk) {
    const int g = (e - H * D) / D, i = e % D;
    if (page >= 0) k_pages[(((long)page * G + g) * page_size + slot) * D + i] = from_f32<T>(own);
    return;
  }
  const int c = e - qk;  // column of the token's values, g * DV + i
  if (vmix_mode == 1) v_first[(long)t * ldv + c] = own;
  if (vmix_mode == 2) {
    const float lam = vmix[0];
    own = (1.0f - lam) * own + lam * v_first[(long)t * ldv + c];
  }
  const int g = c / DV, i = c % DV;
  if (page >= 0) v_pages[(((long)page * G + g) * DV + i) * page_size + slot] = from_f32<T>(own);
}

// ---------------------------------------------------------------------------
// Post pass of an attention projection raw [T][ld] float = q (H heads of D) | k (G of D) | v (G of DV, absent
// when the keys are the values) | whatever follows (an output gate, which this pass leaves alone):
//   biases added (bias [H*D + G*D (+ G*DV)] or null);
//   v = k as projected, with its bias, before any norm (keys_are_values; DV == D);
//   q and k each divided by the root mean square over ALL their heads at once (the whole projection is one
//   vector: x / sqrt(mean(x^2) + eps)), times a weight an element (q_norm [H*D], k_norm [G*D]; null: no norm);
//   or, with per_head, every head of q and of k divided by its own root mean square over D (per_head 1: no weights;
//   per_head 2: times q_norm [D] / k_norm [D], one weight vector that all heads share);
//   q and k rotated on their first `rot` dimensions at the token's position, pairs (i, i + rot/2) or, with
//   `neighbours`, (2i, 2i + 1), angle tables [positions][rot/2];
//   q -> q_out [T][H*Dp] (T);  k -> key pages [page][G][slot][Dp], Dp >= D with zeros beyond D (a kernel that loads
//   16 bytes at a time wants heads of a multiple of that);  v -> value pages [page][G][DV][slot].
// A token's row is dealt to workgroups of 256 elements (each forms the row's sums of squares itself where a norm
// is asked for).  The sums of squares: thread t adds the squares of elements t, t + 256, ... in
// ascending order, then a butterfly over the wave and the wave sums in wave order: a function of the sizes only.
// ---------------------------------------------------------------------------
constexpr int kMaxNormedHeads = 1024;  // query and key heads of a projection whose heads are normalised one by one

__device__ __forceinline__ float block_sum256(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  return ((scratch[0] + scratch[1]) + scratch[2]) + scratch[3];
}

template <typename T>
__global__ __launch_bounds__(256) void qkv_post_kernel(
    const float* __restrict__ raw, long ld, int H, int G, int D, int Dp, int DV, int keys_are_values, int per_head,
    const float* __restrict__ bias, const float* __restrict__ q_norm, const float* __restrict__ k_norm, float eps,
    const float* __restrict__ cos_table, const float* __restrict__ sin_table, int rot, int neighbours,
    const int* __restrict__ tok_seq, const int* __restrict__ tok_pos, const SeqMeta* __restrict__ seqs,
    const int* __restrict__ table, int table_stride, T* __restrict__ q_out, long ldq, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int page_size) {
  __shared__ float scratch[4];
  __shared__ float head_scale[kMaxNormedHeads];
  const int t = blockIdx.x;
  const float* row = raw + (long)t * ld;
  const int pos = tok_pos[t];
  const int nq = H * D, nk = G * D, nv = G * DV;
  float rq = 1.0f, rk = 1.0f;
  if (per_head) {
    // a wave a head of q | k: lane i adds the squares of the elements i, i + 64, ... ascending, then a butterfly.
    // Where the workgroups of a token each write one run of 256 elements, a workgroup needs the heads of its run only.
    int h_lo = 0, h_hi = H + G;
    if ((long)gridDim.y * 256 >= (long)(H + G) * Dp + (long)G * DV) {
      h_lo = min(H + G, (int)(blockIdx.y * 256 / Dp));
      h_hi = min(H + G, (int)((blockIdx.y * 256 + 255) / Dp) + 1);
    }
    for (int head = h_lo + (threadIdx.x >> 6); head < h_hi; head += 4) {
      float part = 0.f;
      for (int i = threadIdx.x & 63; i < D; i += 64) {
        const float x = row[head * D + i] + (bias ? bias[head * D + i] : 0.f);
        part = part + x * x;
      }
      const float total = wave_sum(part);
      if ((threadIdx.x & 63) == 0) head_scale[head] = 1.0f / sqrtf(total / (float)D + eps);
    }
    __syncthreads();
  }
  if (q_norm && !per_head) {
    float part = 0.f;
    for (int e = threadIdx.x; e < nq; e += 256) {
      const float x = row[e] + (bias ? bias[e] : 0.f);
      part = part + x * x;
    }
    rq = 1.0f / sqrtf(block_sum256(part, scratch) / (float)nq + eps);
  }
  if (k_norm && !per_head) {
    float part = 0.f;
    for (int e = threadIdx.x; e < nk; e += 256) {
      const float x = row[nq + e] + (bias ? bias[nq + e] : 0.f);
      part = part + x * x;
    }
    rk = 1.0f / sqrtf(block_sum256(part, scratch) / (float)nk + eps);
  }
  const int table_row = seqs[tok_seq[t]].table_row;
  const int page = table[(long)table_row * table_stride + pos / page_size];
  const int slot = pos % page_size;
  const int half = rot >> 1;
  const float* cos_row = cos_table + (long)pos * half;
  const float* sin_row = sin_table + (long)pos * half;
  // element e of q | k as the attention reads it: bias, norm, rotation
  auto finished = [&](int e) LS_INLINED {
    const bool is_q = e < nq;
    const float* w = per_head ? nullptr : (is_q ? q_norm : k_norm);
    const float* hw = per_head == 2 ? (is_q ? q_norm : k_norm) : nullptr;   // a head's weights, shared by the heads
    const int at = is_q ? e : e - nq;      // index into the norm weight
    const float r = is_q ? rq : rk;
    float own = row[e] + (bias ? bias[e] : 0.f);
    const int i = e % D;
    if (w) own = own * r * w[at];
    if (per_head) own = own * head_scale[e / D];
    if (hw) own = own * hw[i];
    if (i < rot) {
      const int pe = neighbours ? (e ^ 1) : (i < half ? e + half : e - half);
      float other = row[pe] + (bias ? bias[pe] : 0.f);
      if (w) other = other * r * w[is_q ? pe : pe - nq];
      if (per_head) other = other * head_scale[e / D];
      if (hw) other = other * hw[pe % D];
      const int pair = neighbours ? (i >> 1) : (i < half ? i : i - half);
      const bool lower = neighbours ? (i & 1) == 0 : i < half;
      own = lower ? own * cos_row[pair] - other * sin_row[pair] : own * cos_row[pair] + other * sin_row[pair];
    }
    return own;
  };
  // the workgroups of a token (gridDim.y of them) deal its elements of q | k | v among themselves, 256 at a time;
  // queries and keys are written with Dp >= D elements a head, zeros beyond D
  const int oq = H * Dp, ok = G * Dp;
  for (int e = blockIdx.y * 256 + threadIdx.x; e < oq + ok + nv; e += gridDim.y * 256) {
    if (e < oq) {
      const int head = e / Dp, i = e % Dp;
      q_out[(long)t * ldq + e] = from_f32<T>(i < D ? finished(head * D + i) : 0.f);
    } else if (page < 0) {
      break;
    } else if (e < oq + ok) {
      const int g = (e - oq) / Dp, i = (e - oq) % Dp;
      k_pages[(((long)page * G + g) * page_size + slot) * Dp + i] = from_f32<T>(i < D ? finished(nq + g * D + i) : 0.f);
    } else {
      const int c = e - oq - ok;
      const int from = keys_are_values ? nq + c : nq + nk + c;
      const float v = row[from] + (bias ? bias[from] : 0.f);
      const int g = c / DV, i = c % DV;
      v_pages[(((long)page * G + g) * DV + i) * page_size + slot] = from_f32<T>(v);
    }
  }
}

// ---------------------------------------------------------------------------
// Linear recurrence with a decay and a write gate for every row of the state, one head:
//   S_t = diag(a_t) S_(t-1) + b_t v_t^T,   o_t = S_t^T q_t,     S [D][DV] float, kept per request.
// mode 0 (HGRN2): q = silu(q_raw), f = lower + (1 - lower) sigmoid(f_raw + f_bias), a = f, b = 1 - f.
// mode 1 (retention): q = rotate(q_raw), b = rotate(k_raw) D^(-1/2), a = decay[head] for every row.
// raw [T][ld] float holds q_raw at q_at, f_raw / k_raw at ab_at, v at v_at (H heads each).
//
// Two launches.  The first computes q, a and b of every token once, elementwise over the whole step
// (they do not depend on the state): gates [T][H][3][dp], dp = D rounded up to a multiple of 32,
// zeros beyond D.  The second walks the tokens: a workgroup takes (request, head, block of 16
// columns of the state).  A wave holds 16 rows of these columns: lane (column l16 = lane / 4,
// quarter = lane % 4) keeps the rows 16 g + 4 quarter + {0..3} of its column in registers (few rows a lane
// and many waves: the walk is a chain of dependent instructions, and a second wave on a SIMD fills its gaps), and the
// waves walk the request's tokens in order, sixteen at a time: their gates and values are copied to
// LDS by all threads, every lane adds its rows' part of o_t (fused multiply-adds, written as
// such), the four quarters of a column are neighbouring lanes and are added by exchanges inside the quad,
// and the waves' parts are added in wave order.  The order of all sums is a function of D alone.
//
// The walk is software-pipelined over chunks of sixteen tokens, with two sets of LDS buffers: while
// the waves walk the tokens of one chunk, the gates and values of the next are already requested
// (into registers); after the walk they are written to the other set, one barrier follows, and the
// waves' parts of the chunk's o_t are added and stored while the next chunk is walked.
// ---------------------------------------------------------------------------
constexpr int kRecRows = 4;     // rows of the state a lane keeps (a multiple of 4)
constexpr int kRecCols = 16;    // columns of the state a workgroup takes
constexpr int kRecWaveRows = 4 * kRecRows;  // rows a wave holds
constexpr int kRecTokens = 16;  // tokens copied at a time
constexpr int kRecPer = kRecTokens * 3 * kRecWaveRows / (4 * 64);  // vectors of four gates a thread copies a chunk
constexpr int kRecVPer = kRecTokens * kRecCols / 64;                // the most values a thread fetches (one wave)

__global__ __launch_bounds__(256) void linrec_gates_kernel(
    int mode, const float* __restrict__ raw, long ld, int q_at, int ab_at, int n_tokens, int H, int D, int dp,
    const float* __restrict__ p0, const float* __restrict__ p1, const float* __restrict__ cos_table,
    const float* __restrict__ sin_table, int rot, const int* __restrict__ tok_pos, float* __restrict__ gates) {
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)n_tokens * H * dp) return;
  const int row = (int)(idx % dp), head = (int)((idx / dp) % H), t = (int)(idx / ((long)dp * H));
  float q = 0.f, a = 0.f, b = 0.f;
  if (row < D) {
    const float* src = raw + (long)t * ld;
    const int e = head * D + row;
    if (mode == 0) {
      const float lower = p0[e];
      const float f = lower + (1.0f - lower) * sigmoidf_(src[ab_at + e] + (p1 ? p1[e] : 0.f));
      q = siluf_(src[q_at + e]);
      a = f;
      b = 1.0f - f;
    } else {
      q = src[q_at + e];
      b = src[ab_at + e];
      if (row < rot) {
        const int half = rot >> 1;
        const int pe = row < half ? e + half : e - half;
        const long pos = tok_pos[t];
        q = rotate_element(q, src[q_at + pe], row, rot, cos_table + pos * half, sin_table + pos * half);
        b = rotate_element(b, src[ab_at + pe], row, rot, cos_table + pos * half, sin_table + pos * half);
      }
      b = b * (1.0f / sqrtf((float)D));
      a = p0[head];
    }
  }
  float* dst = gates + ((long)t * H + head) * 3 * dp + row;
  dst[0] = q;
  dst[dp] = a;
  dst[2 * dp] = b;
}

// A barrier between the waves' LDS writes and reads that waits for this wave's LDS operations only: the global
// loads of the next chunk stay on their way across it.
__device__ __forceinline__ void lds_barrier() { __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Sum over the four neighbouring lanes 4k .. 4k + 3 (a DPP exchange inside the quad, no LDS traffic): first the
// pairs (l, l ^ 1), then the pairs of pairs, so all four lanes end with the same bits.
__device__ __forceinline__ float quad_sum(float v) {
  v = v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0xB1, 0xF, 0xF, true));  // lanes 1 0 3 2
  v = v + __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), 0x4E, 0xF, 0xF, true));  // lanes 2 3 0 1
  return v;
}

__global__ __launch_bounds__(1024) void linrec_kernel(const float* __restrict__ gates, const float* __restrict__ raw,
                                                     long ld, int v_at, int H, int D, int DV,
                                                     const SeqMeta* __restrict__ seqs, float* __restrict__ state,
                                                     float* __restrict__ out, long ldo) {
  extern __shared__ float lds[];
  const int seq = blockIdx.x / H, head = blockIdx.x % H, cb = blockIdx.y;
  const SeqMeta m = seqs[seq];
  if (m.q_len <= 0) return;
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int l16 = lane >> 2, quarter = lane & 3;  // four neighbouring lanes share a column
  const int dp = waves * kRecWaveRows;  // D rounded up to the rows the waves hold
  const int token = 3 * dp;             // floats of a token's gates: q, a, b
  const int set = kRecTokens * token + kRecTokens * kRecCols + waves * kRecTokens * kRecCols;  // floats of one set
  const int c = cb * kRecCols + l16;
  const bool col_ok = c < DV;
  const int row0 = g * kRecWaveRows + quarter * kRecRows;
  float* mine = state + (((long)m.table_row * H + head) * D) * DV;
  float S[kRecRows];
#pragma unroll
  for (int r = 0; r < kRecRows; ++r) S[r] = (row0 + r < D && col_ok) ? mine[(long)(row0 + r) * DV + c] : 0.f;
  const int v_per = (kRecTokens * kRecCols + (int)blockDim.x - 1) / (int)blockDim.x;
  // a chunk's gates are kRecTokens * token consecutive floats of one head: token t at (t * H + head) * token.
  // Thread i copies the vectors i, i + threads, ...; vector k lies in token k / (token / 4).
  const int vec_a_token = token / 4;
  int v_tt[kRecPer], v_in[kRecPer];
#pragma unroll
  for (int j = 0; j < kRecPer; ++j) {
    const int k = j * (int)blockDim.x + (int)threadIdx.x;
    v_tt[j] = k / vec_a_token;
    v_in[j] = 4 * (k % vec_a_token);
  }
  // the operands of the next chunk are requested before a chunk is walked
  f32x4 rg[kRecPer];
  float rv[kRecVPer];

  auto request = [&](int t0) LS_INLINED {
    const int n = min(kRecTokens, m.q_len - t0);
#pragma unroll
    for (int j = 0; j < kRecPer; ++j) {
      const bool in = v_tt[j] < n;
      const float* src = gates + ((long)(m.q_off + t0 + (in ? v_tt[j] : 0)) * H + head) * token + v_in[j];
      rg[j] = *reinterpret_cast<const f32x4*>(src);
    }
#pragma unroll
    for (int j = 0; j < kRecVPer; ++j) {
      const int idx = j * (int)blockDim.x + (int)threadIdx.x;
      const int tt = idx / kRecCols, col = cb * kRecCols + idx % kRecCols;
      rv[j] = (j < v_per && tt < n && col < DV) ? raw[(long)(m.q_off + t0 + tt) * ld + v_at + head * DV + col] : 0.f;
    }
  };

  auto deposit = [&](float* base) LS_INLINED {
#pragma unroll
    for (int j = 0; j < kRecPer; ++j)
      *reinterpret_cast<f32x4*>(base + v_tt[j] * token + v_in[j]) = rg[j];
    float* v_s = base + kRecTokens * token;  // [tokens][columns]
#pragma unroll
    for (int j = 0; j < kRecVPer; ++j) {
      const int idx = j * (int)blockDim.x + (int)threadIdx.x;
      if (j < v_per && idx < kRecTokens * kRecCols) v_s[idx] = rv[j];
    }
  };

  // one chunk: walk the tokens of the set `base`, leave the waves' parts of o_t there
  auto walk_chunk = [&](float* base, int n) LS_INLINED {
    const float* v_s = base + kRecTokens * token;
    float* o_s = base + kRecTokens * token + kRecTokens * kRecCols;  // [waves][tokens][columns]
    // a token's operands: q, a and b of the lane's rows and its column's value
    struct Operands {
      f32x4 q[kRecRows / 4], a[kRecRows / 4], b[kRecRows / 4];
      float v;
    };
    auto fetch = [&](int tt) LS_INLINED {
      Operands x;
      const float* qa = base + tt * token + row0;
      x.v = v_s[tt * kRecCols + l16];
#pragma unroll
      for (int k = 0; k < kRecRows / 4; ++k) {
        x.q[k] = *reinterpret_cast<const f32x4*>(qa + 4 * k);
        x.a[k] = *reinterpret_cast<const f32x4*>(qa + dp + 4 * k);
        x.b[k] = *reinterpret_cast<const f32x4*>(qa + 2 * dp + 4 * k);
      }
      return x;
    };
    auto step = [&](const Operands& x, int tt) LS_INLINED {
      float o = 0.f;
#pragma unroll
      for (int r = 0; r < kRecRows; ++r) {
        S[r] = fmaf(x.a[r >> 2][r & 3], S[r], x.b[r >> 2][r & 3] * x.v);
        o = fmaf(S[r], x.q[r >> 2][r & 3], o);
      }
      o = quad_sum(o);  // the four quarters of the wave: rows kRecRows * quarter .. of the same column
      if (quarter == 0) o_s[(g * kRecTokens + tt) * kRecCols + l16] = o;
    };
    if (n == kRecTokens) {
      // a full chunk is unrolled, and the operands of the token after next are requested before a token is walked
      Operands ahead = fetch(0), next = fetch(1);
#pragma unroll
      for (int tt = 0; tt < kRecTokens; ++tt) {
        const Operands now = ahead;
        ahead = next;
        if (tt + 2 < kRecTokens) next = fetch(tt + 2);
        step(now, tt);
      }
    } else {
      for (int tt = 0; tt < n; ++tt) step(fetch(tt), tt);
    }
  };

  // the waves' parts of a chunk are added in wave order and stored (while the next chunk is walked: that chunk
  // writes the other set, and the barrier at its end stands before the chunk after it writes this one again)
  auto store_chunk = [&](const float* base, int t0, int n) LS_INLINED {
    const float* o_s = base + kRecTokens * token + kRecTokens * kRecCols;
    for (int idx = threadIdx.x; idx < n * kRecCols; idx += blockDim.x) {
      const int tt = idx / kRecCols, l = idx % kRecCols, col = cb * kRecCols + l;
      float o = 0.f;
      for (int w = 0; w < waves; ++w) o = o + o_s[(w * kRecTokens + tt) * kRecCols + l];
      if (col < DV) out[(long)(m.q_off + t0 + tt) * ldo + head * DV + col] = o;
    }
  };

  request(0);
  deposit(lds);
  lds_barrier();
  int at = 0;
  for (int t0 = 0; t0 < m.q_len; t0 += kRecTokens, at ^= 1) {
    const int n = min(kRecTokens, m.q_len - t0);
    const bool more = t0 + kRecTokens < m.q_len;
    if (more) request(t0 + kRecTokens);
    walk_chunk(lds + at * set, n);
    if (more) deposit(lds + (at ^ 1) * set);
    lds_barrier();
    store_chunk(lds + at * set, t0, n);
  }
#pragma unroll
  for (int r = 0; r < kRecRows; ++r)
    if (row0 + r < D && col_ok) mine[(long)(row0 + r) * DV + c] = S[r];
}

// ---------------------------------------------------------------------------
// Per (token, head): x [DV] float divided by its root mean square (eps inside the root), times
// weight[c] if given, times silu (gate_act 0) or sigmoid (gate_act 1) of gate[t][head * DV + c] if given; stored as T.  One wave a
// head: lane i adds the squares of the elements i, i + 64, ... ascending, then a butterfly.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ x, long ldx, int n_tokens,
                                                             int H, int DV, const float* __restrict__ weight,
                                                             const float* __restrict__ gate, long ldg, int gate_act,
                                                             float eps, T* __restrict__ out, long ldo) {
  const long unit = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (unit >= (long)n_tokens * H) return;
  const int t = (int)(unit / H), head = (int)(unit % H), lane = threadIdx.x & 63;
  const float* src = x + (long)t * ldx + head * DV;
  float part = 0.f;
  for (int c = lane; c < DV; c += 64) part = part + src[c] * src[c];
  const float total = wave_sum(part);
  const float scale = 1.0f / sqrtf(total / (float)DV + eps);
  for (int c = lane; c < DV; c += 64) {
    float v = src[c] * scale;
    if (weight) v = v * weight[c];
    if (gate) {
      const float z = gate[(long)t * ldg + head * DV + c];
      v = v * (gate_act == 1 ? sigmoidf_(z) : siluf_(z));
    }
    out[(long)t * ldo + head * DV + c] = from_f32<T>(v);
  }
}

// ---------------------------------------------------------------------------
// Embedding with a second table indexed by a hash of the token and the token before it:
//   out[t] = E[token[t]] * scale + B[(token[t-1] * mul_prev + token[t] * mul_cur) mod buckets],   row `buckets` of B
// for a request's first token.  The token before a portion's first one is the request's state (one int a slot):
// the workgroup of that row reads it and then leaves the portion's last token there for the next step (no other
// workgroup touches the slot).  One workgroup a token.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void embed_pair_kernel(const int* __restrict__ tokens, const int* __restrict__ tok_seq,
                                                         const int* __restrict__ tok_pos, const SeqMeta* __restrict__ seqs,
                                                         const T* __restrict__ table, const T* __restrict__ pairs,
                                                         int buckets, long mul_prev, long mul_cur, int* __restrict__ state,
                                                         long state_stride, float* __restrict__ out, int width,
                                                         long ld_out, float scale) {
  const int t = blockIdx.x;
  const SeqMeta m = seqs[tok_seq[t]];
  const bool first_row = t == m.q_off;
  const int token = tokens[t];
  int* kept = state + (long)m.table_row * state_stride;
  const int before = first_row ? kept[0] : tokens[t - 1];
  long row = buckets;
  if (tok_pos[t] > 0) {
    row = ((long)before * mul_prev + (long)token * mul_cur) % buckets;
    if (row < 0) row += buckets;     // (a slot that was never written must not lead outside the table)
  }
  const T* e_row = table + (long)token * width;
  const T* p_row = pairs + row * width;
  float* dst = out + (long)t * ld_out;
  for (int c = threadIdx.x; c < width; c += 256) dst[c] = to_f32(e_row[c]) * scale + to_f32(p_row[c]);
  if (first_row) {
    __syncthreads();                 // every thread has read the slot
    if (threadIdx.x == 0) kept[0] = tokens[m.q_off + m.q_len - 1];
  }
}

// ---------------------------------------------------------------------------
// Token shift: a sublayer's input h[t] is replaced by h[t] + (h[t-1] - h[t]) * mu, element by element, with h[t-1]
// the unshifted input of the token before (zeros for a request's first token).  n [T][ldn] float holds the unshifted
// inputs of the step; the input of the token before a portion's first one is the request's state (width floats a
// slot), which the threads of that row read and then overwrite with the portion's last input.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const float* __restrict__ n, long ldn, const float* __restrict__ mu,
                                                          const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                          const SeqMeta* __restrict__ seqs, float* __restrict__ state,
                                                          long state_stride, T* __restrict__ out, long ldo, int width) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= width) return;
  const SeqMeta m = seqs[tok_seq[t]];
  const bool first_row = t == m.q_off;
  float* kept = state + (long)m.table_row * state_stride;
  const float own = n[(long)t * ldn + c];
  float before = first_row ? kept[c] : n[(long)(t - 1) * ldn + c];
  if (tok_pos[t] == 0) before = 0.f;
  out[(long)t * ldo + c] = from_f32<T>(own + (before - own) * mu[c]);
  if (first_row) kept[c] = n[(long)(m.q_off + m.q_len - 1) * ldn + c];
}

// ---------------------------------------------------------------------------
// A step of single tokens: the residual addition that the last sublayer left, the RMS norm and the token shift in one
// launch.  h[t] += P[0][t] + P[1][t] + ... (P may be null); n = h[t] / sqrt(mean(h[t]^2) + eps) * weight;
// out[t] = n + (kept - n) * mu with `kept` the request's state (zeros at its first token), which then becomes n.
// The additions and the sum of squares follow the order of the norm's own launch (thread t adds the squares of the
// elements 1024 c + 4 t + {0..3}, c ascending; a butterfly over the wave; the waves in order), so a token's bits do
// not depend on whether it was decoded alone or stood in a prompt's portion.  width % 4 == 0.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_shift_kernel(float* __restrict__ h, const float* __restrict__ P,
                                                                int slices, int p_rows, const float* __restrict__ weight,
                                                                const float* __restrict__ mu, const int* __restrict__ tok_seq,
                                                                const int* __restrict__ tok_pos,
                                                                const SeqMeta* __restrict__ seqs, float* __restrict__ state,
                                                                long state_stride, T* __restrict__ out, int width, long ldh,
                                                                long ld_out, float eps) {
  __shared__ float wave_part[4];
  const long row = blockIdx.x;
  float* hrow = h + row * ldh;
  float part = 0.f;
  for (int base = 4 * threadIdx.x; base < width; base += 1024) {
    f32x4 total = f32x4{0.f, 0.f, 0.f, 0.f};
    const f32x4 old = *reinterpret_cast<const f32x4*>(hrow + base);
    for (int s = 0; s < slices; ++s) {
      const f32x4 p = *reinterpret_cast<const f32x4*>(P + ((long)s * p_rows + row) * width + base);
#pragma unroll
      for (int e = 0; e < 4; ++e) total[e] = total[e] + p[e];
    }
    f32x4 fresh;
#pragma unroll
    for (int e = 0; e < 4; ++e) fresh[e] = old[e] + total[e];
    if (slices > 0) *reinterpret_cast<f32x4*>(hrow + base) = fresh;
#pragma unroll
    for (int e = 0; e < 4; ++e) part = part + fresh[e] * fresh[e];
  }
  part = wave_sum(part);
  if ((threadIdx.x & 63) == 0) wave_part[threadIdx.x >> 6] = part;
  __syncthreads();
  const float total = ((wave_part[0] + wave_part[1]) + wave_part[2]) + wave_part[3];
  const float scale = 1.0f / sqrtf(total / (float)width + eps);
  float* kept = state + (long)seqs[tok_seq[row]].table_row * state_stride;
  const bool first = tok_pos[row] == 0;
  T* dst = out + row * ld_out;
  for (int base = 4 * threadIdx.x; base < width; base += 1024) {
    const f32x4 v = *reinterpret_cast<const f32x4*>(hrow + base);  // this thread wrote it above
    const f32x4 w = *reinterpret_cast<const f32x4*>(weight + base);
    const f32x4 m = *reinterpret_cast<const f32x4*>(mu + base);
    const f32x4 before = *reinterpret_cast<const f32x4*>(kept + base);
    f32x4 n;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      n[e] = (v[e] * scale) * w[e];
      dst[base + e] = from_f32<T>(n[e] + ((first ? 0.f : before[e]) - n[e]) * m[e]);
    }
    *reinterpret_cast<f32x4*>(kept + base) = n;
  }
}

}  // namespace ls

LS_DEFINE_ERROR_API

#define LS_MIXERS_LISTED(X) \
  X(ls_dyt) X(ls_glu_clamped) X(ls_softcap) X(ls_talk_qkv) X(ls_linrec) X(ls_head_norm_gate)
LS_DEFINE_LISTED_CALLS(LS_MIXERS_LISTED)

using namespace ls;

extern "C" int ls_dyt(int dtype, float* h, const float* P, int slices, int p_rows, const float* weight,
                      const float* bias, const float* alpha, void* out, const int* rows, int n_rows, int width,
                      long ldh, long ld_out, void* stream) {
  LS_REQUIRE(n_rows > 0 && width > 0 && ldh >= width && h, "dyt: bad sizes");
  LS_REQUIRE(!out || (weight && bias && alpha && ld_out >= width), "dyt: an output needs weight, bias and alpha");
  LS_REQUIRE(!P || (slices > 0 && p_rows > 0), "dyt: bad slice sums");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long p_stride = (long)p_rows * width;
  if (dtype == kF32)
    hipLaunchKernelGGL(dyt_kernel<float>, dim3(n_rows, (width + 255) / 256), dim3(256), 0, s, h, P, slices, p_stride, weight, bias, alpha,
                       (float*)out, rows, width, ldh, ld_out);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(dyt_kernel<bf16_t>, dim3(n_rows, (width + 255) / 256), dim3(256), 0, s, h, P, slices, p_stride, weight, bias, alpha,
                       (bf16_t*)out, rows, width, ldh, ld_out);
  else
    return fail("dyt: unknown dtype %d", dtype);
  return check_launch("dyt");
}

extern "C" int ls_embed_pair(int dtype, const int* tokens, const int* tok_seq, const int* tok_pos, const void* seqs,
                             const void* table, int vocab, const void* pairs, int buckets, long mul_prev, long mul_cur,
                             int* state, long state_stride, float* out, int n_tokens, int width, long ld_out, float scale,
                             void* stream) {
  LS_REQUIRE(n_tokens > 0 && vocab > 0 && width > 0 && buckets > 0 && ld_out >= width && state_stride >= 1,
             "embed_pair: bad sizes");
  LS_REQUIRE(tokens && tok_seq && tok_pos && seqs && table && pairs && state && out, "embed_pair: null operand");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (dtype == kF32)
    hipLaunchKernelGGL(embed_pair_kernel<float>, dim3(n_tokens), dim3(256), 0, s, tokens, tok_seq, tok_pos,
                       (const SeqMeta*)seqs, (const float*)table, (const float*)pairs, buckets, mul_prev, mul_cur, state,
                       state_stride, out, width, ld_out, scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(embed_pair_kernel<bf16_t>, dim3(n_tokens), dim3(256), 0, s, tokens, tok_seq, tok_pos,
                       (const SeqMeta*)seqs, (const bf16_t*)table, (const bf16_t*)pairs, buckets, mul_prev, mul_cur, state,
                       state_stride, out, width, ld_out, scale);
  else
    return fail("embed_pair: unknown dtype %d", dtype);
  return check_launch("embed_pair");
}

extern "C" int ls_token_shift(int out_dtype, const float* n, long ldn, const float* mu, const int* tok_seq,
                              const int* tok_pos, const void* seqs, float* state, long state_stride, void* out, long ldo,
                              int n_tokens, int width, void* stream) {
  LS_REQUIRE(n_tokens > 0 && width > 0 && ldn >= width && ldo >= width && state_stride >= width, "token_shift: bad sizes");
  LS_REQUIRE(n && mu && tok_seq && tok_pos && seqs && state && out, "token_shift: null operand");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)n_tokens, (unsigned)((width + 255) / 256));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(token_shift_kernel<float>, grid, dim3(256), 0, s, n, ldn, mu, tok_seq, tok_pos, (const SeqMeta*)seqs,
                       state, state_stride, (float*)out, ldo, width);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(token_shift_kernel<bf16_t>, grid, dim3(256), 0, s, n, ldn, mu, tok_seq, tok_pos,
                       (const SeqMeta*)seqs, state, state_stride, (bf16_t*)out, ldo, width);
  else
    return fail("token_shift: unknown dtype %d", out_dtype);
  return check_launch("token_shift");
}

extern "C" int ls_add_rmsnorm_shift(int out_dtype, float* h, const float* P, int slices, int p_rows, const float* weight,
                                    const float* mu, const int* tok_seq, const int* tok_pos, const void* seqs, float* state,
                                    long state_stride, void* out, int n_rows, int width, long ldh, long ld_out, float eps,
                                    void* stream) {
  LS_REQUIRE(n_rows > 0 && width > 0 && width % 4 == 0 && ldh >= width && ldh % 4 == 0 && ld_out >= width &&
                 state_stride >= width && state_stride % 4 == 0 && eps > 0.f,
             "add_rmsnorm_shift: bad sizes (rows of a multiple of four floats)");
  LS_REQUIRE(h && weight && mu && tok_seq && tok_pos && seqs && state && out, "add_rmsnorm_shift: null operand");
  LS_REQUIRE(!P ? slices == 0 : (slices > 0 && p_rows >= n_rows), "add_rmsnorm_shift: bad slice sums");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(h) % 16 == 0 && reinterpret_cast<uintptr_t>(weight) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(mu) % 16 == 0 && reinterpret_cast<uintptr_t>(state) % 16 == 0 &&
                 (!P || reinterpret_cast<uintptr_t>(P) % 16 == 0),
             "add_rmsnorm_shift: operands must be 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (out_dtype == kF32)
    hipLaunchKernelGGL(add_rmsnorm_shift_kernel<float>, dim3(n_rows), dim3(256), 0, s, h, P, slices, p_rows, weight, mu,
                       tok_seq, tok_pos, (const SeqMeta*)seqs, state, state_stride, (float*)out, width, ldh, ld_out, eps);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(add_rmsnorm_shift_kernel<bf16_t>, dim3(n_rows), dim3(256), 0, s, h, P, slices, p_rows, weight, mu,
                       tok_seq, tok_pos, (const SeqMeta*)seqs, state, state_stride, (bf16_t*)out, width, ldh, ld_out, eps);
  else
    return fail("add_rmsnorm_shift: unknown dtype %d", out_dtype);
  return check_launch("add_rmsnorm_shift");
}

extern "C" int ls_glu_clamped(int out_dtype, const float* x, long ldx, void* out, long ldo, int rows, int width,
                              float limit, float alpha, void* stream) {
  LS_REQUIRE(rows > 0 && width > 0 && ldo >= width && ldx >= 2 * width && x && out, "glu_clamped: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)(((long)rows * width + 255) / 256));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(glu_clamped_kernel<float>, grid, dim3(256), 0, s, x, ldx, (float*)out, ldo, rows, width, limit,
                       alpha);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(glu_clamped_kernel<bf16_t>, grid, dim3(256), 0, s, x, ldx, (bf16_t*)out, ldo, rows, width,
                       limit, alpha);
  else
    return fail("glu_clamped: unknown dtype %d", out_dtype);
  return check_launch("glu_clamped");
}

extern "C" int ls_softcap(float* x, long ld, int rows, int width, float cap, void* stream) {
  LS_REQUIRE(rows > 0 && width > 0 && ld >= width && x && cap > 0.f, "softcap: bad sizes");
  dim3 grid((unsigned)(((long)rows * width + 255) / 256));
  hipLaunchKernelGGL(softcap_kernel, grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream), x, ld, rows, width,
                     cap);
  return check_launch("softcap");
}

extern "C" int ls_talk_qkv(int dtype, const float* raw, long ld, int n_tokens, int H, int G, int D, int DV,
                           const float* bias, const float* cos_table, const float* sin_table, int rot,
                           int table_positions, int max_pos, const int* tok_seq, const int* tok_pos, const void* seqs,
                           const int* table, int table_stride, void* q_out, long ldq, void* k_pages, void* v_pages,
                           int page_size, int vmix_mode, const float* vmix, float* v_first, long ldv, void* stream) {
  LS_REQUIRE(n_tokens > 0 && H > 0 && G > 0 && D > 0 && DV > 0 && H % G == 0, "talk_qkv: bad head sizes");
  const long width = (long)H * D + (long)G * D + (long)G * DV;
  LS_REQUIRE(ld >= width && ldq >= (long)H * D && raw && q_out && k_pages && v_pages && table && seqs && tok_seq &&
                 tok_pos && page_size > 0 && table_stride > 0,
             "talk_qkv: bad operands");
  LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "talk_qkv: %d rotated dimensions of %d", rot, D);
  LS_REQUIRE(rot == 0 || (cos_table && sin_table && max_pos < table_positions),
             "talk_qkv: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
  LS_REQUIRE(max_pos / page_size < table_stride, "talk_qkv: position %d is beyond the block table", max_pos);
  LS_REQUIRE(vmix_mode >= 0 && vmix_mode <= 2 && (vmix_mode == 0 || (v_first && ldv >= (long)G * DV)) &&
                 (vmix_mode != 2 || vmix),
             "talk_qkv: bad value mixing");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)((n_tokens * width + 255) / 256));
#define LS_TALK_QKV(T_)                                                                                              \
  hipLaunchKernelGGL(talk_qkv_kernel<T_>, grid, dim3(256), 0, s, raw, ld, n_tokens, H, G, D, DV, bias, cos_table,    \
                     sin_table, rot, tok_seq, tok_pos, (const SeqMeta*)seqs, table, table_stride, (T_*)q_out, ldq,   \
                     (T_*)k_pages, (T_*)v_pages, page_size, vmix_mode, vmix, v_first, ldv)
  if (dtype == kF32)
    LS_TALK_QKV(float);
  else if (dtype == kBF16)
    LS_TALK_QKV(bf16_t);
  else
    return fail("talk_qkv: unknown dtype %d", dtype);
#undef LS_TALK_QKV
  return check_launch("talk_qkv");
}

extern "C" int ls_qkv_post(int dtype, const float* raw, long ld, int n_tokens, int H, int G, int D, int Dp, int DV,
                           int keys_are_values, int per_head, const float* bias, const float* q_norm, const float* k_norm, float eps,
                           const float* cos_table, const float* sin_table, int rot, int neighbours,
                           int table_positions, int max_pos, const int* tok_seq, const int* tok_pos, const void* seqs,
                           const int* table, int table_stride, void* q_out, long ldq, void* k_pages, void* v_pages,
                           int page_size, void* stream) {
  LS_REQUIRE(n_tokens > 0 && H > 0 && G > 0 && D > 0 && Dp >= D && DV > 0 && H % G == 0, "qkv_post: bad head sizes");
  LS_REQUIRE(!keys_are_values || DV == D, "qkv_post: keys of %d elements cannot be values of %d", D, DV);
  const long width = (long)H * D + (long)G * D + (keys_are_values ? 0 : (long)G * DV);
  LS_REQUIRE(ld >= width && ldq >= (long)H * Dp && raw && q_out && k_pages && v_pages && table && seqs && tok_seq &&
                 tok_pos && page_size > 0 && table_stride > 0,
             "qkv_post: bad operands");
  LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "qkv_post: %d rotated dimensions of %d", rot, D);
  LS_REQUIRE(rot == 0 || (cos_table && sin_table && max_pos < table_positions),
             "qkv_post: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
  LS_REQUIRE(max_pos / page_size < table_stride, "qkv_post: position %d is beyond the block table", max_pos);
  LS_REQUIRE((q_norm == nullptr) == (k_norm == nullptr) && (!q_norm || eps > 0.f), "qkv_post: bad norm");
  LS_REQUIRE(!per_head || (((per_head == 1 && !q_norm) || (per_head == 2 && q_norm)) && eps > 0.f && H + G <= kMaxNormedHeads),
             "qkv_post: a norm a head has no weights (1) or one weight vector for all heads (2), and takes up to %d heads",
             kMaxNormedHeads);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  // Without a norm every element stands alone: a thread an element.  With one, every workgroup of a token forms the
  // row's sums itself, so a step of many tokens gives each token one workgroup, and a few tokens are spread out.
  const unsigned all = (unsigned)(((long)(H + G) * Dp + (long)G * DV + 255) / 256);
  const unsigned pieces = !(q_norm || per_head) ? all : (n_tokens <= 64 ? all : 1u);
#define LS_QKV_POST(T_)                                                                                               \
  hipLaunchKernelGGL(qkv_post_kernel<T_>, dim3(n_tokens, pieces), dim3(256), 0, s, raw, ld, H, G, D, Dp, DV, keys_are_values, per_head, \
                     bias, q_norm, k_norm, eps, cos_table, sin_table, rot, neighbours, tok_seq, tok_pos,              \
                     (const SeqMeta*)seqs, table, table_stride, (T_*)q_out, ldq, (T_*)k_pages, (T_*)v_pages, page_size)
  if (dtype == kF32)
    LS_QKV_POST(float);
  else if (dtype == kBF16)
    LS_QKV_POST(bf16_t);
  else
    return fail("qkv_post: unknown dtype %d", dtype);
#undef LS_QKV_POST
  return check_launch("qkv_post");
}

extern "C" int ls_linrec_max_dim() { return 16 * kRecWaveRows; }

extern "C" long ls_linrec_gate_floats(int n_tokens, int H, int D) {
  const int dp = (D + kRecWaveRows - 1) / kRecWaveRows * kRecWaveRows;
  return (long)n_tokens * H * 3 * dp;
}

extern "C" int ls_linrec(int mode, const float* raw, long ld, int q_at, int ab_at, int v_at, int n_tokens, int H, int D,
                         int DV, const float* p0, const float* p1, const float* cos_table, const float* sin_table,
                         int rot, int table_positions, int max_pos, const int* tok_pos, const void* seqs, int n_seqs,
                         float* state, float* gates, float* out, long ldo, void* stream) {
  LS_REQUIRE(mode == 0 || mode == 1, "linrec: unknown mode %d", mode);
  LS_REQUIRE(n_seqs > 0 && n_tokens > 0 && H > 0 && D > 0 && DV > 0 && D <= ls_linrec_max_dim(),
             "linrec: bad sizes (heads %d, rows %d of at most %d, columns %d)", H, D, ls_linrec_max_dim(), DV);
  LS_REQUIRE(raw && seqs && state && out && p0 && gates && ldo >= (long)H * DV, "linrec: bad operands");
  LS_REQUIRE(reinterpret_cast<uintptr_t>(gates) % 16 == 0, "linrec: the gates must be 16-byte aligned");
  LS_REQUIRE(q_at >= 0 && ab_at >= 0 && v_at >= 0 && ld >= q_at + (long)H * D && ld >= ab_at + (long)H * D &&
                 ld >= v_at + (long)H * DV,
             "linrec: the projections do not fit the rows");
  if (mode == 1) {
    LS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "linrec: %d rotated dimensions of %d", rot, D);
    LS_REQUIRE(rot == 0 || (cos_table && sin_table && tok_pos && max_pos < table_positions),
               "linrec: position %d is beyond the rotation tables (%d)", max_pos, table_positions);
  }
  const int waves = (D + kRecWaveRows - 1) / kRecWaveRows;
  const int dp = waves * kRecWaveRows;
  const size_t lds =
      2 * sizeof(float) * (size_t)(3 * kRecTokens * dp + kRecTokens * kRecCols + waves * kRecTokens * kRecCols);
  if (lds > 48 * 1024) {  // (more than the default bound of dynamic LDS: say so once a size)
    static size_t allowed = 0;
    if (lds > allowed) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(linrec_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return fail("linrec: %s", hipGetErrorString(e));
      allowed = lds;
    }
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const long elements = (long)n_tokens * H * dp;
  hipLaunchKernelGGL(linrec_gates_kernel, dim3((unsigned)((elements + 255) / 256)), dim3(256), 0, s, mode, raw, ld, q_at,
                     ab_at, n_tokens, H, D, dp, p0, p1, cos_table, sin_table, mode == 1 ? rot : 0, tok_pos, gates);
  dim3 grid((unsigned)(n_seqs * H), (unsigned)((DV + kRecCols - 1) / kRecCols));
  hipLaunchKernelGGL(linrec_kernel, grid, dim3(64 * waves), lds, s, gates, raw, ld, v_at, H, D, DV,
                     (const SeqMeta*)seqs, state, out, ldo);
  return check_launch("linrec");
}

extern "C" int ls_head_norm_gate(int out_dtype, const float* x, long ldx, int n_tokens, int H, int DV,
                                 const float* weight, const float* gate, long ldg, int gate_act, float eps, void* out,
                                 long ldo, void* stream) {
  LS_REQUIRE(n_tokens > 0 && H > 0 && DV > 0 && x && out && ldx >= (long)H * DV && ldo >= (long)H * DV &&
                 (!gate || ldg >= (long)H * DV) && (gate_act == 0 || gate_act == 1),
             "head_norm_gate: bad sizes");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)(((long)n_tokens * H + 3) / 4));
  if (out_dtype == kF32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, grid, dim3(256), 0, s, x, ldx, n_tokens, H, DV, weight, gate, ldg,
                       gate_act, eps, (float*)out, ldo);
  else if (out_dtype == kBF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16_t>, grid, dim3(256), 0, s, x, ldx, n_tokens, H, DV, weight, gate,
                       ldg, gate_act, eps, (bf16_t*)out, ldo);
  else
    return fail("head_norm_gate: unknown dtype %d", out_dtype);
  return check_launch("head_norm_gate");
}
