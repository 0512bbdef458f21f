// Attention whose heads talk to each other before the softmax, over the paged cache, with a sliding
// window that keeps the first tokens, and with keys and values of different sizes:
//
//   raw_g[i, j]  = (q_g[i] . k_kv(g)[j]) * scale                  for all query heads g
//   s_h[i, j]    = sum_g talk[h, g] raw_g[i, j]                   (the heads' scores are mixed)
//   visible(i,j) = j <= i and (i - j < window or j < keep_first)  (absolute positions)
//   o_h[i]       = sum_j softmax_j(s_h[i, .])[j] v_kv(h)[j]
//
// Because every head's score at a (query, key) pair needs all heads' raw scores there, a workgroup
// takes a block of 16 query rows of one request with ALL heads, and walks the visible keys in
// tiles of 32 keys anchored at absolute positions (the kept first tiles, then the window's).  The
// library is compiled for one shape: LS_TA_HEADS query heads, LS_TA_KV_HEADS key/value heads,
// keys of LS_TA_DIM and values of LS_TA_VDIM elements, so that the heads' scores and the output
// accumulators are registers.  The heads are dealt to NW waves.  Per tile:
//   1. every wave forms the transposed raw scores S^T = K Q^T of its own heads with the MFMA atom
//      (keys are the first operand, so a lane ends with four consecutive keys of one query row:
//      the layout in which the probabilities enter the value product) and leaves them in LDS;
//   2. after a barrier it mixes all heads' raw scores into its own heads' scores (the mixing is
//      per (query, key) pair, i.e. per lane and register), masks, and runs the online softmax
//      (row statistics over the four lanes that share a query row);
//   3. O^T += V^T P^T per head with the atom (value columns are the first operand, so the lane
//      that holds a row's statistics also holds the row's accumulators).
// One workgroup that walks all visible keys of a row block would leave most of the GPU idle (a step
// of decoded tokens has one row block a request; the late row blocks of a long prompt see many
// times the keys of the early ones): a row block's tiles are dealt to several work items in
// contiguous runs, each leaves (max, sum, unnormalised output) of its run for every row, and a
// second kernel folds the runs in ascending order.
//
// A second way of talking mixes the heads' WEIGHTS, after each head's own softmax (MODE 1 and 2 of the kernel):
//
//   p_g[i, j]    = exp(raw_g[i, j]) / (exp(sink_g) + sum over visible j' of exp(raw_g[i, j']))     (the sink is optional)
//   w_h[i, j]    = sum_g talk[h, g] p_g[i, j]
//   o_h[i]       = gate_h[i] * sum_j w_h[i, j] v_kv(h)[j],    gate = sigmoid(g_h[i]) elementwise (optional)
//
// A mixed weight needs every head's finished statistics, so the keys are walked twice.  MODE 1 forms each head's raw
// scores and leaves the maximum and the sum of every (work item, row, head) in `stats`; no wave needs another's
// scores there.  MODE 2 folds the statistics of all runs of its row block (with the sink), forms the raw scores
// again, turns them into finished weights, exchanges those through LDS, mixes them and adds O^T += V^T W^T: nothing
// is rescaled afterwards, so the runs of a row block simply add up (talk_sum_kernel, which also applies the gate).
// Scores, weights, statistics and accumulators are float; products read the compute dtype T.
// Keys a request does not hold (beyond its length, pages a window has released) enter as zeros and
// are masked; their values are replaced by zeros before the product.

#include "common.h"

#ifndef LS_TA_HEADS
#error "compile with -DLS_TA_HEADS, -DLS_TA_KV_HEADS, -DLS_TA_DIM and -DLS_TA_VDIM"
#endif

namespace ls {

constexpr int H = LS_TA_HEADS, G = LS_TA_KV_HEADS, D = LS_TA_DIM, DV = LS_TA_VDIM;
static_assert(H % G == 0, "query heads must be a multiple of the key/value heads");
static_assert(D % 8 == 0, "key size must be a multiple of 8");
static_assert(DV % 4 == 0, "value size must be a multiple of 4");
static_assert(H <= 32, "the heads' raw scores of a tile must fit into LDS");
constexpr int NW = H % 8 == 0 ? 8 : (H % 4 == 0 ? 4 : (H % 2 == 0 ? 2 : 1));  // waves of a workgroup
constexpr int HPW = H / NW;                                // heads a wave owns
constexpr int VB = (DV + 15) / 16;                         // blocks of 16 value columns (the last may be partial)
constexpr int kTileKeys = 32;
constexpr int GS = H / G;  // query heads that read one key/value head
// consecutive own heads of a wave that read the same key/value head: its keys and values are loaded once for them
constexpr int SH = HPW % GS == 0 ? GS : (GS % HPW == 0 ? HPW : 1);

struct SeqMeta {
  int q_off, q_len, q_start, kv_len, table_row, reserved[3];
};

// A barrier between the waves' LDS writes and reads.  It waits for this wave's LDS operations only, not for its
// global loads: the keys of the next tile stay on their way across it (the compiler still waits for a loaded
// register before its first use).
__device__ __forceinline__ void lds_barrier() { __asm__ volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <typename T>
__device__ __forceinline__ typename Atom<T>::vec_t load_or_zero(const T* p, bool ok) {
  typedef typename Atom<T>::vec_t vec_t;
  // (an address that is always valid, the value chosen afterwards: the loads of a tile can be in flight together)
  vec_t v = *reinterpret_cast<const vec_t*>(p);
  return ok ? v : Atom<T>::zero();
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

constexpr int kFoldAtOnce = 16;  // runs whose statistics the second pass requests together (the host deals a row block to at most as many)
constexpr int kStatRows = 16;   // rows of a work item in `stats` (also for decoded tokens, which use row 0)

// MODE 0: the heads' scores are mixed before the softmax.  MODE 1 / 2: the two passes that mix the heads' weights.
template <typename T, int MODE>
__global__ __launch_bounds__(64 * NW) void talk_attention_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int page_size,
    const int* __restrict__ table, int table_stride, const SeqMeta* __restrict__ seqs, const int* __restrict__ blocks,
    const float* __restrict__ talk, float scale, int window, int keep_first, T* __restrict__ out, long ldo,
    float* __restrict__ part, int part_rows, const float* __restrict__ sink, float* __restrict__ stats,
    const float* __restrict__ gate, long ldg) {
  constexpr int VEC = Atom<T>::VEC, KC = Atom<T>::KCHUNK;
  constexpr int KCH = (D + KC - 1) / KC;  // chunks of a key (lanes beyond D in the last one bring zeros)
  __shared__ f32x4 raw_s[H][2][64];  // [head][half of the tile][lane]: the lane's four keys of that half
  __shared__ float talk_s[H * H];
  // a work item: request of the step, block of 16 of its rows, which run of the tiles, of how many runs
  const int seq = blocks[4 * blockIdx.x], rb = blocks[4 * blockIdx.x + 1];
  const int run = blocks[4 * blockIdx.x + 2], n_runs = max(1, blocks[4 * blockIdx.x + 3]);
  const SeqMeta m = seqs[seq];
  const int row0 = rb * 16;
  if (row0 >= m.q_len) return;
  const int nrows = min(16, m.q_len - row0);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4;
  for (int i = threadIdx.x; i < H * H; i += 64 * NW) talk_s[i] = talk[i];
  const int p_first = m.q_start + row0, p_last = p_first + nrows - 1;
  const bool row_ok = l16 < nrows;
  const int my_pos = p_first + l16;
  const int* my_table = table + (long)m.table_row * table_stride;
  const T* q_row = q + (long)(m.q_off + row0 + (row_ok ? l16 : 0)) * ldq;

  float m_run[HPW], l_run[HPW];
  f32x4 acc[HPW][VB];
#pragma unroll
  for (int x = 0; x < HPW; ++x) {
    m_run[x] = kNegSentinel;
    l_run[x] = 0.f;
#pragma unroll
    for (int b = 0; b < VB; ++b) acc[x][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int lo_tile = max(0, p_first - window + 1) / kTileKeys;
  const int hi_tile = p_last / kTileKeys;
  const int kept_tiles = min((keep_first + kTileKeys - 1) / kTileKeys, lo_tile);
  const int n_tiles = kept_tiles + (hi_tile - lo_tile + 1);
  __syncthreads();

  const int per_run = (n_tiles + n_runs - 1) / n_runs;
  const int step_end = min(n_tiles, (run + 1) * per_run);

  // MODE 2: every own head's finished maximum and the inverse of its finished sum, folded over the runs of this row
  // block in ascending order (their work items follow each other), with the sink
  float m_all[HPW], inv_all[HPW];
  if constexpr (MODE == 2) {
#pragma unroll
    for (int x = 0; x < HPW; ++x) {
      const int h = w * HPW + x;
      const float* st = stats + (((long)(blockIdx.x - run) * kStatRows + (row_ok ? l16 : 0)) * H + h) * 2;
      const long stride = (long)kStatRows * H * 2;
      // (the statistics of up to kFoldAtOnce runs are requested together: one wait instead of one a run)
      float mk[kFoldAtOnce], lk[kFoldAtOnce];
#pragma unroll
      for (int k = 0; k < kFoldAtOnce; ++k) {
        const long at = (long)min(k, n_runs - 1) * stride;
        mk[k] = st[at];
        lk[k] = st[at + 1];
      }
      float top = sink ? sink[h] : kNegSentinel;
#pragma unroll
      for (int k = 0; k < kFoldAtOnce; ++k) top = fmaxf(top, k < n_runs ? mk[k] : kNegSentinel);
      for (int k = kFoldAtOnce; k < n_runs; ++k) top = fmaxf(top, st[k * stride]);
      float total = 0.f;
#pragma unroll
      for (int k = 0; k < kFoldAtOnce; ++k) total = total + (k < n_runs ? lk[k] * softmax_exp<T>(mk[k] - top) : 0.f);
      for (int k = kFoldAtOnce; k < n_runs; ++k) total = total + st[k * stride + 1] * softmax_exp<T>(st[k * stride] - top);
      if (sink) total = total + softmax_exp<T>(sink[h] - top);
      m_all[x] = top;
      inv_all[x] = row_ok && total > 0.f ? 1.0f / total : 0.f;
    }
  }

  // A tile's keys are requested while the tile before it is worked on: its addresses (page and slot of the
  // lane's key of each half as a row of K, and of its four keys as columns of V^T) and the key vectors of the
  // key/value heads the wave reads.
  struct Ahead {
    long k_at[2], v_at[2];
    bool k_ok[2], v_ok[2][4];
    typename Atom<T>::vec_t kv[2][HPW / SH][KCH];
  };
  auto request = [&](int step, Ahead& t) LS_INLINED {
    const int tile = step < kept_tiles ? step : lo_tile + (step - kept_tiles);
    const int key0 = tile * kTileKeys;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int key = key0 + 16 * half + l16;
      const int page = key <= p_last ? my_table[key / page_size] : -1;
      t.k_ok[half] = page >= 0;
      t.k_at[half] = ((long)(page >= 0 ? page : 0) * G) * page_size + (page >= 0 ? key % page_size : 0);
      const int key4 = key0 + 16 * half + 4 * quad;
      const int page4 = key4 <= p_last ? my_table[key4 / page_size] : -1;
      t.v_at[half] = ((long)(page4 >= 0 ? page4 : 0) * G * DV) * page_size + (page4 >= 0 ? key4 % page_size : 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) t.v_ok[half][i] = page4 >= 0 && key4 + i <= p_last;
#pragma unroll
      for (int xg = 0; xg < HPW / SH; ++xg) {
        const int g = (w * HPW + xg * SH) / GS;
        const T* k_row = k_pages + (t.k_at[half] + (long)g * page_size) * D;
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
          const bool in = c * KC + VEC * quad + VEC <= D;
          t.kv[half][xg][c] = load_or_zero<T>(k_row + (in ? c * KC + VEC * quad : 0), t.k_ok[half] && in);
        }
      }
    }
  };

  // The queries of the wave's heads do not change from tile to tile: they stay in registers where that takes at
  // most 32 of them (else they are read again for every tile, through the L1 cache).
  constexpr bool kKeepQ = HPW * KCH * (int)(sizeof(typename Atom<T>::vec_t) / 4) <= 32;
  typename Atom<T>::vec_t qv[kKeepQ ? HPW : 1][kKeepQ ? KCH : 1];
  if constexpr (kKeepQ) {
#pragma unroll
    for (int x = 0; x < HPW; ++x)
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        const bool in = c * KC + VEC * quad + VEC <= D;
        qv[x][c] = load_or_zero<T>(q_row + (w * HPW + x) * D + (in ? c * KC + VEC * quad : 0), row_ok && in);
      }
  }

  Ahead now;
  if (run * per_run < step_end) request(run * per_run, now);
  for (int step = run * per_run; step < step_end; ++step) {
    const int tile = step < kept_tiles ? step : lo_tile + (step - kept_tiles);
    const int key0 = tile * kTileKeys;
    long v_at[2];
    bool v_ok[2][4];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      v_at[half] = now.v_at[half];
#pragma unroll
      for (int i = 0; i < 4; ++i) v_ok[half][i] = now.v_ok[half][i];
    }
    // -- 1. transposed raw scores of the wave's own heads ------------------------------------
    f32x4 own[MODE == 1 ? HPW : 1][2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int xg = 0; xg < HPW / SH; ++xg) {
#pragma unroll
        for (int xs = 0; xs < SH; ++xs) {
          const int h = w * HPW + xg * SH + xs;
          f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KCH; ++c) {
            if constexpr (kKeepQ) {
              Atom<T>::mma(s, now.kv[half][xg][c], qv[xg * SH + xs][c]);
            } else {
              const bool in = c * KC + VEC * quad + VEC <= D;
              Atom<T>::mma(s, now.kv[half][xg][c],
                           load_or_zero<T>(q_row + h * D + (in ? c * KC + VEC * quad : 0), row_ok && in));
            }
          }
          if constexpr (MODE == 0) {
            raw_s[h][half][lane] = f32x4{s[0] * scale, s[1] * scale, s[2] * scale, s[3] * scale};
          } else if constexpr (MODE == 1) {
            own[xg * SH + xs][half] = f32x4{s[0] * scale, s[1] * scale, s[2] * scale, s[3] * scale};
          } else {   // the head's finished weights (of keys that the row does not see as well: the mask follows the mixing)
            f32x4 p;
#pragma unroll
            for (int i = 0; i < 4; ++i) p[i] = softmax_exp<T>(s[i] * scale - m_all[xg * SH + xs]) * inv_all[xg * SH + xs];
            raw_s[h][half][lane] = p;
          }
        }
      }
    }
    if (step + 1 < step_end) request(step + 1, now);  // (the products above have taken this tile's keys)
    // what a row sees of this tile
    bool see[2][4];
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + 16 * half + 4 * quad + i;
        see[half][i] = row_ok && key <= my_pos && (my_pos - key < window || key < keep_first);
      }
    if constexpr (MODE == 1) {
      // the statistics of the own heads' raw scores; nothing is exchanged and no value is read
#pragma unroll
      for (int x = 0; x < HPW; ++x) {
        float top = kNegSentinel;
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) top = fmaxf(top, see[half][i] ? own[x][half][i] : kNegSentinel);
        top = quad16_max(top);
        const float m_new = fmaxf(m_run[x], top);
        float sum = 0.f;
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) sum = sum + (see[half][i] ? softmax_exp<T>(own[x][half][i] - m_new) : 0.f);
        sum = quad16_sum(sum);
        l_run[x] = l_run[x] * softmax_exp<T>(m_run[x] - m_new) + sum;
        m_run[x] = m_new;
      }
      continue;
    }
    lds_barrier();
    // -- 2. mix, mask, online softmax ---------------------------------------------------------------
    // every head's raw scores are read once and go into all of the wave's own heads
    float mixed[HPW][2][4];
#pragma unroll
    for (int x = 0; x < HPW; ++x)
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 4; ++i) mixed[x][half][i] = 0.f;
    // (the second pass of mixed weights holds more than the first way of mixing: it reads four heads at a time, so
    // that the reads of all heads are not in registers together)
    constexpr int OU = (MODE == 2 && H > 4) ? 4 : H;
#pragma unroll 1
    for (int o0 = 0; o0 < H; o0 += OU) {
#pragma unroll
      for (int oo = 0; oo < OU; ++oo) {
        const int o = o0 + oo;
        if (o >= H) break;
        const f32x4 r0 = raw_s[o][0][lane], r1 = raw_s[o][1][lane];
#pragma unroll
        for (int x = 0; x < HPW; ++x) {
          const float weight = talk_s[(w * HPW + x) * H + o];
#pragma unroll
          for (int i = 0; i < 4; ++i) {  // (fused multiply-adds, written as such: this loop is the kernel's vector work)
            mixed[x][0][i] = fmaf(weight, r0[i], mixed[x][0][i]);
            mixed[x][1][i] = fmaf(weight, r1[i], mixed[x][1][i]);
          }
        }
      }
    }
    float shrink[HPW];
#pragma unroll
    for (int x = 0; x < HPW; ++x) {     // the scores become the weights, in place
      if constexpr (MODE == 2) {        // (they are weights already, and finished; a weight of a key that is not seen
        shrink[x] = 1.0f;               //  may be anything, also no number: it is replaced, never multiplied)
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) mixed[x][half][i] = see[half][i] ? mixed[x][half][i] : 0.f;
        continue;
      }
      float top = kNegSentinel;
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 4; ++i) top = fmaxf(top, see[half][i] ? mixed[x][half][i] : kNegSentinel);
      top = quad16_max(top);
      const float m_new = fmaxf(m_run[x], top);
      shrink[x] = softmax_exp<T>(m_run[x] - m_new);
      float sum = 0.f;
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          mixed[x][half][i] = see[half][i] ? softmax_exp<T>(mixed[x][half][i] - m_new) : 0.f;
          sum = sum + mixed[x][half][i];
        }
      sum = quad16_sum(sum);
      l_run[x] = l_run[x] * shrink[x] + sum;
      m_run[x] = m_new;
    }
    // -- 3. values: column 16 b + l16 of V^T, keys 4 quad .. 4 quad + 3 of each half ----------------
    // Two things are the same for every lane of most tiles and are asked of the whole wave once: whether all
    // keys of the tile are held (then no value has to be replaced by a zero) and whether no row's maximum moved
    // (then no accumulator has to be scaled).
    bool held = true, moved = false;
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int i = 0; i < 4; ++i) held = held && v_ok[half][i];
#pragma unroll
    for (int x = 0; x < HPW; ++x) moved = moved || shrink[x] != 1.0f;
    const bool all_held = __all(held) != 0 && DV % 16 == 0;
    const bool none_moved = __all(!moved) != 0;
    if (!none_moved) {
#pragma unroll
      for (int x = 0; x < HPW; ++x)
#pragma unroll
        for (int b = 0; b < VB; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[x][b][i] = acc[x][b][i] * shrink[x];
    }
    // the weights as the second operand, once a head
    typename Atom<T>::vec_t pb[HPW][sizeof(T) == 2 ? 1 : 2];
#pragma unroll
    for (int x = 0; x < HPW; ++x) {
      if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pb[x][0][i] = (bf16_t)mixed[x][0][i];
          pb[x][0][4 + i] = (bf16_t)mixed[x][1][i];
        }
      } else {
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) pb[x][half][i] = mixed[x][half][i];
      }
    }
#pragma unroll
    for (int xg = 0; xg < HPW / SH; ++xg) {
      const int g = (w * HPW + xg * SH) / GS;
#pragma unroll
      for (int b = 0; b < VB; ++b) {
        const bool col_ok = 16 * b + l16 < DV;
        const long column = ((long)g * DV + (col_ok ? 16 * b + l16 : 0)) * page_size;
        if constexpr (sizeof(T) == 2) {
          const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(v_pages + v_at[0] + column);
          const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(v_pages + v_at[1] + column);
          bf16x8 a;
          if (all_held) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              a[i] = v0[i];
              a[4 + i] = v1[i];
            }
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              a[i] = (v_ok[0][i] && col_ok) ? v0[i] : (bf16_t)0.f;
              a[4 + i] = (v_ok[1][i] && col_ok) ? v1[i] : (bf16_t)0.f;
            }
          }
#pragma unroll
          for (int xs = 0; xs < SH; ++xs) Atom<T>::mma(acc[xg * SH + xs][b], a, pb[xg * SH + xs][0]);
        } else {
          f32x4 a[2];
#pragma unroll
          for (int half = 0; half < 2; ++half) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(v_pages + v_at[half] + column);
            if (all_held) {
              a[half] = v;
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i) a[half][i] = (v_ok[half][i] && col_ok) ? v[i] : 0.f;
            }
          }
#pragma unroll
          for (int xs = 0; xs < SH; ++xs)
#pragma unroll
            for (int half = 0; half < 2; ++half) Atom<T>::mma(acc[xg * SH + xs][b], a[half], pb[xg * SH + xs][half]);
        }
      }
    }
    lds_barrier();
  }
  if (!row_ok) return;
  if constexpr (MODE == 1) {
    if (quad == 0) {
#pragma unroll
      for (int x = 0; x < HPW; ++x) {
        float* st = stats + (((long)blockIdx.x * kStatRows + l16) * H + w * HPW + x) * 2;
        st[0] = m_run[x];
        st[1] = l_run[x];
      }
    }
    return;
  }
  if (n_runs > 1) {
    // [item][row][head][DV + 2]: the unnormalised output, then max and sum (part_rows 1: decoded tokens, row 0 only)
    if (l16 >= part_rows) return;
#pragma unroll
    for (int x = 0; x < HPW; ++x) {
      float* dst = part + (((long)blockIdx.x * part_rows + l16) * H + w * HPW + x) * (DV + 2);
#pragma unroll
      for (int b = 0; b < VB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (16 * b + 4 * quad + i < DV) dst[16 * b + 4 * quad + i] = acc[x][b][i];
      if (MODE == 0 && quad == 0) {
        dst[DV] = m_run[x];
        dst[DV + 1] = l_run[x];
      }
    }
    return;
  }
  T* dst = out + (long)(m.q_off + row0 + l16) * ldo;
#pragma unroll
  for (int x = 0; x < HPW; ++x) {
    const int h = w * HPW + x;
    const float inv = MODE == 2 ? 1.0f : 1.0f / l_run[x];
    const float* g_row = (MODE == 2 && gate) ? gate + (long)(m.q_off + row0 + l16) * ldg + h * DV : nullptr;
#pragma unroll
    for (int b = 0; b < VB; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = 16 * b + 4 * quad + i;
        if (c < DV) {
          float v = acc[x][b][i] * inv;
          if (g_row) v = v * sigmoid_f(g_row[c]);
          dst[h * DV + c] = from_f32<T>(v);
        }
      }
  }
}

// The runs of a row block whose weights were mixed after the softmax: their outputs add up, in ascending order, and
// the gate multiplies the sum.  One workgroup a (fold item, head, row), as talk_combine_kernel.
template <typename T>
__global__ __launch_bounds__(64) void talk_sum_kernel(const float* __restrict__ part, int part_rows,
                                                      const int* __restrict__ folds, const float* __restrict__ gate,
                                                      long ldg, T* __restrict__ out, long ldo) {
  const int first = folds[4 * blockIdx.x], n_runs = folds[4 * blockIdx.x + 1];
  const int row0 = folds[4 * blockIdx.x + 2], rows = folds[4 * blockIdx.x + 3];
  const int h = blockIdx.y;
  const long stride = (long)part_rows * H * (DV + 2);  // from a run to the next
  for (int r = blockIdx.z; r < rows; r += gridDim.z) {
    const float* mine = part + (((long)first * part_rows + r) * H + h) * (DV + 2);
    for (int c = threadIdx.x; c < DV; c += 64) {
      float sum = 0.f;
      for (int k = 0; k < n_runs; ++k) sum = sum + mine[k * stride + c];
      if (gate) sum = sum * sigmoid_f(gate[(long)(row0 + r) * ldg + (long)h * DV + c]);
      out[(long)(row0 + r) * ldo + h * DV + c] = from_f32<T>(sum);
    }
  }
}

// Fold the runs of row blocks: a fold item (first work item, runs, first packed row, rows) names the work items
// first .. first + runs - 1 of one row block, whose partial results are folded in ascending order for each of its
// rows.  One workgroup a (fold item, head, row).
template <typename T>
__global__ __launch_bounds__(64) void talk_combine_kernel(const float* __restrict__ part, int part_rows,
                                                          const int* __restrict__ folds, T* __restrict__ out,
                                                          long ldo) {
  const int first = folds[4 * blockIdx.x], n_runs = folds[4 * blockIdx.x + 1];
  const int row0 = folds[4 * blockIdx.x + 2], rows = folds[4 * blockIdx.x + 3];
  const int h = blockIdx.y;
  const long stride = (long)part_rows * H * (DV + 2);  // from a run to the next
  for (int r = blockIdx.z; r < rows; r += gridDim.z) {
    const float* mine = part + (((long)first * part_rows + r) * H + h) * (DV + 2);
    float top = kNegSentinel;
    for (int k = 0; k < n_runs; ++k) top = fmaxf(top, mine[k * stride + DV]);
    float total = 0.f;
    for (int k = 0; k < n_runs; ++k) total = total + mine[k * stride + DV + 1] * softmax_exp<T>(mine[k * stride + DV] - top);
    const float inv = 1.0f / total;
    for (int c = threadIdx.x; c < DV; c += 64) {
      float sum = 0.f;
      for (int k = 0; k < n_runs; ++k) sum = sum + mine[k * stride + c] * softmax_exp<T>(mine[k * stride + DV] - top);
      out[(long)(row0 + r) * ldo + h * DV + c] = from_f32<T>(sum * inv);
    }
  }
}

}  // namespace ls

LS_DEFINE_ERROR_API

using namespace ls;

extern "C" int ls_talk_heads() { return H; }
extern "C" int ls_talk_kv_heads() { return G; }
extern "C" int ls_talk_dim() { return D; }
extern "C" int ls_talk_vdim() { return DV; }

// q [T][ldq] (rotated queries, H heads of D); key pages [pages][G][page_size][D], value pages
// [pages][G][DV][page_size]; table [slots][table_stride]; seqs: the step's requests; blocks: n_blocks work items
// of four ints (request of the step, block of 16 of its rows, run, runs); talk [H][H] float; out [T][ldo] (H heads
// of DV).  Work items with runs > 1 leave their results in part (n_blocks * part_rows * H * (DV + 2) floats;
// part_rows 16, or 1 for a step of single decoded tokens) and the n_folds fold items of four ints (first work
// item, runs, first packed row, rows) say which to fold into which rows of out in a second launch.
extern "C" int ls_talk_attention(int dtype, const void* q, long ldq, const void* k_pages, const void* v_pages,
                                 int page_size, const int* table, int table_stride, const void* seqs,
                                 const int* blocks, int n_blocks, const float* talk, float scale, int window,
                                 int keep_first, void* out, long ldo, const int* folds, int n_folds, float* part,
                                 int part_rows, int mix_weights, const float* sink, float* stats, const float* gate,
                                 long ldg, void* stream) {
  // mix_weights: the heads' weights are mixed after each head's own softmax (two passes; stats: n_blocks * 16 * H * 2
  // floats of scratch), with an optional sink [H] in every head's softmax and an optional gate (float [T][ldg], H
  // heads of DV logits) on the output; else the scores are mixed before the softmax, and sink and gate must be null.
  LS_REQUIRE(mix_weights ? stats != nullptr : (!sink && !gate), "talk_attention: a sink and a gate come with mixed weights");
  LS_REQUIRE(!gate || ldg >= (long)H * DV, "talk_attention: the gate's rows are too short");
  LS_REQUIRE(n_folds >= 0 && (n_folds == 0 || (part && folds && (part_rows == 1 || part_rows == 16))),
             "talk_attention: %d fold items need partial results of 1 or 16 rows", n_folds);
  LS_REQUIRE(n_blocks > 0 && q && k_pages && v_pages && table && seqs && blocks && talk && out, "talk_attention: null operand");
  LS_REQUIRE(ldq >= (long)H * D && ldo >= (long)H * DV, "talk_attention: rows are too short");
  LS_REQUIRE(page_size >= 4 && page_size % 4 == 0 && table_stride > 0, "talk_attention: page size %d", page_size);
  LS_REQUIRE(window > 0 && keep_first >= 0, "talk_attention: window %d, kept first tokens %d", window, keep_first);
  LS_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(k_pages) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(v_pages) % 16 == 0,
             "talk_attention: operands must be 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
#define LS_TALK_PASS(T_, MODE_)                                                                                        \
  hipLaunchKernelGGL((talk_attention_kernel<T_, MODE_>), dim3(n_blocks), dim3(64 * NW), 0, s, (const T_*)q, ldq,       \
                     (const T_*)k_pages, (const T_*)v_pages, page_size, table, table_stride, (const SeqMeta*)seqs,     \
                     blocks, talk, scale, window, keep_first, (T_*)out, ldo, part, part_rows, sink, stats, gate, ldg)
#define LS_TALK(T_)                                                                                                    \
  do {                                                                                                                 \
    if (mix_weights) {                                                                                                 \
      LS_TALK_PASS(T_, 1);                                                                                             \
      LS_TALK_PASS(T_, 2);                                                                                             \
      if (n_folds > 0)                                                                                                 \
        hipLaunchKernelGGL(talk_sum_kernel<T_>, dim3(n_folds, H, part_rows), dim3(64), 0, s, part, part_rows, folds,   \
                           gate, ldg, (T_*)out, ldo);                                                                  \
    } else {                                                                                                           \
      LS_TALK_PASS(T_, 0);                                                                                             \
      if (n_folds > 0)                                                                                                 \
        hipLaunchKernelGGL(talk_combine_kernel<T_>, dim3(n_folds, H, part_rows), dim3(64), 0, s, part, part_rows,      \
                           folds, (T_*)out, ldo);                                                                      \
    }                                                                                                                  \
  } while (0)
  if (dtype == kF32) {
    LS_REQUIRE(ldq % 4 == 0, "talk_attention: query rows must be 16-byte aligned");
    LS_TALK(float);
  } else if (dtype == kBF16) {
    LS_REQUIRE(ldq % 8 == 0, "talk_attention: query rows must be 16-byte aligned");
    LS_TALK(bf16_t);
  } else {
    return fail("talk_attention: unknown dtype %d", dtype);
  }
#undef LS_TALK
#undef LS_TALK_PASS
  return check_launch("talk_attention");
}
