// Grouped-query attention over the paged cache whose softmax has a sink, with a choice of what a query
// sees and of what is added to its scores:
//
//   s_h[i, j]    = (q_h[i] . k_kv(h)[j]) * scale + bias_h[min(i - j, n_dist - 1)]   (bias optional)
//   visible(i,j) = lo(i) <= j <= i,   lo(i) = max(window ? i - window + 1 : 0, chunk ? floor(i / chunk) chunk : 0),
//                  or j < keep_first (the first tokens stay visible when a window has passed them; their tiles are
//                  walked before the window's)
//   p_h[i, j]    = exp(s_h[i, j]) / (exp(sink_h) + sum over visible j' of exp(s_h[i, j']))  (without a sink: no term)
//   o_h[i]       = gate_h[i] * sum_j p_h[i, j] v_kv(h)[j],   gate = sigmoid(g_h[i]) elementwise (optional)
//
// i and j are absolute positions; the sink is a score that has no key and no value, so the weights of a
// row add up to less than one.  The bias is a table by distance, one row a head, whose last entry serves
// every larger distance.
//
// The library is compiled for one key size LS_SA_DIM and one value size LS_SA_VDIM.  A wave owns 16 RT
// rows of the 16x16 MFMA atom and walks the visible keys in tiles of 32 anchored at absolute positions.
// Keys are the first operand of the score product (S^T = K Q^T: a lane ends with four consecutive keys of
// one query row, which is how the weights enter the value product) and value columns the first operand of
// O^T += V^T P^T (the lane that holds a row's statistics also holds its accumulators).  A key or value
// fragment is loaded once and multiplied with all RT row tiles.  Two shapes of work:
//   prompt portions  a workgroup takes (request, block of 16 RT rows, key/value head); its waves are the
//                    query heads that read this key/value head, so their loads of K and V meet in the
//                    CU's cache;
//   decoded tokens   a wave takes (request, key/value head) and the MFMA rows are the query heads of the
//                    group (up to 16 a wave).
// The tiles of a row block are dealt to several work items in contiguous runs where that fills the GPU;
// each leaves (unnormalised output, max, sum) of its run for every row and a second kernel folds the
// runs in ascending order, adds the sink and applies the gate.
// Scores, weights, statistics and accumulators are float; products read the compute dtype T.  Keys a
// request does not hold (beyond its length, pages that a window or a chunk's end has released) enter as
// zeros and are masked; their values are replaced by zeros before the product.

#include "common.h"

#include <type_traits>

#ifndef LS_SA_DIM
#error "compile with -DLS_SA_DIM and -DLS_SA_VDIM"
#endif

namespace ls {

constexpr int D = LS_SA_DIM, DV = LS_SA_VDIM;
static_assert(D % 8 == 0 && D <= 640, "key size must be a multiple of 8 up to 640");
static_assert(DV >= 1 && DV <= 512, "value size must be at most 512");
constexpr int VB = (DV + 15) / 16;  // blocks of 16 value columns (the last may be partial)
constexpr int kTileKeys = 32;
constexpr int kMaxWaves = 4;        // query heads of a key/value head that share a workgroup

struct SeqMeta {
  int q_off, q_len, q_start, kv_len, table_row, reserved[3];
};

template <typename T>
__device__ __forceinline__ typename Atom<T>::vec_t load_or_zero(const T* p, bool ok) {
  typedef typename Atom<T>::vec_t vec_t;
  // (an address that is always valid, the value chosen afterwards: the loads of a tile can be in flight together)
  vec_t v = *reinterpret_cast<const vec_t*>(p);
  return ok ? v : Atom<T>::zero();
}

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// First key that a query at position p sees.
__device__ __forceinline__ int first_seen(int p, int window, int chunk) {
  int lo = 0;
  if (window > 0) lo = max(lo, p - window + 1);
  if (chunk > 0) lo = max(lo, p / chunk * chunk);
  return lo;
}

// DEC: a step of single decoded tokens (the rows of a tile are the heads of a key/value group).
template <typename T, int RT, bool DEC>
__global__ __launch_bounds__(64 * (DEC ? 1 : kMaxWaves)) void sink_attention_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int page_size,
    const int* __restrict__ table, int table_stride, const SeqMeta* __restrict__ seqs, const int* __restrict__ items,
    int H, int G, float scale, int window, int chunk, int keep_first, const float* __restrict__ sink,
    const float* __restrict__ dist_bias, int n_dist, const float* __restrict__ gate, long ldg, T* __restrict__ out,
    long ldo, float* __restrict__ part, int part_rows) {
  constexpr int VEC = Atom<T>::VEC, KC = Atom<T>::KCHUNK;
  constexpr int KCH = (D + KC - 1) / KC;  // chunks of a key (lanes beyond D in the last one bring zeros)
  constexpr int ROWS = 16 * RT;
  // a work item: request of the step, block of ROWS of its rows, which run of the tiles, of how many runs
  const int seq = items[4 * blockIdx.x], rb = items[4 * blockIdx.x + 1];
  const int run = items[4 * blockIdx.x + 2], n_runs = max(1, items[4 * blockIdx.x + 3]);
  const SeqMeta m = seqs[seq];
  const int GS = H / G, g = blockIdx.y;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4;
  const int row0 = DEC ? 0 : rb * ROWS;
  if (row0 >= m.q_len) return;
  const int nrows = DEC ? 1 : min(ROWS, m.q_len - row0);
  // the head of a lane's row: one head a wave for prompt portions, a head a row for decoded tokens
  const int in_group = DEC ? blockIdx.z * 16 + l16 : blockIdx.z * kMaxWaves + w;
  if (!DEC && in_group >= GS) return;   // (the whole wave; no barrier follows)
  const bool head_ok = in_group < GS;
  const int my_head = g * GS + (head_ok ? in_group : 0);
  const int p_first = m.q_start + row0, p_last = p_first + nrows - 1;
  const int* my_table = table + (long)m.table_row * table_stride;
  const int page_shift = __ffs(page_size) - 1, page_mask = page_size - 1;   // (pages hold a power of two of keys)

  bool row_ok[RT];
  int my_pos[RT], my_lo[RT];
  const T* q_row[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int row = DEC ? 0 : 16 * r + l16;
    row_ok[r] = DEC ? head_ok : row < nrows;
    my_pos[r] = p_first + (row_ok[r] ? row : 0);
    my_lo[r] = first_seen(my_pos[r], window, chunk);
    q_row[r] = q + (long)(m.q_off + row0 + (row_ok[r] ? row : 0)) * ldq + (long)my_head * D;
  }
  const float* my_bias = dist_bias ? dist_bias + (long)my_head * n_dist : nullptr;

  float m_run[RT], l_run[RT];
  f32x4 acc[RT][VB];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    m_run[r] = kNegSentinel;
    l_run[r] = 0.f;
#pragma unroll
    for (int b = 0; b < VB; ++b) acc[r][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int lo_last = first_seen(p_last, window, chunk);   // (no row of the block begins to see later than this)
  const int lo_tile = first_seen(p_first, window, chunk) / kTileKeys;
  const int hi_tile = p_last / kTileKeys;
  const int kept_tiles = min((keep_first + kTileKeys - 1) / kTileKeys, lo_tile);   // tiles of kept first tokens below the window's
  const int n_tiles = kept_tiles + hi_tile - lo_tile + 1;
  auto tile_at = [&](int step) LS_INLINED { return step < kept_tiles ? step : lo_tile + (step - kept_tiles); };
  const int per_run = (n_tiles + n_runs - 1) / n_runs;
  const int step_end = min(n_tiles, (run + 1) * per_run);

  // A tile's keys are requested while the tile before it is worked on: its addresses (page and slot of the
  // lane's key of each half as a row of K, and of its four keys as columns of V^T), the key vectors and the values.
  typedef typename std::conditional<sizeof(T) == 2, bf16x4, f32x4>::type v4_t;   // four keys of one value column
  // (the values travel with the keys where the registers allow it: not with four row tiles of wide values)
  constexpr bool kAheadV = RT * VB <= 16;
  struct Ahead {
    long v_at[2];
    bool v_ok[2][4];
    typename Atom<T>::vec_t kv[2][KCH];
    v4_t vv[2][kAheadV ? VB : 1];
  };
  auto request = [&](int step, Ahead& t) LS_INLINED {
    const int key0 = tile_at(step) * kTileKeys;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int key = key0 + 16 * half + l16;
      const int page = key <= p_last ? my_table[key >> page_shift] : -1;
      const bool k_ok = page >= 0;
      const long k_at = (((long)(k_ok ? page : 0) * G + g) << page_shift) + (k_ok ? key & page_mask : 0);
      const int key4 = key0 + 16 * half + 4 * quad;
      const int page4 = key4 <= p_last ? my_table[key4 >> page_shift] : -1;
      const long v_at = ((((long)(page4 >= 0 ? page4 : 0) * G + g) * DV) << page_shift) + (page4 >= 0 ? key4 & page_mask : 0);
      t.v_at[half] = v_at;
#pragma unroll
      for (int i = 0; i < 4; ++i) t.v_ok[half][i] = page4 >= 0 && key4 + i <= p_last;
      const T* k_row = k_pages + k_at * D;
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        const bool in = c * KC + VEC * quad + VEC <= D;
        t.kv[half][c] = load_or_zero<T>(k_row + (in ? c * KC + VEC * quad : 0), k_ok && in);
      }
      if constexpr (kAheadV) {   // (the values too: they are on their way while the scores are formed)
#pragma unroll
        for (int b = 0; b < VB; ++b) {
          const long column = (long)(16 * b + l16 < DV ? 16 * b + l16 : 0) << page_shift;
          t.vv[half][b] = *reinterpret_cast<const v4_t*>(v_pages + v_at + column);
        }
      }
    }
  };

  // The queries do not change from tile to tile: they stay in registers where that takes at most 64 of them.
  constexpr bool kKeepQ = RT * KCH * (int)(sizeof(typename Atom<T>::vec_t) / 4) <= 64;
  typename Atom<T>::vec_t qv[kKeepQ ? RT : 1][kKeepQ ? KCH : 1];
  if constexpr (kKeepQ) {
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int c = 0; c < KCH; ++c) {
        const bool in = c * KC + VEC * quad + VEC <= D;
        qv[r][c] = load_or_zero<T>(q_row[r] + (in ? c * KC + VEC * quad : 0), row_ok[r] && in);
      }
  }

  Ahead now;
  if (run * per_run < step_end) request(run * per_run, now);
  for (int step = run * per_run; step < step_end; ++step) {
    const int key0 = tile_at(step) * kTileKeys;
    bool v_ok[2][4];
    long v_at[2];
    v4_t vv[2][kAheadV ? VB : 1];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      v_at[half] = now.v_at[half];
#pragma unroll
      for (int i = 0; i < 4; ++i) v_ok[half][i] = now.v_ok[half][i];
      if constexpr (kAheadV) {
#pragma unroll
        for (int b = 0; b < VB; ++b) vv[half][b] = now.vv[half][b];
      }
    }
    // -- 1. transposed scores ----------------------------------------------------------------------
    f32x4 s[RT][2];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        s[r][half] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
          if constexpr (kKeepQ) {
            Atom<T>::mma(s[r][half], now.kv[half][c], qv[r][c]);
          } else {
            const bool in = c * KC + VEC * quad + VEC <= D;
            Atom<T>::mma(s[r][half], now.kv[half][c],
                         load_or_zero<T>(q_row[r] + (in ? c * KC + VEC * quad : 0), row_ok[r] && in));
          }
        }
      }
    if (step + 1 < step_end) request(step + 1, now);  // (the products above have taken this tile's keys)
    // -- 2. scale, bias, mask, online softmax ------------------------------------------------------------
    // A tile that every row of the block sees whole (most tiles of a long prompt) needs no mask: the same for the
    // whole wave, so the choice costs a scalar branch.
    float shrink[RT];
    bool moved = false;
    auto softmax_tile = [&](auto whole, auto biased) LS_INLINED {
      constexpr bool kWhole = decltype(whole)::value, kBiased = decltype(biased)::value;
#pragma unroll
      for (int r = 0; r < RT; ++r) {
        bool see[2][4];
        float top = kNegSentinel;
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = key0 + 16 * half + 4 * quad + i;
            see[half][i] = kWhole || (row_ok[r] && key <= my_pos[r] && (key >= my_lo[r] || key < keep_first));
            float v = s[r][half][i] * scale;
            if constexpr (kBiased) v = v + my_bias[min(max(my_pos[r] - key, 0), n_dist - 1)];
            s[r][half][i] = v;
            top = fmaxf(top, see[half][i] ? v : kNegSentinel);
          }
        top = quad16_max(top);
        const float m_new = fmaxf(m_run[r], top);
        shrink[r] = softmax_exp<T>(m_run[r] - m_new);
        float sum = 0.f;
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            s[r][half][i] = see[half][i] ? softmax_exp<T>(s[r][half][i] - m_new) : 0.f;
            sum = sum + s[r][half][i];
          }
        sum = quad16_sum(sum);
        l_run[r] = l_run[r] * shrink[r] + sum;
        m_run[r] = m_new;
        moved = moved || shrink[r] != 1.0f;
      }
    };
    // (the mask and the bias are instances of the code, chosen by scalar branches once a tile)
    const bool whole_tile = key0 + kTileKeys - 1 <= p_first && (key0 >= lo_last || key0 + kTileKeys <= keep_first);
    if (my_bias) {
      if (whole_tile) softmax_tile(std::true_type{}, std::true_type{});
      else softmax_tile(std::false_type{}, std::true_type{});
    } else {
      if (whole_tile) softmax_tile(std::true_type{}, std::false_type{});
      else softmax_tile(std::false_type{}, std::false_type{});
    }
    // -- 3. values: column 16 b + l16 of V^T, keys 4 quad .. 4 quad + 3 of each half ----------------
    bool held = true;
#pragma unroll
    for (int half = 0; half < 2; ++half)
#pragma unroll
      for (int i = 0; i < 4; ++i) held = held && v_ok[half][i];
    const bool all_held = __all(held) != 0 && DV % 16 == 0;
    if (__all(!moved) == 0) {
#pragma unroll
      for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int b = 0; b < VB; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[r][b][i] = acc[r][b][i] * shrink[r];
    }
    typename Atom<T>::vec_t pb[RT][sizeof(T) == 2 ? 1 : 2];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      if constexpr (sizeof(T) == 2) {
        typedef __attribute__((ext_vector_type(8))) float f32x8;
        const f32x8 both = __builtin_shufflevector(s[r][0], s[r][1], 0, 1, 2, 3, 4, 5, 6, 7);
        pb[r][0] = __builtin_convertvector(both, bf16x8);
      } else {
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) pb[r][half][i] = s[r][half][i];
      }
    }
#pragma unroll
    for (int b = 0; b < VB; ++b) {
      const bool col_ok = 16 * b + l16 < DV;
      const long column = (long)(col_ok ? 16 * b + l16 : 0) << page_shift;
      auto value4 = [&](int half) LS_INLINED {
        if constexpr (kAheadV) {
          return vv[half][b];
        } else {
          return *reinterpret_cast<const v4_t*>(v_pages + v_at[half] + column);
        }
      };
      if constexpr (sizeof(T) == 2) {
        const bf16x4 v0 = value4(0), v1 = value4(1);
        bf16x8 a;
        if (all_held) {
          a = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            a[i] = (v_ok[0][i] && col_ok) ? v0[i] : (bf16_t)0.f;
            a[4 + i] = (v_ok[1][i] && col_ok) ? v1[i] : (bf16_t)0.f;
          }
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) Atom<T>::mma(acc[r][b], a, pb[r][0]);
      } else {
        f32x4 a[2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
          const f32x4 v = value4(half);
          if (all_held) {
            a[half] = v;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) a[half][i] = (v_ok[half][i] && col_ok) ? v[i] : 0.f;
          }
        }
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
          for (int half = 0; half < 2; ++half) Atom<T>::mma(acc[r][b], a[half], pb[r][half]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < RT; ++r) {
    if (!row_ok[r]) continue;
    const int row = DEC ? 0 : 16 * r + l16;
    if (n_runs > 1) {
      // [item][row][head][DV + 2]: the unnormalised output, then max and sum
      float* dst = part + (((long)blockIdx.x * part_rows + row) * H + my_head) * (DV + 2);
#pragma unroll
      for (int b = 0; b < VB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (16 * b + 4 * quad + i < DV) dst[16 * b + 4 * quad + i] = acc[r][b][i];
      if (quad == 0) {
        dst[DV] = m_run[r];
        dst[DV + 1] = l_run[r];
      }
      continue;
    }
    // the sink joins the sum as one more score; the row's weights then add up to less than one
    float top = m_run[r], total = l_run[r], keep = 1.0f;
    if (sink) {
      const float sv = sink[my_head];
      top = fmaxf(m_run[r], sv);
      keep = softmax_exp<T>(m_run[r] - top);
      total = l_run[r] * keep + softmax_exp<T>(sv - top);
    }
    const float inv = keep / total;
    T* dst = out + (long)(m.q_off + row0 + row) * ldo + (long)my_head * DV;
    const float* g_row = gate ? gate + (long)(m.q_off + row0 + row) * ldg + (long)my_head * DV : nullptr;
#pragma unroll
    for (int b = 0; b < VB; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = 16 * b + 4 * quad + i;
        if (c < DV) {
          float v = acc[r][b][i] * inv;
          if (g_row) v = v * sigmoid_f(g_row[c]);
          dst[c] = from_f32<T>(v);
        }
      }
  }
}

// ---------------------------------------------------------------------------
// Prompt portions, key and value tiles staged in LDS.  The kernel above spends some 25 vector instructions on
// every MFMA: addresses and selects for each fragment it takes from global memory, and the row statistics of a
// tile of only 32 keys.  Here a workgroup of four waves copies a tile of kStagedKeys keys (128 bytes of keys a
// value column: 64 in bfloat16, 32 in float) into LDS once, with a few 16-byte pieces a thread, and every wave
// reads its fragments from there at constant offsets.  A wave owns 32 rows of one head; the waves of a workgroup
// are min(GS, 4) query heads of the key/value head times 4 / min(GS, 4) groups of 32 rows, so a work item names a
// block of 32, 64 or 128 rows.  The next tile is requested into registers while a tile is worked on.  The
// arithmetic of a row (scores, statistics, sums) is that of the kernel above with larger tiles.
// ---------------------------------------------------------------------------
template <typename T> struct Staged {
  static constexpr int kKeys = 128 / (int)sizeof(T);                 // keys of a tile
  static constexpr int kKeyRow = D * (int)sizeof(T) + 16;            // bytes from a key to the next in LDS
  static constexpr int kValueRow = 128 + 16;                         // bytes from a value column to the next
  static constexpr int kBytes = kKeys * kKeyRow + DV * kValueRow;
  static constexpr bool kFits = kBytes <= 64 * 1024 && D % Atom<T>::VEC == 0;
};

template <typename T>
__global__ __launch_bounds__(256) void sink_attention_staged_kernel(
    const T* __restrict__ q, long ldq, const T* __restrict__ k_pages, const T* __restrict__ v_pages, int page_size,
    const int* __restrict__ table, int table_stride, const SeqMeta* __restrict__ seqs, const int* __restrict__ items,
    int H, int G, float scale, int window, int chunk, int keep_first, const float* __restrict__ sink,
    const float* __restrict__ dist_bias, int n_dist, const float* __restrict__ gate, long ldg, T* __restrict__ out,
    long ldo, float* __restrict__ part, int part_rows) {
  typedef typename Atom<T>::vec_t vec_t;
  typedef typename std::conditional<sizeof(T) == 2, bf16x4, f32x4>::type v4_t;
  constexpr int VEC = Atom<T>::VEC, KC = Atom<T>::KCHUNK;
  constexpr int KCH = D / KC + (D % KC ? 1 : 0);
  constexpr int TK = Staged<T>::kKeys, NG = TK / 16;              // groups of 16 keys in a tile
  constexpr int kKeyRow = Staged<T>::kKeyRow, kValueRow = Staged<T>::kValueRow;
  constexpr int kKeyPieces = TK * (D / VEC), kValuePieces = DV * (TK / VEC);
  constexpr int KP = (kKeyPieces + 255) / 256, VP = (kValuePieces + 255) / 256;
  __shared__ __attribute__((aligned(16))) char lds[Staged<T>::kFits ? Staged<T>::kBytes : 16];
  char* const k_lds = lds;
  char* const v_lds = lds + TK * kKeyRow;
  // the page ids of a tile and of the next one: looked up by a few threads two tiles ahead, so that no thread waits
  // for the block table before it can ask for its pieces
  constexpr int kTilePages = 16;
  __shared__ int page_s[2][kTilePages];

  const int seq = items[4 * blockIdx.x], rb = items[4 * blockIdx.x + 1];
  const int run = items[4 * blockIdx.x + 2], n_runs = max(1, items[4 * blockIdx.x + 3]);
  const SeqMeta m = seqs[seq];
  const int GS = H / G, g = blockIdx.y;
  const int HW = GS < 4 ? GS : 4, RG = 4 / HW;                     // heads and groups of 32 rows a workgroup
  const int block_rows = 32 * RG;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int l16 = lane & 15, quad = lane >> 4;
  const int row0 = rb * block_rows;
  if (row0 >= m.q_len) return;                                      // (the whole workgroup)
  const int nrows = min(block_rows, m.q_len - row0);
  const int p_first = m.q_start + row0, p_last = p_first + nrows - 1;
  const int* my_table = table + (long)m.table_row * table_stride;
  const int page_shift = __ffs(page_size) - 1, page_mask = page_size - 1;

  // this wave's head and rows
  const int in_group = blockIdx.z * HW + w % HW, rg = w / HW;
  const int wave_row0 = 32 * rg;
  const bool active = in_group < GS && rg < RG && wave_row0 < nrows;
  const int my_head = g * GS + (in_group < GS ? in_group : 0);
  const int wave_first = p_first + min(wave_row0, nrows - 1), wave_last = p_first + min(wave_row0 + 31, nrows - 1);
  bool row_ok[2];
  int my_pos[2], my_lo[2];
  vec_t qv[2][KCH];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int row = wave_row0 + 16 * r + l16;
    row_ok[r] = active && row < nrows;
    my_pos[r] = p_first + (row_ok[r] ? row : 0);
    my_lo[r] = first_seen(my_pos[r], window, chunk);
    const T* q_row = q + (long)(m.q_off + row0 + (row_ok[r] ? row : 0)) * ldq + (long)my_head * D;
#pragma unroll
    for (int c = 0; c < KCH; ++c) {
      const bool in = c * KC + VEC * quad + VEC <= D;
      qv[r][c] = load_or_zero<T>(q_row + (in ? c * KC + VEC * quad : 0), row_ok[r] && in);
    }
  }
  const int wave_lo_last = first_seen(wave_last, window, chunk);
  const float* my_bias = dist_bias ? dist_bias + (long)my_head * n_dist : nullptr;

  float m_run[2], l_run[2];
  f32x4 acc[2][VB];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    m_run[r] = kNegSentinel;
    l_run[r] = 0.f;
#pragma unroll
    for (int b = 0; b < VB; ++b) acc[r][b] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int lo_tile = first_seen(p_first, window, chunk) / TK;
  const int hi_tile = p_last / TK;
  const int kept_tiles = min((keep_first + TK - 1) / TK, lo_tile);   // tiles of kept first tokens below the window's
  const int n_tiles = kept_tiles + hi_tile - lo_tile + 1;
  auto tile_at = [&](int step) LS_INLINED { return step < kept_tiles ? step : lo_tile + (step - kept_tiles); };
  const int per_run = (n_tiles + n_runs - 1) / n_runs;
  const int step_begin = run * per_run, step_end = min(n_tiles, (run + 1) * per_run);

  // a thread's pieces of a tile: 16 bytes of a key, and of a value column (VEC consecutive keys, inside one page)
  vec_t k_piece[KP], v_piece[VP];
  // (pages of at least a tile's keys: one page a tile)
  const int tile_pages = max(1, TK >> page_shift);
  auto look_up = [&](int step) LS_INLINED {       // thread i: the page of the tile's i-th run of keys, -1 beyond the block
    const int key0 = tile_at(step) * TK;
    const int key = max(key0, ((key0 >> page_shift) + (int)threadIdx.x) << page_shift);
    const bool in = (int)threadIdx.x < tile_pages && step < step_end && key <= p_last;
    return in ? my_table[key >> page_shift] : -1;
  };
  auto request = [&](int step) LS_INLINED {
    const int key0 = tile_at(step) * TK;
    const int* pages = page_s[step & 1];
    const int first_page = key0 >> page_shift;
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int p = threadIdx.x + 256 * j;
      const int key = key0 + p / (D / VEC), seg = p % (D / VEC);
      const bool in = p < kKeyPieces && key <= p_last;
      const int page = in ? pages[(key >> page_shift) - first_page] : -1;
      const long at = (((long)(page >= 0 ? page : 0) * G + g) << page_shift) + (page >= 0 ? key & page_mask : 0);
      k_piece[j] = load_or_zero<T>(k_pages + at * D + seg * VEC, page >= 0);
    }
#pragma unroll
    for (int j = 0; j < VP; ++j) {
      const int p = threadIdx.x + 256 * j;
      const int col = p / (TK / VEC), key = key0 + (p % (TK / VEC)) * VEC;
      const bool in = p < kValuePieces && key <= p_last;
      const int page = in ? pages[(key >> page_shift) - first_page] : -1;
      const long at = ((((long)(page >= 0 ? page : 0) * G + g) * DV + (in ? col : 0)) << page_shift) + (page >= 0 ? key & page_mask : 0);
      vec_t v = load_or_zero<T>(v_pages + at, page >= 0);
      if (key0 + TK - 1 > p_last) {                                  // (only the tile that holds the block's last row:
#pragma unroll
        for (int i = 0; i < VEC; ++i)                                //  what lies beyond that row is not held)
          if (key + i > p_last) v[i] = (T)0.f;
      }
      v_piece[j] = v;
    }
  };
  auto store = [&]() LS_INLINED {
#pragma unroll
    for (int j = 0; j < KP; ++j) {
      const int p = threadIdx.x + 256 * j;
      if (p < kKeyPieces) *reinterpret_cast<vec_t*>(k_lds + (p / (D / VEC)) * kKeyRow + (p % (D / VEC)) * 16) = k_piece[j];
    }
#pragma unroll
    for (int j = 0; j < VP; ++j) {
      const int p = threadIdx.x + 256 * j;
      if (p < kValuePieces) *reinterpret_cast<vec_t*>(v_lds + (p / (TK / VEC)) * kValueRow + (p % (TK / VEC)) * 16) = v_piece[j];
    }
  };

  if (threadIdx.x < kTilePages) {
    page_s[step_begin & 1][threadIdx.x] = look_up(step_begin);
    page_s[(step_begin + 1) & 1][threadIdx.x] = look_up(step_begin + 1);
  }
  __syncthreads();
  if (step_begin < step_end) {
    request(step_begin);
    store();
  }
  __syncthreads();
  for (int step = step_begin; step < step_end; ++step) {
    const int key0 = tile_at(step) * TK;
    const int page_after = threadIdx.x < kTilePages ? look_up(step + 2) : -1;   // (on its way during the tile)
    if (step + 1 < step_end) request(step + 1);
    if (active && key0 <= wave_last) {
      // -- 1. transposed scores of the tile's groups of 16 keys ----------------------------------
      f32x4 s[2][NG];
#pragma unroll
      for (int ng = 0; ng < NG; ++ng) {
#pragma unroll
        for (int r = 0; r < 2; ++r) s[r][ng] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < KCH; ++c) {
          const bool in = c * KC + VEC * quad + VEC <= D;
          vec_t kf = *reinterpret_cast<const vec_t*>(k_lds + (ng * 16 + l16) * kKeyRow + (in ? c * 64 + quad * 16 : 0));
          if (!in) kf = Atom<T>::zero();
#pragma unroll
          for (int r = 0; r < 2; ++r) Atom<T>::mma(s[r][ng], kf, qv[r][c]);
        }
      }
      // -- 2. scale, bias, mask, online softmax -----------------------------------------------------
      float shrink[2];
      bool moved = false;
      auto softmax_tile = [&](auto whole, auto biased) LS_INLINED {
        constexpr bool kWhole = decltype(whole)::value, kBiased = decltype(biased)::value;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          bool see[NG][4];
          float top = kNegSentinel;
#pragma unroll
          for (int ng = 0; ng < NG; ++ng)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = key0 + 16 * ng + 4 * quad + i;
              see[ng][i] = kWhole || (row_ok[r] && key <= my_pos[r] && (key >= my_lo[r] || key < keep_first));
              float v = s[r][ng][i] * scale;
              if constexpr (kBiased) v = v + my_bias[min(max(my_pos[r] - key, 0), n_dist - 1)];
              s[r][ng][i] = v;
              top = fmaxf(top, see[ng][i] ? v : kNegSentinel);
            }
          top = quad16_max(top);
          const float m_new = fmaxf(m_run[r], top);
          shrink[r] = softmax_exp<T>(m_run[r] - m_new);
          float sum = 0.f;
#pragma unroll
          for (int ng = 0; ng < NG; ++ng)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              s[r][ng][i] = see[ng][i] ? softmax_exp<T>(s[r][ng][i] - m_new) : 0.f;
              sum = sum + s[r][ng][i];
            }
          sum = quad16_sum(sum);
          l_run[r] = l_run[r] * shrink[r] + sum;
          m_run[r] = m_new;
          moved = moved || shrink[r] != 1.0f;
        }
      };
      const bool whole_tile = key0 + TK - 1 <= wave_first && (key0 >= wave_lo_last || key0 + TK <= keep_first);
      if (my_bias) {
        if (whole_tile) softmax_tile(std::true_type{}, std::true_type{});
        else softmax_tile(std::false_type{}, std::true_type{});
      } else {
        if (whole_tile) softmax_tile(std::true_type{}, std::false_type{});
        else softmax_tile(std::false_type{}, std::false_type{});
      }
      // -- 3. values ---------------------------------------------------------------------------
      if (__all(!moved) == 0) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int b = 0; b < VB; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[r][b][i] = acc[r][b][i] * shrink[r];
      }
      constexpr int NC = sizeof(T) == 2 ? NG / 2 : NG;   // chunks of keys of the value product
      vec_t pb[2][NC];
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          if constexpr (sizeof(T) == 2) {
            typedef __attribute__((ext_vector_type(8))) float f32x8;
            const f32x8 both = __builtin_shufflevector(s[r][2 * c], s[r][2 * c + 1], 0, 1, 2, 3, 4, 5, 6, 7);
            pb[r][c] = __builtin_convertvector(both, bf16x8);
          } else {
            pb[r][c] = s[r][c];
          }
        }
#pragma unroll
      for (int b = 0; b < VB; ++b) {
        const bool col_ok = 16 * b + l16 < DV;
        const char* column = v_lds + (col_ok ? 16 * b + l16 : 0) * kValueRow;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          vec_t a;
          if constexpr (sizeof(T) == 2) {
            const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(column + ((2 * c) * 16 + 4 * quad) * 2);
            const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(column + ((2 * c + 1) * 16 + 4 * quad) * 2);
            a = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
          } else {
            a = *reinterpret_cast<const f32x4*>(column + (c * 16 + 4 * quad) * 4);
          }
          if constexpr (DV % 16 != 0) {
            if (!col_ok) a = Atom<T>::zero();
          }
#pragma unroll
          for (int r = 0; r < 2; ++r) Atom<T>::mma(acc[r][b], a, pb[r][c]);
        }
      }
    }
    __syncthreads();                       // every wave has read this tile
    if (step + 1 < step_end) store();
    if (threadIdx.x < kTilePages) page_s[step & 1][threadIdx.x] = page_after;   // (this tile's ids are no longer read)
    __syncthreads();
  }

  if (!active) return;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    if (!row_ok[r]) continue;
    const int row = wave_row0 + 16 * r + l16;
    if (n_runs > 1) {
      float* dst = part + (((long)blockIdx.x * part_rows + row) * H + my_head) * (DV + 2);
#pragma unroll
      for (int b = 0; b < VB; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (16 * b + 4 * quad + i < DV) dst[16 * b + 4 * quad + i] = acc[r][b][i];
      if (quad == 0) {
        dst[DV] = m_run[r];
        dst[DV + 1] = l_run[r];
      }
      continue;
    }
    float top = m_run[r], total = l_run[r], keep = 1.0f;
    if (sink) {
      const float sv = sink[my_head];
      top = fmaxf(m_run[r], sv);
      keep = softmax_exp<T>(m_run[r] - top);
      total = l_run[r] * keep + softmax_exp<T>(sv - top);
    }
    const float inv = keep / total;
    T* dst = out + (long)(m.q_off + row0 + row) * ldo + (long)my_head * DV;
    const float* g_row = gate ? gate + (long)(m.q_off + row0 + row) * ldg + (long)my_head * DV : nullptr;
#pragma unroll
    for (int b = 0; b < VB; ++b)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = 16 * b + 4 * quad + i;
        if (c < DV) {
          float v = acc[r][b][i] * inv;
          if (g_row) v = v * sigmoid_f(g_row[c]);
          dst[c] = from_f32<T>(v);
        }
      }
  }
}

// Fold the runs of row blocks: a fold item (first work item, runs, first packed row, rows) names the work items
// first .. first + runs - 1 of one row block, whose partial results are folded in ascending order for each of its
// rows; the sink joins the sum and the gate multiplies the result.  One workgroup a (fold item, head, row).
template <typename T>
__global__ __launch_bounds__(64) void sink_combine_kernel(const float* __restrict__ part, int part_rows, int H,
                                                          const int* __restrict__ folds, const float* __restrict__ sink,
                                                          const float* __restrict__ gate, long ldg, T* __restrict__ out,
                                                          long ldo) {
  const int first = folds[4 * blockIdx.x], n_runs = folds[4 * blockIdx.x + 1];
  const int row0 = folds[4 * blockIdx.x + 2], rows = folds[4 * blockIdx.x + 3];
  const int h = blockIdx.y;
  const long stride = (long)part_rows * H * (DV + 2);  // from a run to the next
  __shared__ float factor_s[64];
  for (int r = blockIdx.z; r < rows; r += gridDim.z) {
    const float* mine = part + (((long)first * part_rows + r) * H + h) * (DV + 2);
    // lane k holds run k's statistics (runs <= 64): all of them are requested at once
    const int k_mine = threadIdx.x;
    const float m_k = k_mine < n_runs ? mine[k_mine * stride + DV] : kNegSentinel;
    const float l_k = k_mine < n_runs ? mine[k_mine * stride + DV + 1] : 0.f;
    float top = sink ? sink[h] : kNegSentinel;
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) top = fmaxf(top, __shfl_xor(top, step, kWave));
    float top_runs = m_k;
#pragma unroll
    for (int step = 1; step < 64; step <<= 1) top_runs = fmaxf(top_runs, __shfl_xor(top_runs, step, kWave));
    top = fmaxf(top, top_runs);
    const float f_k = k_mine < n_runs ? softmax_exp<T>(m_k - top) : 0.f;
    __syncthreads();
    factor_s[k_mine] = f_k;
    float total = 0.f;
    for (int k = 0; k < n_runs; ++k) total = total + __shfl(l_k, k, kWave) * __shfl(f_k, k, kWave);   // ascending
    if (sink) total = total + softmax_exp<T>(sink[h] - top);
    const float inv = 1.0f / total;
    __syncthreads();
    for (int c = threadIdx.x; c < DV; c += 64) {
      float sum = 0.f;
      int k = 0;
      for (; k + 4 <= n_runs; k += 4) {
        const float p0 = mine[k * stride + c], p1 = mine[(k + 1) * stride + c], p2 = mine[(k + 2) * stride + c],
                    p3 = mine[(k + 3) * stride + c];
        sum = (((sum + p0 * factor_s[k]) + p1 * factor_s[k + 1]) + p2 * factor_s[k + 2]) + p3 * factor_s[k + 3];
      }
      for (; k < n_runs; ++k) sum = sum + mine[k * stride + c] * factor_s[k];
      float v = sum * inv;
      if (gate) v = v * sigmoid_f(gate[(long)(row0 + r) * ldg + (long)h * DV + c]);
      out[(long)(row0 + r) * ldo + h * DV + c] = from_f32<T>(v);
    }
  }
}

}  // namespace ls

LS_DEFINE_ERROR_API

using namespace ls;

extern "C" int ls_sink_dim() { return D; }
extern "C" int ls_sink_vdim() { return DV; }
extern "C" int ls_sink_max_row_tiles() { return 4; }
// The staged kernel for prompt portions: keys of a tile (0: this library's sizes do not fit it) and rows of a work
// item's block for H query heads over G key/value heads.
extern "C" int ls_sink_staged_keys(int dtype) {
  if (dtype == kF32) return Staged<float>::kFits ? Staged<float>::kKeys : 0;
  return Staged<bf16_t>::kFits ? Staged<bf16_t>::kKeys : 0;
}
extern "C" int ls_sink_staged_rows(int H, int G) {
  const int GS = H / (G > 0 ? G : 1);
  return 32 * (4 / (GS < 4 ? (GS > 0 ? GS : 1) : 4));
}

// q [T][ldq] (H heads of D); key pages [pages][G][page_size][D], value pages [pages][G][DV][page_size]; table
// [slots][table_stride]; seqs: the step's requests; items: n_items work items of four ints (request of the step,
// block of 16 row_tiles of its rows, run, runs); row_tiles 1, 2 or 4, or 0 for a step of single decoded tokens.
// sink [H] float or null; dist_bias [H][n_dist] float or null; gate: float [T][ldg] (H heads of DV) or null;
// out [T][ldo].  Work items with runs > 1 leave their results in part (n_items * part_rows * H * (DV + 2) floats;
// part_rows 16 row_tiles, or 1 for decoded tokens) and the n_folds fold items of four ints (first work item, runs,
// first packed row, rows) say which to fold into which rows of out in a second launch.
extern "C" int ls_sink_attention(int dtype, const void* q, long ldq, const void* k_pages, const void* v_pages,
                                 int page_size, const int* table, int table_stride, const void* seqs,
                                 const int* items, int n_items, int row_tiles, int H, int G, float scale, int window,
                                 int chunk, int keep_first, const float* sink, const float* dist_bias, int n_dist, const float* gate,
                                 long ldg, void* out, long ldo, const int* folds, int n_folds, float* part,
                                 int part_rows, void* stream) {
  LS_REQUIRE(row_tiles == 0 || row_tiles == 1 || row_tiles == 2 || row_tiles == 4 || row_tiles == 8,
             "sink_attention: %d row tiles", row_tiles);
  LS_REQUIRE(H > 0 && G > 0 && H % G == 0, "sink_attention: %d query heads over %d key/value heads", H, G);
  LS_REQUIRE(part_rows == (row_tiles == 8 ? ls_sink_staged_rows(H, G) : row_tiles ? 16 * row_tiles : 1),
             "sink_attention: partial results of %d rows", part_rows);
  LS_REQUIRE(row_tiles != 8 || (ls_sink_staged_keys(dtype) > 0 && page_size % (dtype == kF32 ? 4 : 8) == 0),
             "sink_attention: the staged kernel does not take these sizes (page size %d)", page_size);
  LS_REQUIRE(n_folds >= 0 && (n_folds == 0 || (part && folds)), "sink_attention: %d fold items need partial results", n_folds);
  LS_REQUIRE(n_items > 0 && q && k_pages && v_pages && table && seqs && items && out, "sink_attention: null operand");
  LS_REQUIRE(ldq >= (long)H * D && ldo >= (long)H * DV && (!gate || ldg >= (long)H * DV), "sink_attention: rows are too short");
  LS_REQUIRE(page_size >= 4 && (page_size & (page_size - 1)) == 0 && table_stride > 0,
             "sink_attention: page size %d is not a power of two", page_size);
  LS_REQUIRE(window >= 0 && chunk >= 0 && (!dist_bias || n_dist > 0), "sink_attention: window %d, chunk %d, %d distances",
             window, chunk, n_dist);
  LS_REQUIRE(keep_first >= 0 && (keep_first == 0 || (window > 0 && chunk == 0)),
             "sink_attention: %d kept first tokens need a window (and no chunks)", keep_first);
  LS_REQUIRE(reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(k_pages) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(v_pages) % 16 == 0,
             "sink_attention: operands must be 16-byte aligned");
  LS_REQUIRE(dtype == kF32 || dtype == kBF16, "sink_attention: unknown dtype %d", dtype);
  LS_REQUIRE(ldq % (dtype == kF32 ? 4 : 8) == 0, "sink_attention: query rows must be 16-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int GS = H / G;
#define LS_SINK_LAUNCH(T_, RT_, DEC_)                                                                                  \
  hipLaunchKernelGGL((sink_attention_kernel<T_, RT_, DEC_>),                                                           \
                     dim3(n_items, G, DEC_ ? (GS + 15) / 16 : (GS + kMaxWaves - 1) / kMaxWaves),                       \
                     dim3(DEC_ ? 64 : 64 * (GS < kMaxWaves ? GS : kMaxWaves)), 0, s, (const T_*)q, ldq,                \
                     (const T_*)k_pages, (const T_*)v_pages, page_size, table, table_stride, (const SeqMeta*)seqs,     \
                     items, H, G, scale, window, chunk, keep_first, sink, dist_bias, n_dist, gate, ldg, (T_*)out, ldo, \
                     part, part_rows)
#define LS_SINK_STAGED(T_)                                                                                             \
  hipLaunchKernelGGL(sink_attention_staged_kernel<T_>, dim3(n_items, G, (GS + 3) / 4), dim3(256), 0, s, (const T_*)q,  \
                     ldq, (const T_*)k_pages, (const T_*)v_pages, page_size, table, table_stride,                      \
                     (const SeqMeta*)seqs, items, H, G, scale, window, chunk, keep_first, sink, dist_bias, n_dist,     \
                     gate, ldg, (T_*)out, ldo, part, part_rows)
#define LS_SINK_BY_ROWS(T_)                       \
  switch (row_tiles) {                            \
    case 0: LS_SINK_LAUNCH(T_, 1, true); break;   \
    case 1: LS_SINK_LAUNCH(T_, 1, false); break;  \
    case 2: LS_SINK_LAUNCH(T_, 2, false); break;  \
    case 4: LS_SINK_LAUNCH(T_, 4, false); break;  \
    default: LS_SINK_STAGED(T_); break;           \
  }
  if (dtype == kF32) {
    LS_SINK_BY_ROWS(float)
    if (n_folds > 0)
      hipLaunchKernelGGL(sink_combine_kernel<float>, dim3(n_folds, H, part_rows), dim3(64), 0, s, part, part_rows, H,
                         folds, sink, gate, ldg, (float*)out, ldo);
  } else {
    LS_SINK_BY_ROWS(bf16_t)
    if (n_folds > 0)
      hipLaunchKernelGGL(sink_combine_kernel<bf16_t>, dim3(n_folds, H, part_rows), dim3(64), 0, s, part, part_rows, H,
                         folds, sink, gate, ldg, (bf16_t*)out, ldo);
  }
#undef LS_SINK_BY_ROWS
#undef LS_SINK_STAGED
#undef LS_SINK_LAUNCH
  return check_launch("sink_attention");
}
