// The C interface of the mixers library (mixers.hip).  Conventions as in core_api.h: dtype 0 is
// float32 and 1 bfloat16, pointers are device pointers, `stream` is a hipStream_t passed as
// void*, the return value is 0 or a negative code whose message ls_last_error() returns.
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

const char* ls_last_error();

// Dynamic Tanh norm of rows of the float residual stream: h[row] += P[0][row] + P[1][row] + ... first when P
// [slices][p_rows][width] is given; out [n_rows][ld_out] = tanh(alpha[0] * h[row]) * weight + bias, or nothing
// when out is null.  rows: the rows of h to take, or null for the first n_rows.
int ls_dyt(int dtype, float* h, const float* P, int slices, int p_rows, const float* weight, const float* bias,
           const float* alpha, void* out, const int* rows, int n_rows, int width, long ldh, long ld_out, void* stream);

// x float [rows][2 * width] (gates, then ups): out = g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit),
// u = clamp(up, -limit, limit).
int ls_glu_clamped(int out_dtype, const float* x, long ldx, void* out, long ldo, int rows, int width, float limit,
                   float alpha, void* stream);

// x = cap * tanh(x / cap) in place on float rows.
int ls_softcap(float* x, long ld, int rows, int width, float cap, void* stream);

// Post pass of an attention projection with keys of size D and values of size DV (see mixers.hip).
int ls_talk_qkv(int dtype, const float* raw, long ld, int n_tokens, int H, int G, int D, int DV, const float* bias,
                const float* cos_table, const float* sin_table, int rot, int table_positions, int max_pos,
                const int* tok_seq, const int* tok_pos, const void* seqs, const int* table, int table_stride,
                void* q_out, long ldq, void* k_pages, void* v_pages, int page_size, int vmix_mode, const float* vmix,
                float* v_first, long ldv, void* stream);

// Post pass of an attention projection raw = q | k | v (| more): biases, a root-mean-square norm over the whole of q
// and of k (weights q_norm [H*D], k_norm [G*D], or null), rotation in pairs (i, i + rot/2) or of neighbours, keys
// that are also the values (keys_are_values: no v in raw, the biased unnormalised k is stored as v).  per_head: every
// head of q and of k is divided by its own root mean square over D instead (no weights).  Queries and
// keys are written with Dp >= D elements a head, zeros beyond D.
int ls_qkv_post(int dtype, const float* raw, long ld, int n_tokens, int H, int G, int D, int Dp, int DV, int keys_are_values,
                int per_head, const float* bias, const float* q_norm, const float* k_norm, float eps, const float* cos_table,
                const float* sin_table, int rot, int neighbours, int table_positions, int max_pos, const int* tok_seq,
                const int* tok_pos, const void* seqs, const int* table, int table_stride, void* q_out, long ldq,
                void* k_pages, void* v_pages, int page_size, void* stream);

// Linear recurrence S_t = diag(a_t) S_(t-1) + b_t v_t^T, o_t = S_t^T q_t over the tokens of every request of the
// step, state [slots][H][D][DV] float (mode 0: HGRN2 gates from p0 = lower bounds [H*D] and p1 = gate bias or null;
// mode 1: retention with p0 = decay [H] and rotated q, k at the positions tok_pos [n_tokens]).  out [T][ldo] float
// gets o_t.  gates: scratch of ls_linrec_gate_floats(n_tokens, H, D) floats, 16-byte aligned.
int ls_linrec_max_dim();
long ls_linrec_gate_floats(int n_tokens, int H, int D);
int ls_linrec(int mode, const float* raw, long ld, int q_at, int ab_at, int v_at, int n_tokens, int H, int D, int DV,
              const float* p0, const float* p1, const float* cos_table, const float* sin_table, int rot,
              int table_positions, int max_pos, const int* tok_pos, const void* seqs, int n_seqs, float* state,
              float* gates, float* out, long ldo, void* stream);

// Per (token, head): x [DV] / sqrt(mean(x^2) + eps), times weight [DV] and silu(gate) (gate_act 0) or sigmoid(gate)
// (gate_act 1) where given.
int ls_head_norm_gate(int out_dtype, const float* x, long ldx, int n_tokens, int H, int DV, const float* weight,
                      const float* gate, long ldg, int gate_act, float eps, void* out, long ldo, void* stream);

// out [T][ld_out] float = table[token] * scale + pairs[(token before * mul_prev + token * mul_cur) mod buckets]; row
// `buckets` of pairs for a request's first token.  state: one int a slot, the last token of the request so far.
int ls_embed_pair(int dtype, const int* tokens, const int* tok_seq, const int* tok_pos, const void* seqs, const void* table,
                  int vocab, const void* pairs, int buckets, long mul_prev, long mul_cur, int* state, long state_stride,
                  float* out, int n_tokens, int width, long ld_out, float scale, void* stream);

// out [T][ldo] = n[t] + (n[t-1] - n[t]) * mu, n [T][ldn] float; the row before a portion's first one is the request's
// state (width floats a slot; zeros at a request's first token), which is left as the portion's last row.
// A step of single tokens: h[t] += P[0][t] + ... (P null: nothing to add), the RMS norm with `weight`, and the shift
// with the request's state, which becomes the token's normed row; one launch.  width % 4 == 0.
int ls_add_rmsnorm_shift(int out_dtype, float* h, const float* P, int slices, int p_rows, const float* weight,
                         const float* mu, const int* tok_seq, const int* tok_pos, const void* seqs, float* state,
                         long state_stride, void* out, int n_rows, int width, long ldh, long ld_out, float eps, void* stream);
int ls_token_shift(int out_dtype, const float* n, long ldn, const float* mu, const int* tok_seq, const int* tok_pos,
                   const void* seqs, float* state, long state_stride, void* out, long ldo, int n_tokens, int width,
                   void* stream);

// A residual stream of n copies X [rows][n][width] float.  Write (P given): y = P[0][row] + P[1][row] + ..., then
// X'_t = sum_s mix[s][t] X_s + gain[t] y for all copies at once.  Read (out given): u = sum_t take[t] X'_t (take null:
// the plain sum), out [n_rows][ld_out] = u / sqrt(mean(u^2) + eps) * weight.  rows: the rows to take, or null.
int ls_streams_max();
int ls_streams_max_width();
int ls_streams_step(int dtype, float* X, long ldx, int n, int width, const float* P, int slices, int p_rows,
                    const float* mix, const float* gain, const float* take, const float* weight, float eps, void* out,
                    long ld_out, const int* rows, int n_rows, void* stream);

// Post pass of the down projections of attention over a latent, raw = a (QR) | c (CR) | r (RD): a and c normalised
// with their weights, r rotated in neighbouring pairs; a -> a_out, c | r -> key pages (heads of Dp elements, one
// key/value head), c -> value pages.  has_kv 0: a alone.
int ls_latent_post(int dtype, const float* raw, long ld, int n_tokens, int QR, int CR, int RD, int Dp, int has_kv,
                   const float* a_weight, const float* c_weight, float eps, const float* cos_table, const float* sin_table,
                   int rot, int table_positions, int max_pos, const int* tok_seq, const int* tok_pos, const void* seqs,
                   const int* table, int table_stride, void* a_out, long lda, void* k_pages, void* v_pages, int page_size,
                   void* stream);

// Post pass of the queries' up projection qf (heads of D plain and RD rotated dimensions): the plain part to
// plain_out [T][H*D], the rotated part, rotated, to q_out [T][H*Dp] behind the CR dimensions of the latent.
int ls_latent_query(int dtype, const float* qf, long ld, int n_tokens, int H, int D, int RD, int CR, int Dp,
                    const float* cos_table, const float* sin_table, int rot, int table_positions, int max_pos,
                    const int* tok_pos, void* plain_out, long ldp, void* q_out, long ldq, void* stream);

// out[t][head * o_stride + n] = sum_k w[head][n][k] x[t][head * x_stride + k]; w [H][N][K], x and out of one dtype.
int ls_heads_product(int dtype, const void* x, long ldx, int x_stride, const void* w, int H, int N, int K, int n_rows,
                     void* out, long ldo, int o_stride, void* stream);

// The gated delta rule over the tokens of every request of the step (see latent_delta.hip).  raw float = q (G heads of
// D) | k (G of D) | v (H of DV) | b (H) | a (H) | ...; state [slots][state_stride] float = S [H][D][DV], then the
// last M - 1 inputs of the convolutions [M - 1][2 G D + H DV]; taps [2 G D + H DV][M]; out [T][ldo] float gets o_t.
int ls_delta_max_dim();
int ls_delta_padded_dim(int D);
long ls_delta_scratch_floats(int n_tokens, int G, int H, int D, int DV);
long ls_delta_scratch_floats_channel(int n_tokens, int G, int H, int D, int DV);
// chan [T][ldc] float or null: logits of a decay a head and key channel (H * D a token; dt_bias [H * D]; raw then ends
// with b; scratch of ls_delta_scratch_floats_channel floats): g = exp(-exp(A_log_h) softplus(chan + dt_bias)).
int ls_delta_rule(const float* raw, long ld, int n_tokens, int G, int H, int D, int DV, int M, const float* taps,
                  const float* a_log, const float* dt_bias, float unit_eps, const int* tok_seq, const int* tok_pos,
                  const void* seqs, int n_seqs, float* state, long state_stride, float* scratch, float* out, long ldo,
                  const float* chan, long ldc, void* stream);

int ls_listed_index(const char* name);
int ls_call_listed(int index, const long long* words, int n);

#ifdef __cplusplus
}
#endif
