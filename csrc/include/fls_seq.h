// C ABI of libfls_seq.so: the kernels of the stateful (hybrid) models, csrc/kernels/seq.
// Element type codes: 0 = fp32, 1 = bf16.  Every function returns 0 or a HIP error code, runs on
// stream s, and launches nothing when its row count is 0.  Row metadata of a step batch:
//   tok_seq[T] request-in-batch of a row, tok_pos[T] its position, cu[B+1] row offsets of the
//   requests, pos0[B] position of a request's first row in this step, slot[B] its state slot.
#pragma once
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
typedef void* fls_stream_t;
int fls_seq_version(void);
// C[M,N] = A[M,K] . W[N,K]^T (+ bias[N] fp32).  A of type ta, W of type tw (A is rounded to tw
// when they differ); fp32 accumulation on the matrix cores (bf16: 32x32x8; fp32: 32x32x2, true fp32).
// groups > 1 with offs == null: strided batch g: A + (g % a_mod) * a_gs, W + g * w_gs, C / bias + g * c_gs.
// offs != null: row groups: group g owns rows [offs[g], offs[g+1]) of A and C and weight W + g * w_gs;
// M is then the total row count (the bound of every group's rows).
// Epilogue: + bias, then xIELU when act != null (act = {p, q}), stored as type tc (fp32, or bf16 when the
// consumer is the next product).
int fls_seq_gemm(const void* A, int ta, const void* W, int tw, void* C, int tc, const float* bias, const float* act,
                 int M, int N, int K, int lda, int ldw, int ldc, int groups, const int* offs, long long a_gs,
                 int a_mod, long long w_gs, long long c_gs, fls_stream_t s);
// y[r] = w * x[row] / sqrt(mean_g(x[row]^2) + eps) per group of D / groups columns, row = idx ? idx[r] : r.
// add != 0: y (fp32) += instead (the residual update), ty ignored.  woff is added to the weight (1 for
// weights stored around zero).
int fls_seq_group_rmsnorm(const float* x, int ldx, const int* idx, const float* w, void* y, int ty, int ldy,
                          int rows, int D, int groups, float eps, int add, float woff, fls_stream_t s);
// out[t] = table[ids[t]] * scale (fp32 rows of the residual stream)
int fls_seq_embed(const int* ids, const void* table, int tt, float* out, int T, int D, int V, float scale, fls_stream_t s);
// Dynamic Tanh norm: y[r, c] = tanh(alpha[0] x[row, c]) wb[c] + wb[D + c], row = idx ? idx[r] : r; y of type ty
int fls_seq_dyt_norm(const float* x, int ldx, const int* idx, const float* wb, const float* alpha, void* y, int ty,
                     int ldy, int rows, int D, fls_stream_t s);
// x += mult * y, then h = tanh(alpha[0] x) wb[c] + wb[D + c] of the new x (h of type th): residual update + next norm
int fls_seq_add_scaled_dyt(float* x, int ldx, const float* y, int ldy, float mult, const float* wb, const float* alpha,
                           void* h, int th, int ldh, int rows, int D, fls_stream_t s);
// x += mult * y (fp32 rows)
int fls_seq_add_scaled(float* x, int ldx, const float* y, int ldy, int rows, int D, float mult, fls_stream_t s);
int fls_seq_gather_rows(const void* x, int tx, int ldx, const int* idx, void* y, int ldy, int rows, int D, fls_stream_t s);
// xIELU: z > 0: softplus(p) z^2 + z/2; else (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2; act = {p, q}
int fls_seq_xielu(const float* z, int ldz, const float* act, void* y, int ty, int ldy, int rows, int cols, fls_stream_t s);
// y[r, c] = act(gu[r, c]) * gu[r, cols + c]; act: 0 = silu, 1 = gelu (tanh form)
int fls_seq_gate_mul(const float* gu, int ldg, void* y, int ty, int ldy, int rows, int cols, int act, fls_stream_t s);
// y = f(z) elementwise; kind: 0 = tanh, 1 = gelu (exact: 0.5 z (1 + erf(z / sqrt 2)))
int fls_seq_unary(const float* z, int ldz, void* y, int ty, int ldy, int rows, int cols, int kind, fls_stream_t s);
// per row t and head h: the n entries x[t, x_col + h x_hs ...] (x of type tx), RMS-normed over n times w[n] (w != null), the first
// rot entries rotated in pairs (2i, 2i+1) by the angle tok_pos[t] * freqs[i]; written as type to at
// out[row, out_col + h out_hs ...], row = row_map ? row_map[t] : t; raw (nullable, like out, row stride ldr)
// receives the entries unchanged.  unit_after != 0: after the rotation the n entries are divided by
// sqrt(mean(entries^2) + eps), without a weight.  n <= 512.  half != 0: the pairs are (i, i + rot / 2) instead;
// amp: a factor on every cosine and sine
int fls_seq_head_norm_rope(const void* x, int tx, int ldx, int x_col, int x_hs, int heads, int n, const float* w, float eps,
                           const float* freqs, int rot, const int* tok_pos, const int* row_map, void* out, int to,
                           int ldo, int out_col, int out_hs, void* raw, int ldr, int rows, int unit_after, int half, float amp,
                           fls_stream_t s);
int fls_seq_softcap(float* z, int ldz, int rows, int cols, float cap, fls_stream_t s);
int fls_seq_argmax(const float* z, int ldz, int rows, int cols, int* out, fls_stream_t s);
// k rows RMS-normed over all kcols (times kn), k and v rows written at row kv_slot[r] of the pools
int fls_seq_kv_store(const float* k, int ldk, const float* kn, float eps, const float* v, int ldv, void* kc, void* vc,
                     int tc, const int* kv_slot, int rows, int kcols, int vcols, fls_stream_t s);
// attention of every row over the keys of its request's pages that it may see: j <= i and
// (chunk > 0: floor(j / chunk) == floor(i / chunk)) and (window > 0: j > i - window), and besides them the
// first keep_first keys of the sequence; score = cap(scale q.k) - r1[h] log(1 + r2[h] (i - j)) (r1, r2 nullable),
// cap(s) = softcap tanh(s / softcap) if softcap > 0.  Weights: softmax over the visible keys, or, with
// gate_bias[H], sigmoid(score + gate_bias[h]) for every key on its own.  Keys / values: the first G d / G dv
// columns of pool rows ldk / ldv wide (both may be one pool).  q of type tq (fp32 allowed over bf16 pools),
// pools and out of type tc.  out = result * out_scale.  nsplit > 1: every row's keys are cut into nsplit
// ranges that run as blocks of their own (few rows, many keys: decoding) and are merged by a second
// kernel; part: T H nsplit (dv + 4) floats of scratch (16-byte aligned).  has_sink != 0 (softmax only): one more
// entry of score `sink` and no value joins the softmax's sum.  head_gate (nullable) [T, H] fp32, row stride ldhg:
// the output of (row, head) times sigmoid(head_gate[t, h]).
// out of type to (fp32 over bf16 pools allowed).  Gv (0: G), a divisor of G: the value pool holds Gv heads and key head g
// reads value head g % Gv (several score maps over the same values).
int fls_seq_attn_paged(const void* q, int ldq, int tq, const void* kc, int ldk, const void* vc, int ldv, int tc,
                       void* out, int to, int ldo, const int* tok_seq, const int* tok_pos, const int* page_table,
                       int pt_stride, int T, int H, int G, int d, int dv, float scale, float softcap,
                       const float* r1, const float* r2, int chunk, int window, int keep_first,
                       const float* gate_bias, float out_scale, int page_size, int nsplit, float* part,
                       int has_sink, float sink, const float* head_gate, int ldhg, int Gv, fls_stream_t s);
// the same attention on the matrix cores for bf16 pools and rows in tiles: tiles[n_tiles][2] = (first packed
// row, rows <= 128) of one request each, covering every row of the step; q of type tq.  -2: shape not
// served (use the above)
int fls_seq_attn_prefill(const void* q, int ldq, int tq, const void* kc, int ldk, const void* vc, int ldv, void* out,
                         int to, int ldo, const int* tiles, int n_tiles, const int* tok_seq, const int* tok_pos,
                         const int* page_table, int pt_stride, int H, int G, int d, int dv, float scale,
                         float softcap, const float* r1, const float* r2, int chunk, int window, int keep_first,
                         const float* gate_bias, float out_scale, int page_size, int has_sink, float sink,
                         const float* head_gate, int ldhg, int Gv, fls_stream_t s);
// softmax attention of few rows whose H / G <= 32 query heads per key / value head become the columns of one
// matrix-core tile (decode steps over cached latent rows): fp32 q, bf16 pools and out, window and kept first
// keys as above; nsplit ranges of key tiles per row, part: T H nsplit (dv + 4) floats.  -2: shape not served
int fls_seq_attn_heads(const void* q, int ldq, const void* kc, int ldk, const void* vc, int ldv, void* out, int ldo,
                       const int* tok_seq, const int* tok_pos, const int* page_table, int pt_stride, int T, int H,
                       int G, int d, int dv, float scale, int window, int keep_first, float out_scale, int page_size,
                       int nsplit, float* part, fls_stream_t s);
// causal per-channel convolution over each request's rows, history from / to state[slot][taps-1][C];
// b nullable; residual != 0: + the input row; out of type to; one_row_each != 0: the caller knows that every
// request brings exactly one row (the state is then rewritten by the same kernel)
int fls_seq_causal_conv(const float* x, int ldx, const float* w, const float* b, float* state, void* out, int to, int ldo,
                        const int* tok_seq, const int* cu, const int* pos0, const int* slot, int T, int B, int C,
                        int taps, int act, int residual, int one_row_each, fls_stream_t s);
// projected rows z = [q (H d) | k (G d) | v (G dv) | ...] into attention in one pass: causal convolution per channel
// (w [C, taps] nullable, history in state[slot][taps-1][C] as for fls_seq_causal_conv), q and k heads rotated in pairs
// over their first rot entries (angle tok_pos * freqs[i]) and divided by sqrt(mean(head^2) + eps), q to qo (fp32
// [T, H d]), k and v (v as convolved) to row kv_slot[t] of pools of type tc.  G = 0: queries only.  d, dv <= 512.
// Gv (< 0: G): the row holds Gv value heads after its G key heads.  qnw / knw (nullable, [d]): the q / k heads are instead
// RMS-normed BEFORE the rotation, times that weight (x / rms(x) * w, then rotated).
int fls_seq_qkv_conv_rope(const float* z, int ldz, const float* w, float* state, int taps, const int* tok_seq,
                          const int* tok_pos, const int* cu, const int* pos0, const int* slot, const int* kv_slot,
                          int T, int B, int H, int G, int d, int dv, float eps, const float* freqs, int rot, float* qo,
                          int ldq, void* kc, int ldk, void* vc, int ldv, int tc, int one_row_each, int Gv, const float* qnw,
                          const float* knw, fls_stream_t s);
// generalized delta rule, per head a state S[d][d] in state[slot][H][d][d]:
// S_t = diag(w) S_(t-1) - (a * u)(u^T S_(t-1)) + k v^T, o = S_t^T r; u = k / sqrt(sum k^2 + key_eps),
// w = exp(-decay_scale sigmoid(wz + w0)), a = sigmoid(az); out = out_scale o / rms_head(o; norm_eps) norm_w sigmoid(g).
// r, k, v, az, wz, g: fp32 [T, H d] with their row strides; d <= 128.  col_splits > 1 (a divisor of d): the
// columns of every state are cut over that many blocks (few heads x requests, many rows) and the outputs
// are finished by a second kernel; raw: T H d floats of scratch
int fls_seq_delta_rule_scan(const float* r, int ldr, const float* k, int ldk, const float* v, int ldv, const float* az,
                            int lda, const float* wz, int ldw, const float* g, int ldg, const float* w0,
                            const float* norm_w, float* state, void* out, int to, int ldo, const int* cu,
                            const int* pos0, const int* slot, int T, int B, int H, int d, float decay_scale,
                            float key_eps, float norm_eps, float out_scale, int col_splits, float* raw,
                            fls_stream_t s);
// S_t = a_t S_(t-1) + sqrt(1 - a_t^2) sigmoid(g[t, W + c]) u_t, a_t = exp(-c sigmoid(g[t, c]) softplus(lam));
// out = S_t * gelu_tanh(y_t); state[slot][W]
int fls_seq_rglru_scan(const float* u, int ldu, const float* g, int ldg, const float* lam, const float* y, int ldy,
                       float* state, void* out, int to, int ldo, const int* cu, const int* pos0, const int* slot,
                       int B, int W, float c, fls_stream_t s);
// the same over row tiles (tiles[n_tiles][2] as for fls_seq_attn_prefill, tile_cu[B+1] = each request's range of
// tiles, scratch: 2 n_tiles W floats): three passes, every tile walked in parallel
int fls_seq_rglru_scan_tiled(const float* u, int ldu, const float* g, int ldg, const float* lam, const float* y,
                             int ldy, float* state, void* out, int to, int ldo, const int* tiles, int n_tiles,
                             const int* tile_cu, float* scratch, const int* pos0, const int* slot, int B, int W,
                             float c, fls_stream_t s);
// S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t, dt_t = softplus(dt + dt_bias);
// out = y * silu(z) fp32; xbc = [x (nh P) | B (G N) | C (G N)] columns; state[slot][nh][N][P]
int fls_seq_ssd_scan(const float* xbc, int ldx, const float* z, int ldz, const float* dt, int lddt,
                     const float* dt_bias, const float* A_log, const float* Dskip, float* state, float* out, int ldo,
                     const int* cu, const int* pos0, const int* slot, int B, int nh, int P, int N, int G,
                     fls_stream_t s);
// softmax scores over E experts; the top largest of (score + corr) chosen (ties: the lower expert);
// ids[T, top], w[T, top] = bare scores; hist[E] += number of entries per expert (hist zeroed by the caller).
// corr == null: the top largest logits are chosen and w = the softmax over the chosen logits only
int fls_seq_moe_route(const float* logits, int ldl, const float* corr, int T, int E, int top, int* ids, float* w,
                      int* hist, fls_stream_t s);
// scores sigmoid(logit); `groups` equal groups of neighbouring experts, each worth the sum of its two largest scores;
// only experts of the `keep` best groups compete (groups <= 1: all); the top largest scores are chosen (ties: the
// lower expert), w = score / (sum of the chosen + 1e-20) * scale; hist as above.  groups <= 64
int fls_seq_moe_route_grouped(const float* logits, int ldl, int T, int E, int top, int groups, int keep, float scale,
                              int* ids, float* w, int* hist, fls_stream_t s);
// offs[E+1] = exclusive scan of hist; cursor[E] = offs[:E]
int fls_seq_moe_scan(const int* hist, int E, int* offs, int* cursor, fls_stream_t s);
// dest[t, k] = a row in its expert's range; rows[dest] = t
int fls_seq_moe_place(const int* ids, int n, int top, int* cursor, int* dest, int* rows, fls_stream_t s);
// out[t] = sum_k w[t, k] y[dest[t, k]] (fp32, k in order)
int fls_seq_moe_sum(const float* y, int ldy, const int* dest, const float* w, float* out, int ldo, int T, int top,
                    int D, fls_stream_t s);
// x[t] += mult * (sum_k w[t, k] y[dest[t, k]] + sigmoid(gate[t * ldg]) shared[t]); shared nullable, gate nullable (then 1)
int fls_seq_moe_combine(float* x, int ldx, const float* y, int ldy, const int* dest, const float* w, int T, int top,
                        const float* shared, int lds, const float* gate, int ldg, int D, float mult, fls_stream_t s);
// ---- several residual streams per row (streams.hip).  xs: fp32 [rows, S D], a row's S streams side by side
// out[t, c * D ...] = table[ids[t]] * scale + pos_table[tok_pos[t]] (pos_table nullable; positions clamped to P - 1), c < copies
int fls_seq_embed_pos(const int* ids, const void* table, int tt, const void* pos_table, const int* tok_pos, float* out, int T,
                      int D, int V, int P, float scale, int copies, fls_stream_t s);
// u = sum_s coef[s] xs[row, s] (coef nullable: the plain sum), y[r] = u / sqrt(mean(u^2) + eps) * w; row = idx ? idx[r] : r
int fls_seq_streams_norm(const float* xs, int ldx, const int* idx, const float* coef, const float* w, void* y, int ty, int ldy,
                         int rows, int D, int S, float eps, fls_stream_t s);
// all streams at once from the old ones: xs[t, r] <- sum_s mix[s, r] xs[t, s] + mult * out[r] * y[t] * sigmoid(gate[t]);
// hc = [in (S) | out (S) | mix (S x S, [from, to])] (nullable: S = 1, out = mix = 1); gate nullable.  h != null: also
// h[t] = the norm above of the NEW streams with coefficients ncoef (nullable) and weight nw, type th
int fls_seq_streams_update(float* xs, int ldx, const float* y, int ldy, const float* gate, int ldg, const float* hc, float mult,
                           int rows, int D, int S, const float* ncoef, const float* nw, void* h, int th, int ldh, float eps,
                           fls_stream_t s);
int fls_seq_scale(float* z, int ldz, int rows, int cols, float alpha, fls_stream_t s);
// y = o * sigmoid(g); o of type to_, y of type ty
int fls_seq_sigmoid_gate(const void* o, int to_, int ldo, const float* g, int ldg, void* y, int ty, int ldy, int rows, int cols,
                         fls_stream_t s);
// a: fp32 [T, 2 H dv], two score maps' outputs (all heads of map 1, then of map 2); per head o = a1 - lambda a2,
// lambda = exp(sum(lam_w[0] lam_w[1])) - exp(sum(lam_w[2] lam_w[3])) + diff (lam_w: [4, d]); out = o / sqrt(mean(o^2) + eps) (1 - diff)
int fls_seq_diff_combine(const float* a, int lda, const float* lam_w, int d, float diff, int H, int dv, float eps, void* out,
                         int to, int ldo, int T, fls_stream_t s);
// HGRN2, per head a state S[d][dv] in state[slot][H][d][dv]: g = lower + (1 - lower) sigmoid(f (+ fb)),
// S_t = diag(g_t) S_(t-1) + (1 - g_t) v_t^T, o_t = S_t^T silu(q_t); raw: fp32 [T, H dv] (row stride ldo), o before its norm.
// q, f: fp32 [T, H d], v: fp32 [T, H dv] with their row strides; fb nullable; d <= 256
int fls_seq_hgrn2_scan(const float* q, int ldq, const float* f, int ldf, const float* v, int ldv, const float* fb,
                       const float* lower, float* state, float* raw, int ldo, const int* cu, const int* pos0,
                       const int* slot, int B, int H, int d, int dv, fls_stream_t s);
#ifdef __cplusplus
}
#endif
