/*
 * msgl_mix.h -- C ABI of the sequence-mixing kernels (latent attention, linear-recurrence layers, routed experts)
 * for gfx950; implemented by libmsgl_mix.so (mini-sglang_amd/csrc/seqmix.hip, mix_delta.hip, mix_par.hip).
 *
 * Same conventions as msgl_hip.h: raw device pointers, explicit sizes and strides in ELEMENTS, `stream` is a
 * hipStream_t passed as void*, every function returns 0 or a negative code and leaves a message for
 * msgl_mix_last_error(); nothing allocates, frees or synchronises, so every call may be captured in a hipGraph.
 * `dtype` is the model dtype T of the tensors that feed matrix products (bf16 or fp32); the residual stream, norms,
 * scores, recurrent state and router are fp32 whatever T is.
 */
#ifndef MSGL_MIX_H_
#define MSGL_MIX_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSGL_MIX_OK 0
#define MSGL_MIX_EINVAL (-1)
#define MSGL_MIX_ELAUNCH (-2)

#define MSGL_MIX_BF16 0
#define MSGL_MIX_F32 2

#define MSGL_MIX_ACT_NONE 0
#define MSGL_MIX_ACT_RELU2 1 /* max(z, 0)^2 */

#define MSGL_MIX_ABI_VERSION 4

const char* msgl_mix_last_error(void);
int msgl_mix_abi_version(void);

/* x32[t] = table[ids[t]] as fp32, h[t] = the same row in T. */
int msgl_mix_embed(float* x32, void* h, const void* table, const int* ids, int tokens, int W, int dtype, void* stream);

/* s = alpha * x_in + sum_p gate[t, p] * y[t, p]   (y: [rows, parts, W] in T or null with parts = 0; gate: fp32 [rows, parts] or
 * null = ones);   out = s / sqrt(mean(s^2) + eps) * (1 + w).  Written to x_out (fp32, may alias x_in) and / or h_out (T).
 * router != null: the normed row (its copy in T) is routed in the same launch -- fp32 logits over E experts, then the selection
 * of msgl_mix_route -> ids int32 [rows, top], wts fp32 [rows, top]. */
int msgl_mix_postnorm(const float* x_in, float* x_out, void* h_out, const void* y, int parts, const float* gate, const void* w,
                      float alpha, float eps, int rows, int W, int dtype, const void* router, const void* bias, int E, int top, int G,
                      int keep, int* ids, float* wts, void* stream);

/* One projection row per token = [q: H x (d + r) | latent R | shared rotated key part r] (the last two only with has_kv).
 * Writes the rotated query parts into q_abs[t, h, R : R + r] (fp32, rows of R + r) and, with has_kv, the RMS-normed latent
 * (plain weight c_norm_w) and the rotated key part into cache[out_loc[t]] (rows of R + r, T).
 * cos_sin: fp32 [positions, rot_dims] = cos | sin halves; entries rot_dims .. r of a rotated part pass unchanged.  Pair i of a
 * rotated part is (i, i + rot_dims / 2), or (2i, 2i + 1) with interleaved != 0. */
int msgl_mix_latent_prep(const void* proj, int64_t ld_proj, float* q_abs, void* cache, const int* out_loc, const int* positions,
                         const float* cos_sin, const void* c_norm_w, float eps, int tokens, int H, int d, int r, int rot_dims, int R,
                         int has_kv, int interleaved, int dtype, void* stream);

/* Causal attention of H heads over ONE shared key row per token: score = q_abs[t, h] . cache[slot] * scale over dk entries,
 * softmax in fp32, out[t, h] = sum_j p_j cache[slot_j][0 : dv] (fp32).  Requests as in the paged backend: table rows of token
 * slots, seq_lens = keys after this forward, cu_q = exclusive prefix of new tokens; prefill portions, single decoded tokens
 * and any mix of them in one launch.
 * bf16 caches run on the matrix cores (Q and the softmax weights rounded to bf16 for the two products, fp32 accumulation and fp32
 * softmax); `splits` > 1 cuts every request's keys into that many ranges whose partial results (workspace: fp32,
 * msgl_mix_latent_attn_workspace_floats) a second launch merges -- for steps with few query rows and many keys.  fp32 caches
 * take the plain fp32 kernel (splits is ignored).
 * sink (fp32 [H], may be null): one more term exp(sink[h]) in head h's softmax denominator, with no key and no value. */
int msgl_mix_latent_attn_workspace_floats(int total_q, int H, int dv, int splits);
int msgl_mix_latent_attn(float* out, const float* q_abs, const void* cache, const int* table, int64_t table_stride, const int* req_rows,
                         const int* seq_lens, const int* cu_q, int batch, int total_q, int H, int dk, int dv, float scale,
                         const float* sink, int dtype, int splits, float* workspace, void* stream);

/* Linear recurrence per (request, head): S <- decay[h] S + k v^T, out = S^T q, with q, k, v = SiLU of the projection row
 * [q: H x d | k: H x d | v: H x dv | ...].  state: fp32 [slots, H, d, dv], row slots[b]; a request whose first new token is at
 * position 0 (seq_lens[b] == its new tokens) starts from zero.  out: fp32 [tokens, H * dv].
 * n_items > 0: the new tokens are cut into chunks that run in parallel -- items[3 i] = (request, first token, end token) with
 * offsets from the request's first new token, every request's chunks in order and covering all its new tokens, item_first[b] ..
 * item_first[b + 1] = the chunks of request b; three launches (every chunk's own state contribution, a scan over the chunks
 * of a request, every chunk's outputs from the state before it); scratch: fp32 [n_items, H, d, dv]. */
int msgl_mix_lightning(float* out, const void* qkv, int64_t ld_qkv, float* state, const float* decay, const int* cu_q, const int* seq_lens,
                       const int* slots, int batch, int H, int d, int dv, int dtype, int n_items, const int* items, const int* item_first,
                       float* scratch, void* stream);

/* out = o / sqrt(mean(o^2) + eps) * w * sigmoid(gate) over rows of N (o fp32, out and gate T). */
int msgl_mix_gated_norm(void* out, const float* o, const void* gate, int64_t ld_gate, const void* w, float eps, int rows, int N, int dtype,
                        void* stream);

/* Router on fp32 logits z [tokens, E] (= router weights x the token, accumulated in fp32 by a product kernel): s = softmax(z);
 * choice = s + bias (bias in T, may be null); only experts of the `keep` best of G equal groups of neighbours (group score = its
 * largest choice) can win; ids = the `top` largest choices, wts = their s / (sum + 1e-20). */
int msgl_mix_route(int* ids, float* wts, const float* z, const void* bias, int tokens, int E, int top, int G, int keep, int dtype,
                   void* stream);

/* seg[E + 1], perm[n]: flat (token, choice) indices bucketed by expert, stable inside a bucket; counts[E] is scratch. */
int msgl_mix_moe_sort(int* seg, int* perm, int* counts, const int* ids, int n, int E, void* stream);

/* C[g] = act(A[g] B[g]^T) with fp32 accumulation; groups advance by *_gs elements.  With seg, group g owns rows
 * seg[g] .. seg[g + 1] of one shared row space of at most M rows (A and C do not advance per group then); a_rows / c_rows
 * make that row space indirect (A row = a_rows[m] / a_div, C row = c_rows[m]).  ta / tb / tc: dtype codes. */
int msgl_mix_gemm_nt(void* C, const void* A, const void* B, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int groups,
                     int64_t a_gs, int64_t b_gs, int64_t c_gs, const int* seg, const int* a_rows, int a_div, const int* c_rows, int act,
                     int ta, int tb, int tc, void* stream);

/* ---- pre-norm hybrid decoders: windowed attention with mixed heads, gated delta-rule layers, depth-averaged stream ---- */

/* x32[t] = table[ids[t]] / sqrt(mean(row^2) + eps) * w  (fp32). */
int msgl_mix_embed_norm(float* x32, const void* table, const int* ids, const void* w, float eps, int tokens, int W, int dtype,
                        void* stream);

/* s = x_in + sum_p gate[t, p] * y[t, p]  (y: [rows, parts, W] in T or null with parts = 0; gate: fp32 or null = ones) -> sum_out
 * (fp32, may be null).  n_mix > 0: the row that goes on is sum_{j < n_mix - 1} mix_w[j] * hist[j * hist_stride + t * W ..] +
 * mix_w[n_mix - 1] * s -> x_out (sum_out may be the next row of hist).  w != null: h_out = row / sqrt(mean(row^2) + eps) * w in T.
 * router != null: the normed row (its copy in T) is routed in the same launch: logits = router row . h + bias, the `top`
 * largest logits win, wts = softmax over the winners' logits. */
int msgl_mix_prenorm(const float* x_in, const void* y, int parts, const float* gate, float* sum_out, const float* hist,
                     int64_t hist_stride, const float* mix_w, int n_mix, float* x_out, const void* w, void* h_out, float eps, int rows,
                     int W, int dtype, const void* router, const void* bias, int E, int top, int* ids, float* wts, void* stream);

/* out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3 over rows of N (powers element-wise, N(.) = the row divided by its root mean
 * square, eps inside the root); coef: 4 floats on the device. */
int msgl_mix_poly_act(void* out, const void* z, int64_t ldz, const float* coef, float eps, int rows, int N, int dtype, void* stream);

/* out[r, i] = silu(gate_up[r, i]) * gate_up[r, N + i]  (rows of 2 N -> rows of N). */
int msgl_mix_silu_mul(void* out, const void* gate_up, int rows, int N, int dtype, void* stream);

/* Router on fp32 logits z [tokens, E] (+ bias in T, may be null): ids = the `top` largest logits (ties: lowest index, in
 * descending order), wts = softmax over those logits only. */
int msgl_mix_route_top(int* ids, float* wts, const float* z, const void* bias, int tokens, int E, int top, int dtype, void* stream);

/* Cache rows of a key/value attention layer: k = src[t, k_off : +nk] -> k_cache[out_loc[t]], v = src[t, v_off : +nv] ->
 * v_cache[out_loc[t]]; with v_first the stored v is (1 - lam) v + lam v_first[t]  (lam: one number in T on the device). */
int msgl_mix_kv_store(void* k_cache, void* v_cache, const int* out_loc, const void* src, int64_t ld_src, int k_off, int v_off, int nk,
                      int nv, const void* v_first, int64_t ld_first, const void* lam, int tokens, int dtype, void* stream);

/* Causal attention over the last `window` keys (0 = all) with the heads' scores mixed before the softmax:
 * s_h(i, j) = scale * sum_g talk[h, g] q_g(i) . k_group(g)(j), softmax over visible j in fp32, o_h = sum_j p_h(j) v_group(h)(j),
 * out[t, h] = o_h * sigmoid(src[t, g_off + h]) in T.  q = src[t, 0 : H d]; cache rows [slots, G d] / [slots, G dv]; requests as in
 * msgl_mix_latent_attn (table rows of token slots, seq_lens = keys after this forward, cu_q = prefix of new tokens).
 * `splits` > 1 cuts every token's visible keys into that many ranges whose partial results (workspace: fp32,
 * msgl_mix_window_attn_workspace_floats) a second launch merges -- for steps with few query tokens. */
int msgl_mix_window_attn_workspace_floats(int total_q, int H, int dv, int splits);
int msgl_mix_window_attn(void* out, const void* src, int64_t ld_src, int g_off, const void* k_cache, const void* v_cache, const int* table,
                         int64_t table_stride, const int* req_rows, const int* seq_lens, const int* cu_q, int batch, int total_q, int H,
                         int G, int d, int dv, int window, float scale, const float* talk, int dtype, int splits, float* workspace,
                         void* stream);

/* Causal convolution over time per channel, then SiLU: out[t, c] = silu(bias[c] + sum_j taps[c, j] in[pos - (n - 1) + j, c]) (fp32;
 * out_t: the same rows in T; either may be null; bias in T, may be null);
 * inputs of this forward are src[t, 0 : C], earlier ones come from state[slots[b]] ([n - 1, C] in T per request: the inputs
 * of the n - 1 positions before the portion), positions before 0 count as zero.  The first `unit_heads` groups of d channels
 * leave as unit vectors (x / sqrt(sum x^2 + 1e-6)), the first `scaled_heads` of them times d^-1/2.  A second launch moves every
 * request's state on to its last n - 1 inputs. */
int msgl_mix_short_conv(float* out, void* out_t, const void* src, int64_t ld_src, const void* taps, const void* bias, void* state, const int* cu_q,
                        const int* seq_lens, const int* slots, int batch, int total, int C, int n, int unit_heads, int scaled_heads, int d,
                        int dtype, void* stream);

/* Gated delta rule per (request, head): S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.  qkv: fp32 rows
 * [q: G x d | k: G x d | v: H x dv] (head h reads q/k group h / (H / G)); state: fp32 [slots, H, d, dv], row slots[b], zero for a
 * request whose first new token is at position 0; beta = sigmoid(b_raw[t, h]); g = exp(rate[h] * softplus(a_raw[t, i] +
 * dt_bias[i])) with i = h (per_channel = 0: one decay per head) or h * d + channel (per_channel = 1: one per row of S);
 * rate = -exp(A_log) in fp32.  out: fp32 [tokens, H * dv].
 * n_items > 0: the new tokens are cut into chunks that run in parallel (items / item_first as in msgl_mix_lightning).  The rule is
 * linear in S, so a chunk is S_end = P S_start + L: one launch computes every chunk's (L | P) by running the rule over dv + d
 * columns from (0 | identity), a scan walks each request's chunks, a third launch computes every chunk's outputs from its start
 * state.  scratch: fp32, n_items * H * d * (2 dv + d) floats. */
int msgl_mix_delta_rule(float* out, const float* qkv, float* state, const void* b_raw, int64_t ld_b, const void* a_raw, int64_t ld_a,
                        int per_channel, const float* rate, const float* dt_bias, const int* cu_q, const int* seq_lens, const int* slots,
                        int batch, int H, int G, int d, int dv, int dtype, int n_items, const int* items, const int* item_first,
                        float* scratch, void* stream);

/* out[t, h, e] = o[t, h, e] / sqrt(mean_e(o[t, h]^2) + eps) * w[e] * act(gate[t, h * dv + e]); act: 0 = sigmoid, 1 = SiLU. */
int msgl_mix_head_gated_norm(void* out, const float* o, const void* gate, int64_t ld_gate, const void* w, float eps, int rows, int H,
                             int dv, int gate_act, int dtype, void* stream);

/* ---- parallel-residual hybrid decoders: token shift, latent attention with a sink, sigmoid attention beside a state-space layer ---- */

/* x32[t] = scale * table[ids[t]] + pair[r]  (fp32).  pair (T, [buckets + 1, W], may be null): r = (previous id * mul_prev + id *
 * mul_cur) mod buckets, r = buckets for a token at position 0; the id before a portion's first token is prev_tok[req_rows[b]]. */
int msgl_mix_embed_scaled(float* x32, const void* table, const void* pair, const int* ids, const int* positions, const int* cu_q,
                          const int* req_rows, int batch, const int* prev_tok, float scale, int buckets, int mul_prev, int mul_cur,
                          int tokens, int W, int dtype, void* stream);

/* row = x_in + bias + v0 * y0 + v1 * y1  (y: T rows ld apart, may be null; v, bias: fp32 [W], null = ones / zeros) -> x_out (fp32,
 * null only without parts; never x_in);  h = row / sqrt(mean(row^2) + eps) * (w + w_off) (w: fp32 [W]) -> h_out (T).  shift (fp32 [W]) !=
 * null:  g = h + (h_prev - h) * shift -> g_out (T) with h_prev the unrounded h of the token before -- of the same launch inside a
 * portion, state[req_rows[b]] (fp32 [rows, W]) for a portion's first token, zero at position 0; the last token of request b
 * leaves its h in staging[b] (fp32 [batch, W]) for msgl_mix_commit_rows. */
int msgl_mix_shift_norm(const float* x_in, float* x_out, const void* y0, int64_t ld0, const float* v0, const void* y1, int64_t ld1,
                        const float* v1, const float* bias, const float* w, float w_off, const float* shift, void* h_out, void* g_out,
                        const float* state, float* staging, const int* positions, const int* cu_q, const int* req_rows, int batch,
                        float eps, int rows, int W, int dtype, void* stream);

/* dst[l * dst_stride + slots[b] * W ..] = src[l * src_stride + b * W ..] for l < layers, b < batch (requests without new tokens
 * are skipped); prev_tok != null: prev_tok[slots[b]] = ids[cu_q[b + 1] - 1]. */
int msgl_mix_commit_rows(float* dst, int64_t dst_stride, const float* src, int64_t src_stride, int layers, const int* slots, int batch, int W,
                         int* prev_tok, const int* ids, const int* cu_q, void* stream);

/* Projection row [q: H x d | k: G x d | v: G x dv | ...] (+ bias: fp32, same layout, may be null): the first rot_dims entries of
 * every q and k head turn (cos_sin and pairing as in msgl_mix_latent_prep), with bit 0 of `unit` every q and k head, with bit 1
 * every v head is divided by its
 * root mean square; q -> q_out (fp32 [tokens, H * d]), k and v -> cache rows at out_loc ([slots, G * d], [slots, G * dv], T). */
int msgl_mix_qk_prep(const void* proj, int64_t ld_proj, const float* bias, float* q_out, void* k_cache, void* v_cache, const int* out_loc,
                     const int* positions, const float* cos_sin, int rot_dims, int interleaved, int unit, float eps, int tokens, int H,
                     int G, int d, int dv, int dtype, void* stream);

/* Causal attention without normalisation over keys: out[t, h] = out_scale * sum_{j <= t} sigmoid(c(scale q_h . k_j) + pb[h]) v_j,
 * c(s) = softcap * tanh(s / softcap) (softcap <= 0: c(s) = s), query head h reads key/value head h / (H / G).  q: fp32 [tokens,
 * H * d]; out: T, rows ld_out apart; requests as in msgl_mix_latent_attn.  `splits` > 1 cuts every request's keys into ranges whose
 * partial sums (workspace: fp32, msgl_mix_sigmoid_attn_workspace_floats) a second launch adds. */
int msgl_mix_sigmoid_attn_workspace_floats(int total_q, int H, int dv, int splits);
int msgl_mix_sigmoid_attn(void* out, int64_t ld_out, const float* q, const void* k_cache, const void* v_cache, const int* table,
                          int64_t table_stride, const int* req_rows, const int* seq_lens, const int* cu_q, int batch, int total_q, int H,
                          int G, int d, int dv, float scale, float softcap, const float* pb, float out_scale, int dtype, int splits,
                          float* workspace, void* stream);

/* State-space recurrence per (request, head): dt = softplus(dt_raw[t, h] + dt_bias[h]); S <- exp(rate[h] dt) S + dt B x^T;
 * y = S^T C + D[h] x.  xbc: fp32 rows [x: H x P | B: G x N | C: G x N] (head h reads group h / (H / G)); dt_raw: T rows ld_dt
 * apart; state: fp32 [slots, H, N, P], row slots[b], zero for a request whose first new token is at position 0; rate = -exp(A_log).
 * out: fp32 [tokens, H * P].  n_items > 0: chunks as in msgl_mix_lightning (a chunk is S_end = exp(rate * sum dt) S_start + L);
 * scratch: fp32, n_items * H * (N * P + 1) floats. */
int msgl_mix_ssd(float* out, const float* xbc, int64_t ld_x, const void* dt_raw, int64_t ld_dt, float* state, const float* rate,
                 const float* dt_bias, const float* D, const int* cu_q, const int* seq_lens, const int* slots, int batch, int H, int G, int N,
                 int P, int dtype, int n_items, const int* items, const int* item_first, float* scratch, void* stream);

/* v = y * silu(z) (y fp32 [rows, N], z T rows ld_z apart); every one of `groups` equal parts of a row is divided by its own root
 * mean square; out = v * w * out_scale (w fp32 [N]; out T, rows ld_out apart). */
int msgl_mix_gate_group_norm(void* out, int64_t ld_out, const float* y, const void* z, int64_t ld_z, const float* w, float eps, int rows,
                             int N, int groups, float out_scale, int dtype, void* stream);

/* out = z > 0 ? a z^2 + z / 2 : b (exp(z) - 1 - z) + z / 2 with a = softplus(pq[0]), b = 1/2 + softplus(pq[1]) (pq: 2 floats on the
 * device); z rows ldz apart, out rows of N. */
int msgl_mix_xielu(void* out, const void* z, int64_t ldz, const float* pq, int rows, int N, int dtype, void* stream);

/* ---- looped pre-norm hybrid decoders (csrc/mix_scan.hip) ---- */

/* Closes a sublayer and opens the next.  row = x_in + mult * (sum of the p0 rows of y0[t] and the p1 rows of y1[t]) + add -> x_out
 * (fp32, a buffer other than x_in; y0 [rows, p0, W], y1 [rows, p1, W] in T, add fp32 [W]; each may be absent);  h = row with every
 * one of `groups` equal parts divided by its own root mean square (eps inside the root), times w (T [W]);  h_out[t] (T) = h[t] +
 * sum_j taps[c, j] h[t - (n - 1) + j] (taps T [W, n], null: h itself).  With n > 1 the rows are the new tokens of `batch` requests
 * (cu_q, seq_lens as in msgl_mix_latent_attn): rows before a portion come from state[slots[b]] (fp32 [n - 1, W] per request: the h
 * of the n - 1 positions before the portion), rows before position 0 are zero, and every request's new state rows are left in
 * staging[b] (fp32 [batch, n - 1, W]) for msgl_mix_commit_rows.  cu_q null: plain rows (n must be 1). */
int msgl_mix_norm_conv(const float* x_in, float* x_out, const void* y0, int p0, const void* y1, int p1, float mult, const float* add,
                       const void* w, int groups, float eps, const void* taps, int n, const float* state, float* staging, void* h_out,
                       const int* cu_q, const int* seq_lens, const int* slots, int batch, int rows, int W, int dtype, void* stream);

/* Selective scan per (request, channel c): dt = softplus(dt_in[t, c] + dt_bias[c]); S[c, n] <- exp(dt A[c, n]) S[c, n] + dt x[t, c]
 * B[t, n]; y = sum_n S[c, n] C[t, n] + D[c] x[t, c]; out[t, c] = y silu(z[t, c]).  x, z, dt_in: T rows of C channels (row strides
 * given); bc: T rows [B: N | C: N]; A = -exp(A_log) fp32 [C, N]; state: fp32 [slots, C, N], row slots[b], zero for a request whose
 * first new token is at position 0; out: T [tokens, C].  n_items > 0: chunks as in msgl_mix_lightning (over a chunk S_end =
 * exp(A sum dt) S_start + L); scratch: fp32, n_items * C * (N + 1) floats. */
int msgl_mix_selective_scan(void* out, const void* x, int64_t ld_x, const void* z, int64_t ld_z, const void* dt_in, int64_t ld_dt,
                            const void* bc, int64_t ld_bc, const float* A, const float* dt_bias, const float* D, float* state,
                            const int* cu_q, const int* seq_lens, const int* slots, int batch, int C, int N, int dtype, int n_items,
                            const int* items, const int* item_first, float* scratch, void* stream);

/* Softmax attention over the last `window` keys (window <= 0: all earlier keys) with a sink: out[t, h] = sum_j p_j v_j, p_j =
 * exp(s_j) / (sum over visible keys of exp(s) + exp(sink[h])), s_j = scale q_h . k_j; sink fp32 [H] or null.  Query head h reads
 * key/value head h / (H / G).  q: fp32 [tokens, H * d]; caches and requests as in msgl_mix_sigmoid_attn; `splits` > 1 cuts the
 * visible keys into ranges joined by a second launch (workspace: fp32, msgl_mix_sink_attn_workspace_floats). */
int msgl_mix_sink_attn_workspace_floats(int total_q, int H, int dv, int splits);
int msgl_mix_sink_attn(void* out, int64_t ld_out, const float* q, const void* k_cache, const void* v_cache, const int* table,
                       int64_t table_stride, const int* req_rows, const int* seq_lens, const int* cu_q, int batch, int total_q, int H, int G,
                       int d, int dv, float scale, int window, const float* sink, int dtype, int splits, float* workspace, void* stream);

/* Router on fp32 logits z [tokens, E]: the `top` largest win (ties: lowest index), the weight of a choice is sigmoid(its logit)
 * -> ids int32 [tokens, top], wts fp32 [tokens, top]. */
int msgl_mix_route_sigmoid(int* ids, float* wts, const float* z, int tokens, int E, int top, void* stream);

/* out[t * top + k, :] = wts[t, k] * h[t, :] (T rows of W): the inputs of experts that are weighted before they run. */
int msgl_mix_scale_rows(void* out, const void* h, const float* wts, int tokens, int top, int W, int dtype, void* stream);

/* The three steps above in one launch, a workgroup per token (for steps with few tokens): z = router h (router T [E, W], fp32
 * accumulation), the `top` largest, out[t * top + k, :] = sigmoid(z of choice k) * h[t, :]; ids, wts as above. */
int msgl_mix_route_scale(int* ids, float* wts, void* out, const void* h, const void* router, int tokens, int E, int top, int W, int dtype,
                         void* stream);

/* out (T [rows, N]) = o (fp32 [rows, N]) * sigmoid(g) (T rows ld_g apart). */
int msgl_mix_sigmoid_gate(void* out, const float* o, const void* g, int64_t ld_g, int rows, int N, int dtype, void* stream);

/* x <- cap * tanh(x / cap) in place (T rows of N, ld apart). */
int msgl_mix_softcap(void* x, int64_t ld, int rows, int N, float cap, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif
