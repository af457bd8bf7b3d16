// The C interface of the kernel library. Pointers are device pointers unless named
// host; sizes are in elements; `dtype` is HFA_F32 (0) or HFA_BF16 (1). Every function
// returns 0 on success; otherwise hfa_last_error() describes what was refused.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char* hfa_last_error(void);
int hfa_version(void);

// x[t, :] = table[tokens[t], :] as fp32.  (reference: src/model.c:566-571)
int hfa_embed(const void* table, int table_dtype, const int* tokens, float* x, int n_tokens, int width,
              int vocab, hipStream_t stream);

// out[r, :] = x[rows ? rows[r] : r, :] * rsqrt(mean(x^2) + eps) * w.  (src/mathx.c:65-75)
// With splits > 0 (and no rows): first x[r, :] += sum_s partial[s][r][:] + partial_bias, written
// back: the residual sum of a matrix product that hfa_gemm deferred (src/model.c:609, 623).
int hfa_rmsnorm(float* x, const float* w, void* out, int out_dtype, const int* rows, int n_rows, int width,
                float eps, const float* partial, int splits, const float* partial_bias, hipStream_t stream);

// out[m, n] (+)= sum_k a[m, k] * w[n, k] + bias[n].  a: [M, K] row stride lda; w: [N, K] row
// stride ldw; out row stride ldo. `accumulate` adds into fp32 `out` (the residual sum).
// bf16 operands with K and the row strides multiples of 8 run on the matrix cores (K split over
// `workspace` for small M); everything else, and everything when `force_plain`, runs the plain
// fp32 multiply-add kernel. `epilogue` 1 (matrix cores only): the columns of w come in blocks of
// 32 gate rows, 32 up rows, and out[m, f] = silu(gate) * up has N / 2 columns (src/model.c:537).
// `epilogue` 1 + k (k = HFA_ACT_GELU_ERF, HFA_ACT_GELU_TANH or HFA_ACT_RELU2; not with `accumulate`, never deferred):
// out[m, n] = act_k(sum + bias[n]), the activation computed in fp32 in the product's last lines (on the plain path by
// the elementwise kernel after it).
// `defer`: if K was split, leave the partial sums ([splits][M][N] fp32 at the start of the
// workspace) for the caller's next kernel and report the number of splits in *pending_splits.
// (src/model.c:408-424)
int hfa_gemm(const void* a, int a_dtype, int lda, const void* w, int w_dtype, int ldw, const float* bias,
             void* out, int out_dtype, int ldo, int accumulate, int epilogue, int M, int N, int K,
             void* workspace, size_t workspace_bytes, int defer, int* pending_splits, int force_plain,
             hipStream_t stream);
int hfa_gemm_finish(const void* partial, int splits, const float* bias, void* out, int out_dtype, int ldo,
                    int accumulate, int epilogue, int M, int N, hipStream_t stream);

// The product for up to 32 rows in which every block owns a range of outputs and finishes them itself (bf16
// operands, K a multiple of 128; see gemm_rows.hip), with what follows a product in a decode step in its last lines:
//   HFA_ROWS_OUT     out[m, n] = act(r[m] * sum + bias[n]), fp32 or bf16 (out_dtype); act = out_act (HFA_ACT_*, 0: none)
//   HFA_ROWS_RESID   x[m, n] += sum + bias[n] (fp32, in place); ssq_out[b][m] = block b's share of sum_n x[m, n]^2
//                    ([hfa_gemm_rows_parts()][16] floats, [..][32] from 17 rows up: give room for 32); xg[m, n] = bf16(x[m, n] * g[n]) if xg is given
//   HFA_ROWS_SWIGLU  act[m, f] = bf16(silu(r[m] * sum_gate) * (r[m] * sum_up)), N features, w's 2 N rows in blocks of
//                    32 gate rows, 32 up rows (src/model.c:537)
// r[m] = rsqrt(sum over the parts_in shares ssq_in[.][m] * inv_width + eps), or 1 without ssq_in: the RMS norm of the
// tensor whose product with the norm's weight is `a` (src/mathx.c:65-75), applied to the sums instead of the operand.
// hfa_gemm_rows_supports says whether a shape is taken (1 to 32 rows, K a multiple of 128, strides multiples of 8).
// ssq_in has the layout that a HFA_ROWS_RESID product of the same number of rows left.
#define HFA_ROWS_OUT 0
#define HFA_ROWS_RESID 1
#define HFA_ROWS_SWIGLU 2
int hfa_gemm_rows_parts(void);
int hfa_gemm_rows_supports(int mode, int M, int N, int K, int lda, int ldw);
int hfa_gemm_rows(int mode, const void* a, int lda, const void* w, int ldw, int M, int N, int K, const float* bias,
                  const float* ssq_in, int parts_in, float inv_width, float eps, void* out, int ldo, int out_dtype,
                  int out_act, float* x, int ldx, float* ssq_out, const float* g, void* xg, int ldxg, void* act, int ldact,
                  hipStream_t stream);

// Rotary position encoding on the q (and k) heads inside qkv rows [q | k | v], split-half
// pairing, and the store of k (rotated) and v into cache rows slot_map[t] (src/model.c:468-493,
// 587-600). rot_dim 0: no rotation. n_kv_heads 0: the rows hold q only, nothing is stored.
// Query and key heads have head_dim values, value heads v_head_dim (the same in most models; a
// prompt-sized bf16 call with equal sizes takes a kernel of its own).
// Cache layout: row r = page * page_tokens + offset. Keys: k_cache[r * width + c], width =
// n_kv_heads * head_dim. Values (width n_kv_heads * v_head_dim) lie transposed inside their page, so that
// the keys of one value column are contiguous: v_cache[page * page_tokens * width + c * page_tokens + offset].
// With splits > 0 the input is not qkv but the partial sums of a deferred hfa_gemm
// ([splits][n_tokens][(n_heads + 2 n_kv_heads) * head_dim] fp32) plus partial_bias; the rotated
// queries are written into qkv.
int hfa_rope_store(void* qkv, int dtype, int ld, const int* positions, const float* inv_freq, int rot_dim,
                   int n_heads, int n_kv_heads, int head_dim, int v_head_dim, void* k_cache, void* v_cache,
                   const int* slot_map, int page_tokens, int n_tokens, const float* partial, int splits,
                   const float* partial_bias, hipStream_t stream);

// `run` (a request's tokens in one call) from which hfa_paged_attention takes the kernel for prompt
// portions for the whole call; see the launcher in attention_mfma.hip.
int hfa_attention_prompt_rows(void);

// Softmax attention of each token's query heads over its request's cached keys and values
// (src/model.c:499-528). Key j of the request in slot s lies in cache row
// block_table[s, j / page_tokens] * page_tokens + j % page_tokens. A key is visible to the
// query at position p iff j <= p and (window == 0 or p - j < window) and (mask_chunk == 0 or
// j / mask_chunk == p / mask_chunk: a mask by runs of mask_chunk positions counted from 0). q_start[n_seqs + 1] gives
// each request's run of tokens (consecutive positions of one slot); max_q_len and max_seq_len
// bound the runs and the positions. Key rows are kv_width wide with head_dim values a head, value rows
// v_width with v_head_dim a head; out has v_head_dim values per query head. bf16 with one head size for
// both that is a multiple of 32, page_tokens a power of two from 4
// and at most 32 query heads per key/value head runs on the matrix cores, the key range
// split over `workspace` when there are few queries; everything else, and everything when
// `force_plain`, runs the plain kernel. `slopes` (one fp32 per query head, or null) is the hook for a position
// encoding that enters the scores rather than the queries and keys: the score of key j for the query at p
// becomes dot * scale + slopes[h] * (j - p); with slopes the plain kernel runs. `sink` 1: the softmax has one more term
// of score 0 that has no value, p_j = exp(s_j) / (1 + sum_i exp(s_i)) (every kernel takes it). `cross_values` 1: every
// head's weights are applied to the values of every key/value group: out is [token][G rounds][H heads][v_head_dim], round r
// of head h being its weights on the values of group (h's group + r) mod G (see hfa_talk_mix; on the matrix cores one pass a round).
// `softcap` > 0: score <- softcap tanh(score / softcap) before the weights are formed. `weights` 0: softmax; 1: no softmax, a
// visible key weighs sigmoid(score + head_bias[h]) (head_bias: one fp32 per query head, or null), not normalised over the keys.
// Sigmoid weights (with or without a cap) run on the matrix cores under the same conditions as the softmax; a cap under a softmax goes the plain way.
int hfa_paged_attention(const void* q, int dtype, int ldq, const void* k_cache, const void* v_cache,
                        int kv_width, int v_width, const int* block_table, int max_blocks, const int* token_slot,
                        const int* positions, const int* q_start, int n_seqs, int max_q_len, int max_seq_len,
                        void* out, int ldo, int n_tokens, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                        int page_tokens, int window, int mask_chunk, float scale, const float* slopes, int sink, int cross_values,
                        float softcap, int weights, const float* head_bias,
                        void* workspace, size_t workspace_bytes, int force_plain, hipStream_t stream);

// Decoded tokens (one a request) whose queries, new keys and new values are still the 32-bit rows [q | k | v] that
// the product left (`raw`, bias added): rotation of queries and keys (cos_sin: hfa_rope_table's output for the step's
// tokens, [token][head_dim / 2 cosines, head_dim / 2 sines]; null: none), the store of the new key and value into
// cache rows slot_map[t], and attention over the cache, in one kernel (plus the merge of key chunks): what
// hfa_rope_store and hfa_paged_attention give one after the other. With slot_map null the rows are [q] only and nothing
// is stored (a layer that reads keys and values which another layer stored in this step). bf16 cache, matrix cores only: ask
// hfa_decode_attention_supports first.
int hfa_rope_table(const int* positions, const float* inv_freq, int half, float* out, int n_tokens, hipStream_t stream);
int hfa_decode_attention_supports(int n_heads, int n_kv_heads, int head_dim, int rot_dim, int page_tokens, int kv_width,
                                  int ld_raw, int ldo);
int hfa_decode_attention(const float* raw, int ld_raw, const float* cos_sin, void* k_cache, void* v_cache, int kv_width,
                         const int* slot_map, const int* block_table, int max_blocks, const int* token_slot,
                         const int* positions, const int* q_start, int n_seqs, int max_seq_len, void* out, int ldo,
                         int n_heads, int n_kv_heads, int head_dim, int page_tokens, int window, int mask_chunk, float scale,
                         void* workspace, size_t workspace_bytes, hipStream_t stream);

// Layer norm: out[r, :] = (x[rows ? rows[r] : r, :] - mean) / sqrt(var + eps) * w + b (b null: no shift), var the mean
// squared deviation, all in fp32. With splits > 0 (and no rows) a deferred product's partial sums
// ([splits][x_rows][width]) and partial_bias are first added into x, as in hfa_rmsnorm.
int hfa_layernorm(float* x, const float* w, const float* b, void* out, int out_dtype, const int* rows, int n_rows,
                  int width, float eps, const float* partial, int splits, const float* partial_bias, int x_rows,
                  hipStream_t stream);

// RMS norm in groups: a row of `width` values is cut into `groups` equal runs, each divided by sqrt(mean(run^2) + eps),
// the whole times w; x and out fp32 or bf16, sums in fp32. rows: out[r] = norm(x[rows[r]]). gate_kind 1: the row is
// multiplied by silu(gate[r]) before the norm; 2: the result is multiplied by sigmoid(gate[r]), 3: by silu(gate[r]) (no rows then). row_scale
// (null: none; fp32 [n_rows, groups], rows in order): run g of row r is multiplied by row_scale[r, g] before everything else.
int hfa_group_rmsnorm(const void* x, int x_dtype, int ldx, const float* w, void* out, int out_dtype, int ldo, const int* rows,
                      int n_rows, int width, int groups, float eps, const void* gate, int gate_dtype, int ldg, int gate_kind,
                      const float* row_scale, hipStream_t stream);

// Rows [q: H D | k: G D | v: G Dv] of a step: optional RMS norm of the whole q part and of the whole k part (weights
// q_norm_w, k_norm_w, eps), rotation of the first rot_dim dimensions of each q and k head (pairing 0: i with i + rot_dim / 2,
// 1: 2 i with 2 i + 1), optional v <- (1 - *v_blend) v + *v_blend v_other[t] (v_other [T, G Dv]); v_keep [T, G Dv] receives
// the values as projected. q goes back into the row, k and v into cache rows slot_map[t] (or the row, if null).
int hfa_qkv_prepare(void* qkv, int dtype, int ld, const int* positions, const float* inv_freq, int rot_dim, int pairing,
                    int n_heads, int n_kv_heads, int head_dim, int v_head_dim, const float* q_norm_w, const float* k_norm_w,
                    float eps, const float* v_blend, const void* v_other, void* v_keep, void* k_cache, void* v_cache,
                    const int* slot_map, int page_tokens, int n_tokens, hipStream_t stream);

// Mixers with per-request state (recurrent.hip). A request's tokens of a step are rows q_start[s] .. q_start[s + 1] - 1;
// its state is row seq_slot[s] of `state` (fp32, state_ld floats a row).
// hfa_causal_conv: out[t, c] = act(bias[c] + sum_j taps[c, j] in[t - (K - 1) + j, c]) (fp32 out; act HFA_ACT_SILU or none);
// inputs before the step's first token come from the state row ([K - 1][C], oldest first), which then receives the
// step's last K - 1 inputs.
// hfa_linear_scan: per head h (keys and queries of head h / (n_heads / qk_heads)), S [qk_dim][v_dim] in the state row (in the
// kernel's own order, padded: hfa_linear_scan_state_floats values a row, zero for a new request; qk_dim at most 256):
// S <- a_t S + k_t (b_t v_t)^T, y_t = S^T q_t + skip[h] v_t (skip null: 0). gate 0: a_t = decay[h], b_t = 1. gate 1:
// dt = softplus(step[t, h] + step_bias[h]), a_t = exp(-exp(a_log[h]) dt), b_t = dt. y fp32. gate 2: exponential gates under a
// running maximum m (kept beside the states): li = cap tanh((step + step_bias) / cap), lf = logsigmoid(cap tanh((step2 +
// step_bias2) / cap)), m_t = max(lf + m, li), a_t = exp(lf + m - m_t), b_t = exp(li - m_t); the state has one more column that
// holds n_t = a_t n + b_t k_t, and denom[t, h] = 1 / (max(|n_t . q_t|, exp(-m_t)) + 1e-6) leaves beside y (which is not divided).
// A state row then holds hfa_linear_scan_state_floats(heads, qk_dim, v_dim + 1) + hfa_linear_scan_max_floats(...) values.
// q_scale multiplies the queries.
// hfa_delta_scan: the gated delta rule on fp32 inputs, S in hfa_linear_scan's layout: g_t[n] = exp(-exp(a_log[h]) softplus(a[t,
// h N + n] + dt_bias[h N + n])), S <- g_t * S (row by row), u = sigmoid(b[t, h]) (v_t - S^T k_t), S <- S + k_t u^T, y_t = S^T q_t,
// with k_t, q_t first divided by sqrt(sum of squares + unit_eps) and q_t multiplied by q_scale. max_q_len: the most tokens of a
// request (an upper bound will do; it only chooses between a walk for prompt portions and one for single tokens).
int hfa_causal_conv(const void* in, int dtype, int ld_in, const float* taps, const float* bias, int n_channels, int n_taps,
                    float* state, size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs, int max_q_len, float* out,
                    int ldo, int act, hipStream_t stream);
size_t hfa_linear_scan_state_floats(int n_heads, int qk_dim, int v_dim);
int hfa_linear_scan(const void* q, int ldq, const void* k, int ldk, int qk_heads, int qk_dim, const void* v, int ldv, int n_heads,
                    int v_dim, int dtype, int gate, const float* decay, const void* step, int step_dtype, int ld_step,
                    const float* step_bias, const float* a_log, const float* skip, float* state, size_t state_ld,
                    const int* q_start, const int* seq_slot, int n_seqs, float* y, int ldy, const void* step2,
                    const float* step_bias2, float cap, float q_scale, float* denom, hipStream_t stream);
size_t hfa_linear_scan_max_floats(int n_heads, int qk_dim, int v_dim);
int hfa_delta_scan(const float* q, int ldq, const float* k, int ldk, int qk_heads, int qk_dim, const float* v, int ldv, int n_heads,
                   int v_dim, const float* a, int lda, const float* dt_bias, const float* a_log, const float* b, int ldb,
                   float q_scale, float unit_eps, float* state, size_t state_ld, const int* q_start, const int* seq_slot,
                   int n_seqs, int max_q_len, float* y, int ldy, hipStream_t stream);

// Layers that norm a branch's result before it joins the stream, and what comes with them (sandwich.hip).
// hfa_embed_pos: x[t] = table[tokens[t]] * scale + pos(positions[t]), pos[2i] = sin(p inv_freq[i]), pos[2i + 1] = cos(p inv_freq[i])
// (positions null: no position vector).
// hfa_rmsnorm_add: v = y[r] * sigmoid(gate[r] + gate_bias) (gate null: v = y[r]); out[r] (+)= scale * v / sqrt(mean(v^2) + eps) * w.
// hfa_polynorm: out = coef[0] N(z) + coef[1] N(z^2) + coef[2] N(z^3) + coef[3], N(u) = u / sqrt(mean(u^2) + eps) over a row.
// hfa_scale_rows: x *= s. hfa_head_norm_store: rows [q | k | v]; q and k heads RMS-normed with a weight of one head's size (null:
// as they are), q to q_out, k and v to cache rows slot_map[t] (values transposed inside their page).
// hfa_talk_mix: out[t, h] = sigmoid(gate[t, h]) * sum_g talk[h, g] cross[t, (c(h) - c(g)) mod G, g], cross from hfa_paged_attention
// with cross_values.
int hfa_embed_pos(const void* table, int table_dtype, const int* tokens, const int* positions, const float* inv_freq, float* x,
                  int n_tokens, int width, int vocab, float scale, hipStream_t stream);
int hfa_rmsnorm_add(const float* y, int ldy, const void* gate, int gate_dtype, int ldg, const float* gate_bias, const float* w,
                    float* out, int ldo, int n_rows, int width, float eps, float scale, int accumulate, hipStream_t stream);
int hfa_polynorm(const void* z, int z_dtype, int ldz, const float* coef, void* out, int out_dtype, int ldo, int n_rows, int width,
                 float eps, hipStream_t stream);
int hfa_scale_rows(float* x, int ld, int n_rows, int width, float s, hipStream_t stream);
int hfa_head_norm_store(const void* qkv, int in_dtype, int ld, int n_heads, int n_kv_heads, int head_dim, int v_head_dim,
                        const float* q_w, const float* k_w, float eps, void* q_out, int ldq, void* k_cache, void* v_cache,
                        int out_dtype, const int* slot_map, int page_tokens, int n_tokens, hipStream_t stream);
int hfa_talk_mix(const void* cross, int cross_dtype, const float* talk, const void* gate, int gate_dtype, int ldg, void* out,
                 int out_dtype, int ldo, int n_tokens, int n_heads, int n_kv_heads, int v_head_dim, hipStream_t stream);

// hfa_scale_add: out[r, c] (+)= scale * col[c] * y[r, c] in fp32 (col null: 1). hfa_gate_mul: out = x * act(gate) element by
// element, formed in fp32; act is HFA_ACT_SIGMOID or HFA_ACT_SILU.
int hfa_scale_add(const float* y, int ldy, const float* col, float scale, float* out, int ldo, int n_rows, int width,
                  int accumulate, hipStream_t stream);
int hfa_gate_mul(const void* x, int x_dtype, int ldx, const void* gate, int gate_dtype, int ldg, void* out, int out_dtype,
                 int ldo, int n_rows, int width, int act, hipStream_t stream);

// Attention through latents (latent.hip). hfa_latent_pack lays a step's rows out for hfa_rope_store and hfa_paged_attention with one
// key/value head whose key is [rotated part: R | latent: C] and whose value is the latent: from `down` ([T, >= C + R] fp32: the
// latent before its norm, then the rotated key part) and `q` ([T, H (D + R)], head by head [D unrotated | R to be rotated]) it
// writes packed[t] = [H heads of (R | C: left alone) | R | C | C]: the queries' parts to be rotated, the key's part to be rotated,
// and the latent c = down[:C] / sqrt(mean(down[:C]^2) + eps) * w twice (as the key's rest and as the value). Sums in fp32.
// `folded` ([T, H C] of q's type, or null): the heads' C parts are copied from there (else they are left alone).
int hfa_latent_pack(const float* down, int ld_down, const void* q, int q_dtype, int ldq, const float* w, float eps, void* packed,
                    int out_dtype, int ld_packed, int n_tokens, int n_heads, int dim, int rot, int latent, const void* folded,
                    int ld_folded, hipStream_t stream);

// hfa_channel_scan (recurrent.hip): per head, S [qk_dim][v_dim] in hfa_linear_scan's layout: S <- diag(a_t) S + k_t v_t^T, y_t = S^T
// (q_scale q_t), with a decay per key channel a_t = decay[t, h qk_dim + n] (fp32); kcomp 1: k_t = 1 - a_t (k is not read), else k_t
// is read from k. q_act HFA_ACT_SILU: the queries pass silu first (0: as they are). hfa_channel_decay forms the decays in fp32 from
// x = z[r, c] + bias[c] (bias null: 0): form 0: a = lower[c] + (1 - lower[c]) sigmoid(x); form 1: a = sigmoid(x)^inv_tau =
// exp(inv_tau logsigmoid(x)).
int hfa_channel_decay(const void* z, int z_dtype, int ldz, const float* bias, int form, const float* lower, float inv_tau,
                      float* out, int ldo, int n_rows, int width, hipStream_t stream);
int hfa_channel_scan(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype, const float* decay,
                     int ld_decay, int kcomp, int q_act, int n_heads, int qk_dim, int v_dim, float q_scale, float* state,
                     size_t state_ld, const int* q_start, const int* seq_slot, int n_seqs, float* y, int ldy, hipStream_t stream);

// out[r, c] = act(in[r, c]) for rows of `width` values with strides ldi and ldo, computed in fp32:
// the exact gelu 0.5 z (1 + erf(z / sqrt 2)), its tanh form, relu(z)^2, silu or the logistic function.
#ifndef HFA_ACT_GELU_ERF
#define HFA_ACT_NONE 0
#define HFA_ACT_GELU_ERF 1
#define HFA_ACT_GELU_TANH 2
#define HFA_ACT_RELU2 3
#define HFA_ACT_SILU 4
#define HFA_ACT_SIGMOID 5
#define HFA_ACT_LAST 5
#endif
int hfa_activation(const void* in, int ldi, void* out, int ldo, int dtype, int n_rows, int width, int kind,
                   hipStream_t stream);

// x <- cap * tanh(x / cap) on fp32 rows, in place (logits that a model squashes).
int hfa_softcap(float* x, int ld, int n_rows, int width, float cap, hipStream_t stream);

// Mixture of experts (moe.hip). hfa_moe_route: fp32 router logits [n_tokens, n_experts] -> ids and weights
// [n_tokens, top]; scoring 0 = softmax over all experts, 1 = logistic per expert, 2 = exp(logit - largest logit) (with renorm:
// the softmax over the chosen logits alone); experts form n_groups equal runs of
// neighbours of which the `keep` best (by their best expert) may be chosen from; weights = score (/ sum of the chosen
// + 1e-20 if renorm) * out_scale. hfa_moe_plan puts the n_pairs = n_tokens * top pairs in expert order (row_pair) and
// lists tiles of at most tile_rows rows of one expert (tiles: 3 ints a tile, room for n_pairs / tile_rows + n_experts;
// *n_tiles on the device). hfa_moe_gemm: for every row r of the plan, out[o(r), :] = act(a[s(r), :] . w[e(r)]^T)
// (* pair_scale[pair] if given); w is [n_experts][N][K] (bf16, or fp32 beside activations of either type); s(r) = row_pair[r] / a_div if a_div > 0 else r; o(r) =
// row_pair[r] if out_by_pair else r. tile_rows must be what hfa_moe_tile_rows gave for the plan.
// hfa_moe_combine: x[t, :] += sum_k y[t * top + k, :]. `gated` 1 (N a multiple of 64, act 0): w's rows come in blocks of 32 gate rows
// and 32 up rows, out has N / 2 columns, and with c = pair_scale of the row's pair (null: 1), g = min(c gate, limit), u = clamp(c up,
// -limit, limit) (limit <= 0: unbounded): out = g sigmoid(alpha g) (u + shift), formed from the 32-bit sums in the product's last lines.
int hfa_moe_route(const float* logits, int ld, int n_tokens, int n_experts, int top, int n_groups, int keep,
                  int scoring, int renorm, float out_scale, int* ids, float* weights, hipStream_t stream);
int hfa_moe_plan(const int* ids, int n_pairs, int n_experts, int tile_rows, int* row_pair, int* tiles, int* n_tiles,
                 hipStream_t stream);
int hfa_moe_tile_rows(int dtype, int w_dtype, int n_pairs, int n_experts, int N, int K);
int hfa_moe_gemm(const void* a, int lda, int dtype, int a_div, const void* w, int w_dtype, const int* row_pair, const int* tiles,
                 const int* n_tiles, int max_tiles, int tile_rows, void* out, int ldo, int out_dtype, int out_by_pair,
                 const float* pair_scale, int act, int N, int K, int force_plain, int gated, float gate_alpha, float gate_limit,
                 float gate_shift, hipStream_t stream);
int hfa_moe_combine(const float* y, float* x, int n_tokens, int top, int width, hipStream_t stream);
// Gated experts: row r of the expert-ordered rows holds [gate: F | up: F] fp32 sums; with c = pair_scale[row_pair[r]]
// (null: 1), g = min(c gate, limit), u = clamp(c up, -limit, limit) (limit <= 0: unbounded): out[r, f] = g sigmoid(alpha g) (u + shift).
// `interleaved`: the row holds blocks of 32 gate sums and 32 up sums instead.
int hfa_moe_gated_act(const float* gu, int ld, const int* row_pair, const float* pair_scale, void* out, int out_dtype, int ldo,
                      int n_rows, int F, float alpha, float limit, float shift, int interleaved, hipStream_t stream);

// out[t, i] = silu(gate_up[t, i]) * gate_up[t, width + i].  (src/model.c:532-538)
int hfa_swiglu(const void* gate_up, void* out, int dtype, int n_tokens, int width, hipStream_t stream);

// dst[idx[i]] = val[i]
int hfa_scatter_i32(int* dst, const int* idx, const int* val, int n, hipStream_t stream);

// dst[dst_idx[i]] = src[src_idx[i]] (tokens sampled on the device go into the next step's inputs)
int hfa_move_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n, hipStream_t stream);

// out[r] = first index of the maximum of logits[r, :].  (src/sample.c:72-77)
// `workspace` holds the candidates of the first of its two stages (n_rows * 64 * 8 bytes).
int hfa_argmax(const float* logits, int ld, int* out, int n_rows, int vocab, void* workspace,
               size_t workspace_bytes, hipStream_t stream);

// hfa_argmax for callers that cannot allocate or bring a workspace: code under HIP graph capture,
// tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. The
// candidates of the first stage lie in a device array that the library holds itself (128 KiB on every
// GPU it runs on, until the process ends), so the call allocates nothing; the caller still passes
// logits and out. At most HFA_ARGMAX_STATIC_ROWS rows; more are refused. Calls that overlap on one
// GPU share that array and race; nothing needs clearing between calls that follow each other.
// The first call on a device asks the runtime for the array's address there, which is no stream
// operation: it must be an eager call (one made while the stream is being captured is refused with
// a message that says so); every later call on that device may be captured.
#define HFA_ARGMAX_STATIC_ROWS 256
int hfa_argmax_static(const float* logits, int ld, int* out, int n_rows, int vocab, hipStream_t stream);

// All candidates of the chosen rows (rows[i], or row i if rows is null) in the order (logit
// descending, id ascending), as the reference's sort leaves them when top-k is off
// (src/sample.c:59-64, 93-98): ids and vals are [n_rows, vocab]. `scratch` needs
// hfa_order_rows_scratch(n_rows, vocab) bytes, 8-byte aligned.
size_t hfa_order_rows_scratch(int n_rows, int vocab);
int hfa_order_rows(const float* logits, int ld, const int* rows, int* ids, float* vals, int n_rows, int vocab,
                   void* scratch, size_t scratch_bytes, hipStream_t stream);

// The draw over ordered rows (src/sample.c:99-114): vals/ids [n_rows, vocab] as hfa_order_rows leaves them,
// params[r] = {temp, top_p, min_p, u} with u the request's uniform number in [0, 1), cuts[r] = candidates
// left by top-k (1..vocab). tokens[r] = the drawn id. vals is overwritten with the probabilities.
int hfa_draw_rows(float* vals, const int* ids, int n_rows, int vocab, const float* params, const int* cuts,
                  int* tokens, hipStream_t stream);

// The k best of each row in the order (logit descending, id ascending) (src/sample.c:59-64),
// and stats[r] = {max, log(sum(exp(l - max)))} (src/sample.c:25-33). k <= 1024.
int hfa_topk(const float* logits, int ld, int* ids, float* vals, float* stats, int n_rows, int vocab, int k,
             hipStream_t stream);

// Random weights on the device: element e of the tensor with `key` by the counter-based rule that
// weights/random_init.py states (the host's writer computes the same bits). dtype HFA_F32 or HFA_BF16
// with rule 0 (N(0, std): scale = std / sqrt(8 (65536^2 - 1) / 12)) or 1 (1 + that); dtype 2 (int32)
// with rule 2 (uniform below `bound`). The reference's one generator for model and oracle:
// tools/mkmodel.pl:104-127.
int hfa_random_fill(void* out, int dtype, size_t n, uint64_t key, float scale, int rule, int bound,
                    hipStream_t stream);

// The device's own peaks (the reference's read_sum and fma_burn, src/kern.h:17-23): a streaming read
// of `bytes` (16-byte aligned; `sink` is 16 bytes that are almost never written) by `blocks_per_cu`
// blocks of 256 threads a CU, a copy, and a burn of
// the matrix cores on register operands (`zeros`: all-zero operands, else small pseudo-random ones):
// `out` takes one float per thread of the launch, hfa_probe_mfma_threads() of them; *flops is what it
// computed. The caller times them.
int hfa_probe_read(const void* src, size_t bytes, void* sink, int blocks_per_cu, hipStream_t stream);
int hfa_probe_copy(const void* src, void* dst, size_t bytes, hipStream_t stream);
int hfa_probe_mfma_threads(void);
int hfa_probe_mfma(float* out, int iters, int zeros, double* flops, hipStream_t stream);

#ifdef __cplusplus
}
#endif
