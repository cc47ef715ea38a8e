/* qserve_serve.h -- C ABI of libqserve_serve.so: the kernels of the paged serving engine (qserve_amd/serving).
 *
 * Every tensor is a device pointer; `dtype` selects the storage type of activations, weights and cache rows
 * (QSV_BF16 = bfloat16 with 32-bit accumulation, QSV_F32 = float everywhere).  The residual stream, norm statistics,
 * attention scores / weights, rotary angles and router scores are float in both modes.  All launches go to `stream`
 * (a hipStream_t) and return 0 or an error code; qsv_last_error() describes the last failure of the calling thread.
 */
#pragma once
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define QSV_OK 0
#define QSV_EINVAL 1
#define QSV_BF16 0
#define QSV_F32 1

int qsv_version(void);
const char* qsv_arch(void);
const char* qsv_last_error(void);

/* x[t] = table[tokens[t]] (float) and h[t] = the same row in the storage type. */
int qsv_embed(float* x, void* h, const void* table, const int32_t* tokens, int n_tokens, int width, int dtype, void* stream);

/* x[t] = table[tokens[t]] * scale + s(pos[t]),  s(p)[2i] = sin(p freq[i]),  s(p)[2i + 1] = cos(p freq[i])   (float; freq float
 * [(width + 1) / 2]). */
int qsv_embed_sinusoid(float* x, const void* table, const int32_t* tokens, const int32_t* pos, const float* freq, float scale,
                       int n_tokens, int width, int dtype, void* stream);
/* x[t] += a[t] + (b[t] + c[t]) (each of a, b, c may be NULL); h[t] = x[t] / sqrt(mean(x[t]^2) + eps) * w in the storage type
 * (h == NULL: the sum only). */
int qsv_add_rms_norm(float* x, void* h, const void* a, const void* b, const void* c, const void* w, float eps, int n_tokens,
                     int width, int dtype, void* stream);
/* Sublayers between two norms: x[t] += rms_norm(y[t]) * w_post (y == NULL: nothing added), then h[t] = rms_norm(x[t]) * w_next in
 * the storage type (h == NULL: the sum only).  A weight is one gain for all coordinates (its *_wide flag 0) or one per coordinate. */
int qsv_add_normed_rms_norm(float* x, void* h, const void* y, const void* w_post, int post_wide, const void* w_next, int next_wide,
                            float eps, int n_tokens, int width, int dtype, void* stream);
/* Queries and keys RMS-normed per head (per_head != 0: weights [dim], shared by the heads) or over the whole projection (weights
 * [heads * dim] / [kv_heads * dim]), then turned by the position: pair (2i, 2i + 1), i < rot_n / 2, of every head by rope[pos[t], :,
 * i] (float [positions, 2, rot_n / 2], cos then sin; rope == NULL: no rotation).  q, k, v: rows of type qkv_dtype with their strides.
 *   qf[t, h]         = [ 0 (vdim) | q'[t, h] * scale ]     float [T, heads, vdim + dim]
 *   pool[g, slot[t]] = [ v[t, g] | k'[t, g] ]              [kv_heads, pool_rows, vdim + dim]     (k == NULL: nothing is written) */
int qsv_qk_norm_rope_prep(float* qf, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                          int64_t v_stride, int qkv_dtype, int heads, int kv_heads, int dim, int vdim, const void* q_w,
                          const void* k_w, int per_head, float eps, const float* rope, int rot_n, float scale, void* pool,
                          int64_t pool_rows, const int64_t* slot, const int32_t* pos, int n_tokens, int dtype, void* stream);
/* out[r] = rms_norm(x[rows[r]]) * w in the storage type (rows == NULL: row r). */
int qsv_rms_norm_rows(void* out, const float* x, const int32_t* rows, const void* w, float eps, int n_rows, int width, int dtype,
                      void* stream);
/* Queries and keys RMS-normed over the whole projection (all heads at once), values optionally blended, cache rows written:
 *   qf[t, h]         = [ 0 (vdim) | (q[t] / rms(q[t]) * q_w)[h] * scale ]          float [T, heads, vdim + dim]
 *   pool[g, slot[t]] = [ v'[t, g] | (k[t] / rms(k[t]) * k_w)[g] ]                  [kv_heads, pool_rows, vdim + dim]
 *   v' = (1 - mix) v + mix v_first[t] if v_first (storage type, rows vf_stride apart, [kv_heads * vdim]) is given, else v.
 * q, k, v are column ranges of proj (row stride `stride`). */
int qsv_normed_attention_prep(float* qf, void* pool, int64_t pool_rows, const void* proj, int64_t stride, int q_off, int k_off,
                              int v_off, int heads, int kv_heads, int dim, int vdim, const void* q_w, const void* k_w, float eps,
                              float scale, const void* v_first, int64_t vf_stride, float mix, const int64_t* slot, int n_tokens,
                              int dtype, void* stream);

/* x[t] += layer_norm(y[t]) * w (no bias; variance = mean of squared deviations); h[t] = x[t] in the storage type. */
int qsv_add_layer_norm(float* x, void* h, const void* y, const void* w, float eps, int n_tokens, int width, int dtype,
                       void* stream);

/* out[r] = layer_norm(x[rows[r]]) * w in the storage type (rows == NULL: row r). */
int qsv_layer_norm_rows(void* out, const float* x, const int32_t* rows, const void* w, float eps, int n_rows, int width,
                        int dtype, void* stream);

/* Latent projections of one attention layer, per token t, from `down` (row stride down_stride elements):
 *   cq[t]            = rms_norm(down[t, q_off : q_off + q_rank]) * q_w
 *   pool[slot[t]]    = [ rms_norm(down[t, kv_off : kv_off + kv_rank]) * kv_w | rot(down[t, kv_off + kv_rank : + rot_dim]) ]
 * rot() rotates the pairs (2i, 2i+1), i < rot_n / 2, by the angle whose cos / sin are rope[pos[t]][0 / 1][i]
 * (rope: float [positions, 2, rot_n / 2], already scaled); the remaining rot_dim - rot_n values are copied.
 * Cache rows have row_width = kv_rank + rot_dim elements. */
int qsv_latent_prep(const void* down, int64_t down_stride, int q_off, int q_rank, const void* q_w, void* cq,
                    int kv_off, int kv_rank, const void* kv_w, int rot_dim, int rot_n, const float* rope,
                    void* pool, const int64_t* slot, const int32_t* pos, float eps, int n_tokens, int dtype, void* stream);

/* qf[t, h] = scale * [ q_abs[h, t, 0 : rank] | rot(q[t, h, dim : dim + rot_dim]) ]  (float [T, H, rank + rot_dim]).
 * q: [T, H, dim + rot_dim], q_abs: [H, T, rank] (the query carried into the latent space), both in the storage type. */
int qsv_latent_query(float* qf, const void* q, const void* q_abs, const float* rope, const int32_t* pos, float scale,
                     int n_tokens, int heads, int dim, int rot_dim, int rot_n, int rank, int dtype, void* stream);

/* Softmax attention of every token over the cached latent rows of its sequence:
 *   score(t, h, j) = qf[t, h] . pool[row(seq[t], j)]   for  max(0, pos[t] - window + 1) <= j <= pos[t]  (window 0: all j <= pos)
 *   out[t, h]      = sum_j softmax_j(score) * pool[row][0 : rank]            (storage type, [T, H, rank])
 * row(s, j) = block_table[s * table_stride + j / page] * page + j % page.  variant: 0 = default kernel choice.
 * Several pools in one launch: heads [g * heads_per_pool, (g + 1) * heads_per_pool) read the pool that starts pool_stride
 * elements after pool g - 1 (one pool for all heads: heads_per_pool = heads, pool_stride = 0). */
/* Two further restrictions and one further term, for attention layers that have them (0 / NULL: none):
 *   chunk > 0:  only j with floor(j / chunk) == floor(pos[t] / chunk) are visible (chunks counted from position 0);
 *   bias:       float [heads, bias_len]; bias[h, min(pos[t] - j, bias_len - 1)] is added to the score (after the query's scale).
 * Keys behind the window and a sink (0 / NULL: none; both need window > 0 and chunk == 0):
 *   keep_first: positions j < keep_first stay visible to every later query;
 *   sink:       float [heads]; exp(sink[h]) is one more term of the softmax's denominator, without a value;
 *   pooled:     a second set of pools (pooled_stride elements apart, same row layout), block_rows rows per page: the block of
 *               pool_block positions that starts at position s of the sequence has row block_table[s / page] * block_rows +
 *               (s % page) / pool_block (written by qsv_pool_blocks).  A query at position p also sees the rows of the blocks
 *               b < (p - window + 1) / pool_block, those that end before its window starts; no bias with them. */
int qsv_latent_attention(void* out, const float* qf, const void* pool, const int32_t* block_table, int table_stride,
                         const int32_t* seq, const int32_t* pos, int window, int n_tokens, int heads, int rank,
                         int row_width, int page, int heads_per_pool, int64_t pool_stride, int chunk, const float* bias,
                         int bias_len, int keep_first, const float* sink, const void* pooled, int64_t pooled_stride, int pool_block,
                         int block_rows, int dtype, int variant, void* stream);
/* pooled[g, row(block)] = mean over the block's positions of pool[g, row(position)], for every token of the step whose position
 * ends a block of pool_block positions ((pos + 1) % pool_block == 0); float sum, one rounding. */
int qsv_pool_blocks(void* pooled, int64_t pooled_rows, const void* pool, int64_t pool_rows, const int32_t* block_table,
                    int table_stride, const int32_t* seq, const int32_t* pos, int n_tokens, int n_pools, int row_width,
                    int pool_block, int page, int block_rows, int dtype, void* stream);

int qsv_latent_attention_tile_tokens(int heads);
int qsv_latent_attention_mfma_ok(int rank, int row_width, int dtype);
/* The same attention on the bf16 matrix cores.  The host cuts every sequence's tokens of the step into work tiles of at most
 * qsv_latent_attention_tile_tokens(heads_per_pool) consecutive tokens: tiles int32 [n_tiles, 3] = (sequence slot, first flat token
 * index, tokens).  qsv_latent_attention_mfma_ok() says whether the sizes are taken (bfloat16 storage, rank and row width
 * multiples of 8, row width <= 576); otherwise use qsv_latent_attention. * key_splits > 1 cuts every tile's keys over that many workgroups and merges the partial results in a second launch (steps
 * with few tiles: decoding); part_o (float [key_splits, n_tokens, heads, rank]) and part_ml (float [key_splits, n_tokens,
 * heads, 2]) are its workspace.  q_first: every query is zero before this element (0 if unknown); the score product skips the
 * steps that lie wholly before it. */
int qsv_latent_attention_mfma(void* out, const float* qf, const void* pool, const int32_t* block_table, int table_stride,
                              const int32_t* pos, const int32_t* tiles, int n_tiles, int window, int heads, int rank,
                              int row_width, int page, int key_splits, float* part_o, float* part_ml, int n_tokens,
                              int q_first, int heads_per_pool, int64_t pool_stride, int chunk, const float* bias, int bias_len,
                              int keep_first, const float* sink, const void* pooled, int64_t pooled_stride, int pool_block,
                              int block_rows, void* stream);

/* o[t, i] *= sigmoid(g[t * g_stride + i]),  i < n. */
int qsv_sigmoid_gate(void* o, const void* g, int64_t g_stride, int n_tokens, int n, int dtype, void* stream);

/* Grouped top-k router: scores s = softmax(router . h[t]) over n_experts (score_fn QSV_SCORE_SOFTMAX) or sigmoid(router . h[t])
 * (QSV_SCORE_SIGMOID); the choice goes by c = s + correction (float [n_experts], may be NULL: c = s).  The experts form n_groups
 * equal groups of neighbours, a group's score is its largest c (group_top 1) or the sum of its two largest (group_top 2), only
 * experts of the best keep_groups groups are eligible (the others cannot be chosen whatever their c); the top_k eligible experts
 * with the largest c are chosen.  idx [T, top_k] int32, weight [T, top_k] float = their s times `scale`; renorm != 0 divides the
 * chosen s by their sum first (with softmax scores: the softmax over the chosen logits only).
 * bias (may be NULL, [n_experts], storage type) is added to the logits before anything else. */
#define QSV_SCORE_SOFTMAX 0
#define QSV_SCORE_SIGMOID 1
int qsv_moe_route(int32_t* idx, float* weight, const void* h, const void* router, const void* bias, int renorm, int n_tokens,
                  int width, int n_experts, int top_k, int n_groups, int keep_groups, int score_fn, const float* correction,
                  int group_top, float scale, int dtype, void* stream);

/* Activations of the first expert product: QSV_ACT_RELU_SQ relu(z)^2; QSV_ACT_GLU: the weight rows come in pairs (2f = gate,
 * 2f + 1 = up), output f = silu(gate) * up, and the output is half as wide as the product. */
#define QSV_ACT_NONE 0
#define QSV_ACT_RELU_SQ 1
#define QSV_ACT_GLU 2
/* QSV_ACT_CLAMPED_GLU: the same pairs with g = min(gate, limit), u = clamp(up, -limit, limit), output f = g sigmoid(1.702 g) (u + 1);
 * `limit` is read by this activation only.  Expert indices >= n_experts name identity experts (output = input): the up kernels
 * skip their slots and the down / combine kernels add weight * h[t] for them. */
#define QSV_ACT_CLAMPED_GLU 3
/* act[t, k] = activation(up[idx[t, k]] . h[t])     up: [E, ff, width] -> act [T, top_k, ff or ff / 2] (storage type). */
int qsv_moe_up(void* act, const void* h, const void* up, const int32_t* idx, int n_tokens, int top_k, int width, int ff,
               int activation, float limit, int n_experts, int dtype, void* stream);

/* y[t] = sum_k weight[t, k] * down[idx[t, k]] . act[t, k]     down: [E, width, ff] -> y [T, width] (storage type). */
int qsv_moe_down(void* y, const void* act, const void* down, const int32_t* idx, const float* weight, int n_tokens,
                 int top_k, int width, int ff, const void* h, int n_experts, int dtype, void* stream);

/* Expert-sorted form for many tokens: slots (t, k) are sorted by expert on the host side of the ABI, the expert products run
 * as ordinary matrix products over contiguous runs of sorted slots, and these kernels do the rest:
 *   out[i] = src[order[i] / div]                                   (rows into sorted order)
 *   a[i]   = relu(a[i])^2                                           (in place)
 *   y[t]   = sum_k weight[t, k] * ys[inv[t * top_k + k]]            (sorted rows back, weighted; float accumulation) */
/* Expert-major form (bfloat16): out[s, r] = act(W[e][r, :] . X[x_index ? x_index[s] / div : s, :]) for the sorted slots
 * s in [offsets[e], offsets[e + 1]) of every expert e; W [n_experts, rows, K]; act = one of QSV_ACT_* (QSV_ACT_GLU: out is
 * rows / 2 wide).  Every weight is read once per launch.  K a multiple of 8, at most 4096. */
int qsv_expert_rows(void* out, const void* X, const int64_t* x_index, int div, const void* W, const int64_t* offsets,
                    int n_experts, int rows, int K, int act, float limit, void* stream);
/* Grouped expert product on the bf16 matrix cores (prompt phase): the same out[s, n] for work tiles (expert, first sorted slot,
 * slots <= qsv_grouped_gemm_tile_slots()) listed in tiles int32 [n_tiles, 3]; K a multiple of qsv_grouped_gemm_k_step(), n_rows
 * a multiple of 4, n_tiles <= 65535.  act: QSV_ACT_* (QSV_ACT_GLU: out is n_rows / 2 wide). */
int qsv_grouped_gemm_tile_slots(void);
int qsv_grouped_gemm_k_step(void);
int qsv_grouped_gemm(void* out, const void* X, const int64_t* x_index, int div, const void* W, const int32_t* tiles,
                     int n_tiles, int n_rows, int K, int act, float limit, void* stream);
int qsv_gather_rows(void* out, const void* src, const int64_t* order, int div, int n_rows, int width, int dtype, void* stream);
int qsv_relu_sq(void* a, int64_t n, int dtype, void* stream);
/* (idx != NULL: slots with idx[t, k] >= n_experts take h[t] in place of a sorted row) */
int qsv_moe_combine(void* y, const void* ys, const int64_t* inv, const float* weight, int n_tokens, int top_k, int width,
                    const int32_t* idx, const void* h, int n_experts, int dtype, void* stream);


/* ---- several residual streams, statistics-free norm, token shift (serve_streams.hip) ---------------------------------------- */
/* x[t, s] = table[tokens[t]] * scale for every stream s     x: float [T, streams, width] */
int qsv_embed_streams(float* x, const void* table, const int32_t* tokens, float scale, int n_tokens, int streams, int width,
                      int dtype, void* stream);
/* h[t] = n_t + (n_before - n_t) * shift,  n_t = tanh(alpha * sum_s w_in[s] x[t, s]) * norm_w + norm_b  (shift == NULL: h = n).
 * n_before: the previous row of the batch if run_off[t] > 0, else prev[state_rd[t]] (zeros if state_rd[t] < 0); the token with
 * state_wr[t] >= 0 (the last of its run) stores n_t into prev[state_wr[t]].  prev: float [2 * slots, width]. */
int qsv_hc_read(void* h, const float* x, const float* w_in, const void* norm_w, const void* norm_b, float alpha,
                const void* shift, float* prev, const int32_t* run_off, const int32_t* state_rd, const int32_t* state_wr,
                int n_tokens, int streams, int width, int dtype, void* stream);
/* x[t, r] <- sum_s mix[s, r] x[t, s] + w_out[r] * y[t] for all r at once (at most 16 streams).  h_next != NULL: also the next
 * sublayer's input from the new streams, h_next[t] = tanh(alpha * sum_r w_in_next[r] x[t, r]) * norm_w + norm_b (no token shift). */
int qsv_hc_write(float* x, const void* y, const float* mix, const float* w_out, int n_tokens, int streams, int width, void* h_next,
                 const float* w_in_next, const void* norm_w, const void* norm_b, float alpha, int dtype, void* stream);
/* out[r] = tanh(alpha * sum_s x[rows[r], s]) * norm_w + norm_b  (rows == NULL: row r). */
int qsv_dyt_sum_rows(void* out, const float* x, const int32_t* rows, const void* norm_w, const void* norm_b, float alpha,
                     int n_rows, int streams, int width, int dtype, void* stream);
/* out[t] = (rms_norm(a[t]) * wa + rms_norm(b[t]) * wb) / 2 over `width`. */
int qsv_rms_pair_mean(void* out, const void* a, const void* wa, const void* b, const void* wb, float eps, int n_tokens,
                      int width, int dtype, void* stream);
/* out[r, f] = act(a[r, 2f]) * a[r, 2f + 1]     a: [n_rows, 2 ff]; act QSV_GLU_SILU or QSV_GLU_GELU_TANH (gelu in its tanh form) */
#define QSV_GLU_SILU 0
#define QSV_GLU_GELU_TANH 1
#define QSV_GLU_CLAMPED 2   /* g = min(gate, limit), u = clamp(up, -limit, limit): g sigmoid(1.702 g) (u + 1) */
int qsv_glu(void* out, const void* a, int n_rows, int ff, int act, float limit, int dtype, void* stream);

/* ---- matrix-state recurrences and the attention beside them (serve_recurrent.hip) ------------------------------------------- */
/* out[t, c] (float, [T, heads * dim]) = a_log ? exp(-exp(a_log[c / dim]) * softplus(z[t, c] + bias[c]))
 *                                             : sigmoid(z[t, c] + bias[c]) ^ (1 / tau) */
int qsv_decay(float* out, const void* z, int64_t z_stride, const void* bias, const float* a_log, float tau, int n_tokens,
              int heads, int dim, int dtype, void* stream);
/* Causal convolution over time per channel, then silu (act 1; act 0: no activation), of the columns [off, off + channels) of proj; w float [channels, taps],
 * the last tap is the current token's.  Inputs before a run's start come from hist[state_rd[t]] (float [2 * slots, taps - 1,
 * channels], oldest first; zeros if state_rd[t] < 0); the run's last token (state_wr[t] >= 0) writes the new history.  The
 * first n_unit groups of unit_dim channels are then divided by sqrt(sum of squares + 1e-6).  out: float [T, channels]. */
int qsv_conv_silu_unit(float* out, const void* proj, int64_t stride, int off, int channels, int taps, const float* w,
                       float* hist, const int32_t* run_off, const int32_t* state_rd, const int32_t* state_wr, int n_unit,
                       int unit_dim, int act, int n_tokens, int dtype, void* stream);
/* Per run (slot, first token, tokens, first position) and head, token by token, with S = state[slot, head] (float [dim, vdim],
 * zeros if the first position is 0) written back at the end, g = decay[t, head]:
 *   beta == NULL:  S <- diag(g) S + k v^T                                  o = S^T q * q_scale
 *   else:          S <- diag(g) S;  u = sigmoid(beta[t, head]) (v - S^T k);  S <- S + k u^T;  o = S^T q * q_scale
 * q, k: [T, qk_heads, dim] (head h reads h / (heads / qk_heads)), v: [T, heads, vdim], each with its row stride, of type
 * qkv_dtype; o: float [T, heads, vdim].  max_run: the longest run's tokens as the host knows them (1: every run is one decoded
 * token - a kernel without staging is used; any larger value, or 0 for unknown: the general kernel). */
/* Variants (0 / NULL: as above): head_decay != 0: decay is float [T, heads], one factor for all rows of a head's state;
 * kscale (float [T, heads]): k is multiplied by kscale[t, head] where it enters the state; v_cols < vdim: v has v_cols columns per
 * head and the state's column v_cols is fed with ones (it then holds sum of decayed kscale k: a normaliser, read out by q like
 * the others), further columns with zeros. */
/* Element-wise gated recurrence over every run (slot, first token, tokens, first position): S = state[slot] (float [width], zeros
 * if the first position is 0), per token S <- (1 - z) S + z c with z = sigmoid(proj[t, z_off + i] + b_z[i]), u = proj[t, x_off + i] +
 * b_x[i], c = u + 1/2 if u >= 0 else sigmoid(u); out[t, i] = S * silu(proj[t, g_off + i]) (storage type); S is written back.
 * max_run: the longest run's tokens as the host knows them (0: unknown); up to 32 a thread walks its channel's run, above that the
 * run's segments are scanned side by side and composed. */
int qsv_min_gru_scan(void* out, const void* proj, int64_t stride, int z_off, int x_off, int g_off, const void* b_z, const void* b_x,
                     float* state, const int32_t* runs, int n_runs, int max_run, int width, int dtype, void* stream);
int qsv_recurrent_scan(float* o, const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                       int64_t v_stride, int qkv_dtype, const float* decay, const void* beta, int64_t beta_stride,
                       int beta_dtype, float* state, const int32_t* runs, int n_runs, int max_run, int heads, int qk_heads,
                       int dim, int vdim, float q_scale, const float* kscale, int head_decay, int v_cols, void* stream);
/* out[t, h] = o[t, h] / rms(o[t, h]) * w * gate_fn(gate[t, h]) over vdim; gate_kind 0: silu, 1: sigmoid.  o's heads are o_stride
 * floats apart (0: vdim); w is [vdim], shared by the heads, or with w_per_head [heads, vdim].  den_m (float [T, heads], may be
 * NULL): o[t, h] is first divided by max(|o[t, h, vdim]|, exp(-den_m[t, h])) + 1e-6 (o_stride > vdim: the extra column). */
int qsv_head_rms_gate(void* out, const float* o, const void* w, const void* gate, int64_t gate_stride, int gate_kind, float eps,
                      int n_tokens, int heads, int vdim, int o_stride, int w_per_head, const float* den_m, int dtype, void* stream);
/* Exponential input and forget gates with a running maximum, per run (slot, first token, tokens, first position) and head:
 *   li = cap tanh((zi[t, h] + bias_i[h]) / cap),  lf = logsigmoid(cap tanh((zf[t, h] + bias_f[h]) / cap)),
 *   m_t = max(lf + m_(t-1), li),  a[t, h] = exp(lf + m_(t-1) - m_t),  b[t, h] = exp(li - m_t),  m[t, h] = m_t      (float [T, heads])
 * m_(t-1) of a run's first token is m_state[slot, h] (0 if the run starts at position 0); the run's last m goes back there. */
int qsv_max_gates(float* a, float* b, float* m, const void* zi, const void* zf, int64_t z_stride, const float* bias_i,
                  const float* bias_f, float cap, float* m_state, const int32_t* runs, int n_runs, int heads, int dtype, void* stream);
/* Rotations in the halves layout (pair p of n rotated dimensions = p and p + n / 2; rope: float [positions, 2, n / 2]):
 *   qf[t, h]           = [ 0 (vdim) | rot_k(q[t, h]) * scale ]            float [T, heads, vdim + dim]
 *   pool[g, slot[t]]   = [ rot_v(v[t, g]) | rot_k(k[t, g]) ]              [kv_heads, pool_rows, vdim + dim]
 * rot_k turns the first rot_n of dim dimensions, rot_v all vdim; q, k, v are column ranges of proj. */
int qsv_attention_prep(float* qf, void* pool, int64_t pool_rows, const void* proj, int64_t stride, int q_off, int k_off, int v_off,
                       int heads, int kv_heads, int dim, int vdim, int rot_n, const float* rope_k, const float* rope_v,
                       float scale, const int64_t* slot, const int32_t* pos, int n_tokens, int dtype, void* stream);
/* o[t, h, 0:n] turned by sign * pos[t], in place. */
int qsv_rotate_heads(void* o, const float* rope, const int32_t* pos, float sign, int n_tokens, int heads, int n, int dtype,
                     void* stream);

#ifdef __cplusplus
}
#endif
