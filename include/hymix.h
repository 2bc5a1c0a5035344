/*
 * libhymix - MI355X (gfx950) kernels of a decoder that mixes rotary attention layers with delta-rule recurrent
 * layers on a float32 residual: scaled embedding, the gated sublayer boundary with RMS norms on both sides,
 * token shift with a carried row per sequence, the preparation of q/k/v (projection norms, partial rotation,
 * unit-norm heads, value blending between layers, paged cache store), attention over the paged cache with
 * sinks and sliding windows that keep the first tokens, the generalized delta rule with a float32 state per
 * sequence, and squared ReLU.  Later additions: the grouped-norm and the Dynamic-Tanh residual boundaries, pooled
 * blocks, chunked masks and sigmoid weights in the attention kernels, interleaved rotation on any frequency table and
 * unit-RMS value heads in the preparation, and linear attention with a constant decay per head and a float32 state.
 *
 * Conventions (those of libqlinear and libseqmix): all pointers are DEVICE pointers owned by the caller,
 * matrices are row-major and dense unless a stride (in elements) is named; `stream` is a hipStream_t passed as
 * void*; nothing here allocates, frees or synchronises, so every call may be captured into a hipGraph;
 * 0 = launched, a negative HM_E* code = rejected before any launch, with a message from hm_last_error().
 *
 * `dtype` selects the storage type of activations, weights and caches: HM_F32 or HM_BF16.  Whatever the storage
 * type, the residual, norms, gates, angles, attention scores and weights, and everything inside the recurrence
 * are float32.
 *
 * A step's batch: B sequences contribute portions of consecutive tokens, T tokens in all, packed sequence after
 * sequence.  tok_seq[t] = index of the token's sequence in the step, tok_pos[t] = its position in the sequence,
 * qstart[b] = first row of sequence b (qstart[B] = T), seq_pos0[b] = position of its first token in this step,
 * seq_slot[b] = its state slot, slot_mapping[t] = cache row (block * block_size + offset) of the token,
 * block_tables [B, max_blocks].
 */
#ifndef HYMIX_H
#define HYMIX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HM_F32 0
#define HM_BF16 1

#define HM_OK 0
#define HM_EINVAL (-1)
#define HM_ESHAPE (-2)
#define HM_EWORKSPACE (-3)
#define HM_ELAUNCH (-4)

int hm_version(void);
const char* hm_last_error(void);

/* x[t] = embed[ids[t]] * scale (f32). */
int hm_embed_scaled(int dtype, const int64_t* ids, const void* embed, float scale, float* x, int64_t T, int W, void* stream);

/* The boundary between two sublayers, per token t, in one launch (x is [T, W] f32, updated in place):
 *   y != NULL:       z = y[t] * sigmoid(gate[t] + gate_bias);  x[t] += mult * z / sqrt(mean(z^2) + eps) * post_w
 *   next_w != NULL:  h_out[t] = x[t] / sqrt(mean(x[t]^2) + eps) * next_w
 *   carry_src != NULL: for the last token of every sequence's portion, carry_state[seq_slot * slot_stride + :] = carry_src[t]
 * gate rows are gate_stride elements apart. */
int hm_sublayer_close(int dtype, float* x, const void* y, const void* gate, int64_t gate_stride, const void* gate_bias,
                      const void* post_w, float mult, const void* next_w, float eps, void* h_out, const void* carry_src,
                      void* carry_state, int64_t slot_stride, const int32_t* tok_seq, const int32_t* qstart,
                      const int32_t* seq_slot, int64_t T, int W, void* stream);

/* out[t] = h[t] + (prev - h[t]) * mu;  prev = h[t-1] inside a portion, state[seq_slot * slot_stride + :] at a portion's
 * start, zero at position 0. */
int hm_token_shift(int dtype, const void* h, const void* mu, const void* state, int64_t slot_stride, const int32_t* tok_seq,
                   const int32_t* tok_pos, const int32_t* qstart, const int32_t* seq_slot, void* out, int64_t T, int W,
                   void* stream);

/* out[t, c] = max(z[t, c], 0)^2; z rows are z_stride elements apart. */
int hm_relu_squared(int dtype, const void* z, int64_t z_stride, void* out, int64_t T, int F, void* stream);

/* qkv [T, H*D + G*D + G*V] (rows row_stride apart), per token:
 *   q_norm_w / k_norm_w != NULL: RMS norm over the whole q (k) projection with that weight;
 *   the first 2 * rot_half channels of every q and k head turn by tok_pos * inv_freq[i] (channel i with i + rot_half);
 *   unit_norm: every rotated head divided by its RMS;
 *   v_first != NULL: v <- (1 - lam[0]) v + lam[0] v_first[t];
 *   k and v go to row slot_mapping[t] of the caches [rows, G, D] / [rows, G, V] (a negative row: not stored);
 *   q_out [T, H, D].
 * q_head_w / k_head_w != NULL ([D], one row shared by the heads): before the rotation every q (k) head is divided by its
 * own RMS and multiplied by that row; q_head_scale != NULL (f32 [H]): query head h times q_head_scale[h] after it.
 * k_cache == v_cache == NULL: the rows hold q only (keys and values are another layer's), nothing is stored.
 * interleaved: the rotation pairs channel 2i with 2i + 1 instead of i with i + rot_half; rot_mag multiplies every cosine
 * and sine (1 = a pure rotation; inv_freq may hold any table, e.g. one rescaled for longer contexts); v_unit_norm: every
 * value head is divided by sqrt(mean(head^2) + eps), no weight, before it is stored (not together with v_first). */
int hm_qkv_prepare(int dtype, const void* qkv, int64_t row_stride, int H, int G, int D, int V, const void* q_norm_w,
                   const void* k_norm_w, float eps, const float* inv_freq, int rot_half, int unit_norm, const int32_t* tok_pos,
                   const int32_t* slot_mapping, void* k_cache, void* v_cache, const void* v_first, int64_t v_first_stride,
                   const float* lam, void* q_out, int64_t T, const void* q_head_w, const void* k_head_w,
                   const float* q_head_scale, int interleaved, float rot_mag, int v_unit_norm, void* stream);

/* Attention of q [T, H, D] over the paged caches, any sizes, f32 arithmetic: the token at position i sees key j <= i,
 * and with window > 0 only if i - j < window or j < keep_first.  sink != NULL (f32 [H]): exp(sink[h]) joins the softmax
 * denominator.  o [T, H, V].
 * Pooled blocks (pool > 0, needs window > 0 and keep_first == 0): beside its window the token at position i sees one
 * key and value for every block of `pool` tokens whose last token lies at or before i - window: the block's mean key and
 * mean value, row e % pool_rows of page block_table[e / pool_rows] of kp_cache [pages, pool_rows, G, D] and vp_cache
 * [pages, pool_rows, G, V] for block e (pool_rows * pool >= block_size); they share the softmax with the tokens.
 * chunk > 0 (chunked mask; without kept first tokens and pooled blocks): the token at position i sees key j <= i only if
 * i / chunk == j / chunk, chunks counted from position 0 of the sequence.
 * sigmoid_w (without sink and pooled blocks): the weight of a visible key is sigmoid(score * scale + head_bias[h])
 * (head_bias f32 [H], NULL = 0) and the weights are not normalised over the keys. */
int hm_attn_rows(int dtype, const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                 const int32_t* tok_seq, const int32_t* tok_pos, const float* sink, int window, int keep_first, float scale,
                 void* o, int64_t T, int H, int G, int D, int V, int block_size, int max_blocks, const void* kp_cache,
                 const void* vp_cache, int pool, int pool_rows, int chunk, const float* head_bias, int sigmoid_w, void* stream);

/* The mean key and mean value of every block of `pool` tokens that the step completes, as the caches hold them (f32
 * sums), written to the pooled caches (layout above).  Sequence b's portion covers positions [seq_pos0[b], ctx_lens[b]);
 * max_q = the longest portion of the step.  Launch it after the step's keys and values are stored. */
int hm_pool_blocks(int dtype, const void* k_cache, const void* v_cache, void* kp_cache, void* vp_cache,
                   const int32_t* block_tables, const int32_t* seq_pos0, const int32_t* ctx_lens, int B, int max_q, int G, int D,
                   int V, int block_size, int max_blocks, int pool, int pool_rows, void* stream);

/* The same attention on the matrix cores, bf16 storage only, dim and vdim multiples of 8 up to 128, block_size % 64 == 0.
 * Portions of any length (max_q = the longest portion of the step): */
int hm_attn_tiles(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables, const int32_t* qstart,
                  const int32_t* seq_pos0, const float* sink, int window, int keep_first, float scale, void* o, int B, int max_q,
                  int H, int G, int D, int V, int block_size, int max_blocks, const void* kp_cache, const void* vp_cache, int pool,
                  int pool_rows, int chunk, const float* head_bias, int sigmoid_w, void* stream);
/* Single-token queries (q [B, H, D], ctx[b] = keys of sequence b incl. the new one): the visible key tiles are split
 * over `splits` workgroups per (sequence, key/value head) and merged in split order by a second launch.  At most 32
 * query heads per key/value head.  workspace: hm_attn_decode_workspace_bytes(B, H, V, splits) bytes. */
size_t hm_attn_decode_workspace_bytes(int64_t B, int H, int V, int splits);
int hm_attn_decode(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables, const int32_t* ctx,
                   const float* sink, int window, int keep_first, float scale, void* o, int64_t B, int H, int G, int D, int V,
                   int block_size, int max_blocks, int splits, void* workspace, size_t workspace_bytes, const void* kp_cache,
                   const void* vp_cache, int pool, int pool_rows, int chunk, const float* head_bias, int sigmoid_w, void* stream);

/* prep [T, H, 5, D] f32 = decay | a*u | u | k | r from the columns r_off, k_off, a_off (H*D wide) and z_off (rank wide) of
 * proj:  decay = exp(-decay_scale * sigmoid(w2 tanh(z) + w0)), a = sigmoid(a_pre + a_bias), u = k / sqrt(sum k^2 + unit_eps)
 * per head.  w2 [H*D, rank]. */
int hm_delta_prepare(int dtype, const void* proj, int64_t row_stride, int r_off, int k_off, int a_off, int z_off,
                     const void* w2, const void* w0, const void* a_bias, int rank, float decay_scale, float unit_eps,
                     float* prep, int64_t T, int H, int D, void* stream);

/* For every sequence b and head, over the tokens of its portion in order:
 *   S <- diag(decay) S - (a u)(u^T S) + k v^T (both terms from the old S);  o[t] = S^T r
 * state f32 [slots, H, D, D] is read at the start unless seq_pos0[b] == 0 (then S = 0) and written at the end.
 * v [T, H*D] in the storage type, rows v_stride apart.  o f32 [T, H, D].  D <= 256.  max_q = the longest portion of the
 * step (a hint for staging: results do not depend on it). */
int hm_delta_recurrence(int dtype, const float* prep, const void* v, int64_t v_stride, float* state, const int32_t* qstart,
                        const int32_t* seq_pos0, const int32_t* seq_slot, float* o, int B, int H, int D, int max_q, void* stream);

/* out[t, h*D + i] = o[t, h, i] / sqrt(mean_i o[t, h]^2 + eps) * norm_w[h*D + i] * sigmoid(g[t, h*D + i]). */
int hm_delta_gate_norm(int dtype, const float* o, const void* g, int64_t g_stride, const void* norm_w, float eps, void* out,
                       int64_t T, int H, int D, void* stream);

/* Linear attention with a constant decay per head.  q, k [T, H*D] and v [T, H*V] are the columns q_off, k_off, v_off of
 * proj (rows row_stride apart) passed through silu.  For every sequence b and head, over the tokens of its portion:
 *   S <- decay[h] S + k v^T;  o[t] = S^T q
 * state f32 [slots, H, D, V] is read at the start unless seq_pos0[b] == 0 (then S = 0) and written at the end.  decay f32
 * [H].  o f32 [T, H, V].  D <= 256.  max_q = the longest portion of the step (a hint for staging only). */
int hm_lightning_recurrence(int dtype, const void* proj, int64_t row_stride, int q_off, int k_off, int v_off,
                            const float* decay, float* state, const int32_t* qstart, const int32_t* seq_pos0,
                            const int32_t* seq_slot, float* o, int B, int H, int D, int V, int max_q, void* stream);

/* The boundary between two sublayers of a residual whose sublayers sit between two Dynamic-Tanh norms,
 * dyt(z) = tanh(alpha[0] z) * w + b per channel (alpha f32 on the device, w and b in the storage type); x [T, W] f32 is
 * updated in place, one elementwise launch:
 *   y != NULL, ids == NULL:  x[t] += dyt_post(y[t])
 *   y != NULL, ids != NULL:  x[t]  = y[ids[t]]                             (y = an embedding table; no norm)
 *   h_out != NULL:           h_out[t] = next_w ? dyt_next(x[t]) : x[t], in the storage type. */
int hm_dyt_residual(int dtype, float* x, const void* y, const int64_t* ids, const void* post_w, const void* post_b,
                    const float* post_alpha, const void* next_w, const void* next_b, const float* next_alpha, void* h_out,
                    int64_t T, int W, void* stream);

/* The boundary between two sublayers of a residual that is normalised on the sublayers' OUTPUT, with an RMS norm over
 * `groups` equal consecutive parts of the vector (each part divided by its own sqrt(mean(part^2) + eps)); x [T, W] f32 is
 * updated in place, per token in one launch:
 *   y != NULL, ids == NULL:  x[t] += group_norm(y[t]) * post_w
 *   y != NULL, ids != NULL:  x[t]  = group_norm(y[ids[t]]) * post_w       (y = an embedding table)
 *   h_out != NULL:           h_out[t] = next_w ? group_norm(x[t]) * next_w : x[t], in the storage type. */
int hm_group_norm_residual(int dtype, float* x, const void* y, const int64_t* ids, const void* post_w, const void* next_w,
                           int groups, float eps, void* h_out, int64_t T, int W, void* stream);

/* x[i] <- cap * tanh(x[i] * scale / cap) (cap <= 0: x[i] * scale), f32 in place. */
int hm_scale_softcap(float* x, int64_t n, float scale, float cap, void* stream);

#ifdef __cplusplus
}
#endif
#endif
