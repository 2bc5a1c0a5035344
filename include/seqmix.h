/*
 * libseqmix - MI355X (gfx950) kernels of the sequence-mixing and feed-forward mechanisms that sit between
 * the matrix products of a decoder layer: multi-stream residuals (hyper-connections) with their RMS norm,
 * short causal convolutions with per-sequence state, latent (compressed key/value) attention over a paged
 * cache, PolyNorm and clamped-GLU activations, and grouped top-k expert routing with the expert products.
 *
 * Conventions (those of libqlinear): all pointers are DEVICE pointers owned by the caller, matrices are
 * row-major and dense unless a stride is named; `stream` is a hipStream_t passed as void*; nothing here
 * allocates, frees or synchronises, so every call may be captured into a hipGraph; 0 = launched, a negative
 * SM_E* code = rejected before any launch, with a message from sm_last_error().
 *
 * `dtype` selects the storage type of activations and weights: SM_F32 or SM_BF16.  Whatever the storage
 * type, residual streams, norms, softmax, router scores and convolution sums are float32.
 */
#ifndef SEQMIX_H
#define SEQMIX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SM_F32 0
#define SM_BF16 1

#define SM_ROUTE_SOFTMAX 0
#define SM_ROUTE_SIGMOID 1

#define SM_ACT_CLAMPED_GLU 0
#define SM_ACT_GELU 1
#define SM_ACT_GELU_TANH 2
#define SM_ACT_SILU_GLU 3

#define SM_OK 0
#define SM_EINVAL (-1)
#define SM_ESHAPE (-2)
#define SM_EWORKSPACE (-3)
#define SM_ELAUNCH (-4)

int sm_version(void);
const char* sm_last_error(void);

/* X[t, s, :] = embed[ids[t]] + pos_table[positions[t]] for every stream s (f32 sum).  pos_table may be NULL. */
int sm_embed_streams(int dtype, const int64_t* ids, const int32_t* positions, const void* embed, const void* pos_table,
                     float* X, int64_t T, int S, int W, void* stream);

/* One launch per sublayer boundary of a multi-stream residual, per token t (X is [T, S, W] f32, updated in place):
 *   write phase (y != NULL):   X[t, r] <- sum_s mix[s, r] * X[t, s] + out[r] * y[t]     (all r from the old streams)
 *   read  phase (h_out != NULL): u = sum_s w_in[s] * X[t, s];  h_out[t] = u / sqrt(mean(u^2) + eps) * norm_w
 * mix [S, S] ([from, to]), out [S], w_in [S] are f32; norm_w has the storage type.  S <= 8.  S = 1 with
 * mix = out = w_in = 1 is the ordinary residual add + RMS norm. */
int sm_stream_step(int dtype, float* X, const void* y, const float* mix, const float* out, const float* w_in,
                   const void* norm_w, float eps, void* h_out, int64_t T, int S, int W, void* stream);

/* Causal per-channel convolution over time with carried state, added to its input:
 *   out[t] = h[t] + sum_{j < taps} w[:, j] * h(pos[t] - (taps - 1) + j)
 * where h(p) of a position before this step's tokens comes from the sequence's state (the last taps-1 inputs,
 * state[slot, run, k] = input at position ctx_before - (taps - 1) + k) and is zero for p < 0.
 * tok_seq[t] = index of the token's sequence in the step, tok_pos[t] = its position, qstart[b] = first row of
 * sequence b, seq_slot[b] = its state slot.  state is [slots, runs, taps - 1, W]. */
int sm_canon_conv(int dtype, const void* h, const void* w, const void* state, int run, int runs, const int32_t* tok_seq,
                  const int32_t* tok_pos, const int32_t* qstart, const int32_t* seq_slot, void* out, int64_t T, int W,
                  int taps, void* stream);
/* state[slot, run] <- the last taps-1 inputs of every sequence after this step (older ones shift out). */
int sm_canon_update(int dtype, const void* h, void* state, int run, int runs, const int32_t* qstart,
                    const int32_t* seq_slot, int B, int W, int taps, void* stream);

/* out[t] = x[t] / sqrt(mean(x[t]^2) + eps) * w over R columns, x rows row_stride apart, out dense [T, R]. */
int sm_rms_norm_rows(int dtype, const void* x, int64_t row_stride, const void* w, float eps, void* out, int64_t T, int R,
                     void* stream);

/* c = x / sqrt(mean(x^2) + eps) * w over R columns of rows with stride `row_stride` elements; stored at cache row
 * slot_mapping[t] of a paged cache [rows, R] (slot < 0: skipped). */
int sm_latent_norm_store(int dtype, const void* x, int64_t row_stride, const void* w, float eps, void* cache,
                         const int32_t* slot_mapping, int64_t T, int R, void* stream);

/* Causal softmax attention of absorbed queries over a paged latent cache whose rows are both key and value:
 *   o[t, h] = sum_{j <= pos[t]} softmax_j(scale * q[t, h] . c_j) c_j
 * q, o [T, H, R]; cache [blocks, block_size, R]; block_tables [B, max_blocks]; tok_seq / tok_pos as above.
 * The portable kernel (any R, both storage types): one workgroup per (token, head). */
int sm_latent_attn_rows(int dtype, const void* q, const void* cache, const int32_t* block_tables, const int32_t* tok_seq,
                        const int32_t* tok_pos, void* o, float scale, int64_t T, int H, int R, int block_size,
                        int max_blocks, int RV, int window, void* stream);
/* In the three attention calls: RV > 0 = only the first RV columns of a cache row are values (the rest, e.g. a rotated
 * key part, only enters the scores) and o is [T, H, RV]; RV <= 0 = R.  window > 0: the token at position i sees only the
 * keys j with i - j < window. */

/* A latent with a rotated key part: x rows (x_stride apart) hold [R | Rd]; c = rms_norm(x[:R]) * w and x[R:] with its
 * first rot_dims channels turned by tok_pos * inv_freq[i] (channel 2i with 2i + 1, f32 angles) go to cache row
 * slot_mapping[t] of a paged cache [rows, R + Rd].  q rows (q_stride apart) hold per head [D | Rd]; every head's Rd part
 * is turned the same way and written to columns R .. R + Rd of qa [T, H, R + Rd] (whose first R columns, the absorbed
 * queries, are the caller's). */
int sm_latent_rope_store(int dtype, const void* x, int64_t x_stride, const void* w, float eps, const void* q, int64_t q_stride,
                         void* qa, const float* inv_freq, int rot_dims, const int32_t* tok_pos, void* cache,
                         const int32_t* slot_mapping, int64_t T, int H, int D, int R, int Rd, void* stream);

/* The same product on the matrix cores (bf16, R % 8 == 0, R <= 256, block_size % 64 == 0): a workgroup owns 128
 * consecutive (token, head) rows of one sequence and walks 64-key tiles of the cache.  qstart [B + 1]; seq_pos0[b]
 * = position of the sequence's first token in this step; max_q = the longest portion.  */
int sm_latent_attn_tiles(const void* q, const void* cache, const int32_t* block_tables, const int32_t* qstart,
                         const int32_t* seq_pos0, void* o, float scale, int B, int max_q, int H, int R, int block_size,
                         int max_blocks, int RV, int window, void* stream);

/* Single-token queries (decode) on the matrix cores with the keys split over workgroups: every (sequence, split)
 * writes an unnormalised partial state to `workspace`, a second launch merges them.  ctx[b] = keys visible to the
 * one token of sequence b (row b of q / o). */
size_t sm_latent_decode_workspace_bytes(int64_t B, int H, int R, int splits);
int sm_latent_attn_decode(const void* q, const void* cache, const int32_t* block_tables, const int32_t* ctx, void* o,
                          float scale, int64_t B, int H, int R, int block_size, int max_blocks, int splits,
                          void* workspace, size_t workspace_bytes, int RV, int window, void* stream);

/* PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the F columns of a row;
 * coef = {a, b, c, e} f32 on the device. */
int sm_poly_norm(int dtype, const void* z, const float* coef, float eps, void* out, int64_t T, int F, void* stream);

/* Clamped GLU: gu [T, 2F] = gate | up;  g = min(gate, limit), u = clamp(up, -limit, limit);
 * out = g * sigmoid(alpha * g) * (u + 1). */
int sm_clamped_glu(int dtype, const void* gu, float limit, float alpha, void* out, int64_t T, int F, void* stream);

/* Router: z = router_w h (f32), s = softmax(z) over E experts; experts form `groups` equal groups of neighbours, a
 * group scores its largest s, only experts of the best `keep` groups are eligible (groups <= 1: all are); the `top`
 * eligible experts with the largest s are chosen, weights = their s / (sum + 1e-20).  idx [T, top] i32, wts [T, top] f32. */
/* score = SM_ROUTE_SIGMOID: s = sigmoid(z) instead.  correction != NULL (f32 [E]): the choice (groups and experts) goes
 * by s + correction, the weights stay s.  group_top (1..4): a group scores the sum of its group_top largest choice
 * scores.  renorm == 0: the weights are the chosen s as they are.  bias != NULL (f32 [E]): z = router_w h + bias (with
 * softmax scores and renorm the weights are then the softmax over the chosen experts' logits). */
int sm_moe_route(int dtype, const void* h, const float* router_w, int32_t* idx, float* wts, int64_t T, int W, int E,
                 int top, int groups, int keep, int score, const float* correction, int group_top, int renorm,
                 const float* bias, void* stream);

/* Expert products, one (token, chosen expert) pair at a time (memory-bound form for few tokens):
 * act[p] = clamped_glu(w_gu[e] h[t]) with w_gu [E, 2F, W] (gate rows, then up rows), p = t * top + k; then
 * y[t] = sum_k wts[t, k] * (w_down[e_k] act[t * top + k]) + shared[t]   (w_down [E, W, F]; shared may be NULL). */
/* act_kind = SM_ACT_CLAMPED_GLU as above; SM_ACT_GELU / SM_ACT_GELU_TANH: an expert is w_down act(w_up h) with the exact
 * (erf) or the tanh GELU, and w_gu is [E, F, W] (one part when tiled).  SM_ACT_SILU_GLU: the gated form without the one,
 * g' sigmoid(alpha g') u' (limit = +inf, alpha = 1: silu(gate) * up), w_gu as for the clamped GLU. */
int sm_moe_pairs_gate_up(int dtype, const void* h, const int32_t* idx, const void* w_gu, float limit, float alpha,
                         int act_kind, void* act, int64_t T, int top, int W, int F, void* stream);
int sm_moe_pairs_down(int dtype, const void* act, const int32_t* idx, const float* wts, const void* w_down,
                      const void* shared, void* y, int64_t T, int top, int W, int F, void* stream);

/* The same sum for many tokens on the matrix cores (bf16, W % 8 == 0, F % 8 == 0): pairs are grouped by expert into
 * tiles of 32 rows.  w_gu and w_down are TILED here: blocks of 32 rows x 64 k (4 KB; rows and k zero-padded to whole
 * blocks) in the order (expert, gate|up, row block, k step); inside a block the 8 values k = 64 step + 32 hi + 8 s .. +8
 * of row r sit at byte 16 (64 s + 32 hi + r).  Scratch (caller-owned): n = sm_moe_grouped_tiles(T, top, E) tiles; row_pair int32 [32 n],
 * tile_expert int32 [n], pair_row int32 [T * top], act bf16 [32 n, F], prod bf16 [32 n, W]. */
int sm_moe_grouped_tiles(int64_t T, int top, int E);
int sm_moe_grouped(const void* h, const int32_t* idx, const float* wts, const void* w_gu, const void* w_down,
                   const void* shared, float limit, float alpha, int act_kind, void* y, int64_t T, int top, int E, int W, int F,
                   int32_t* row_pair, int32_t* tile_expert, int32_t* pair_row, void* act, void* prod, void* stream);

/* sm_moe_grouped with tiles of 128 rows (activations of a tile staged once in LDS, every weight fragment reused by four
 * row fragments): the form for large groups.  Same arguments; scratch for n = sm_moe_tiles128_count(T, top, E) tiles:
 * row_pair int32 [128 n], tile_expert int32 [n], pair_row int32 [T * top], act bf16 [128 n, F], prod bf16 [128 n, W]. */
int sm_moe_tiles128_count(int64_t T, int top, int E);
int sm_moe_tiles128(const void* h, const int32_t* idx, const float* wts, const void* w_gu, const void* w_down,
                    const void* shared, float limit, float alpha, int act_kind, void* y, int64_t T, int top, int E, int W, int F,
                    int32_t* row_pair, int32_t* tile_expert, int32_t* pair_row, void* act, void* prod, void* stream);

/* The two ends of sm_moe_grouped on their own (bf16): the grouping (same scratch layout) and the weighted sum of a token's
 * per-pair products prod [32 n, W] (+ shared).  Between them the caller may run the expert products itself. */
int sm_moe_align(const int32_t* idx, int64_t T, int top, int E, int32_t* row_pair, int32_t* tile_expert, int32_t* pair_row,
                 void* stream);
int sm_moe_combine(const void* prod, const int32_t* pair_row, const float* wts, const void* shared, void* y, int64_t T, int top,
                   int W, void* stream);

#ifdef __cplusplus
}
#endif
#endif
