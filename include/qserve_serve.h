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
 * row(s, j) = block_table[s * table_stride + j / page] * page + j % page.  variant: 0 = default kernel choice. */
int qsv_latent_attention(void* out, const float* qf, const void* pool, const int32_t* block_table, int table_stride,
                         const int32_t* seq, const int32_t* pos, int window, int n_tokens, int heads, int rank,
                         int row_width, int page, int dtype, int variant, void* stream);

int qsv_latent_attention_tile_tokens(int heads);
int qsv_latent_attention_mfma_ok(int rank, int row_width, int dtype);
/* The same attention on the bf16 matrix cores.  The host cuts every sequence's tokens of the step into work tiles of at most
 * qsv_latent_attention_tile_tokens(heads) consecutive tokens: tiles int32 [n_tiles, 3] = (sequence slot, first flat token
 * index, tokens).  qsv_latent_attention_mfma_ok() says whether the sizes are taken (bfloat16 storage, rank and row width
 * multiples of 8, row width <= 576); otherwise use qsv_latent_attention. * key_splits > 1 cuts every tile's keys over that many workgroups and merges the partial results in a second launch (steps
 * with few tiles: decoding); part_o (float [key_splits, n_tokens, heads, rank]) and part_ml (float [key_splits, n_tokens,
 * heads, 2]) are its workspace. */
int qsv_latent_attention_mfma(void* out, const float* qf, const void* pool, const int32_t* block_table, int table_stride,
                              const int32_t* pos, const int32_t* tiles, int n_tiles, int window, int heads, int rank,
                              int row_width, int page, int key_splits, float* part_o, float* part_ml, int n_tokens,
                              void* stream);

/* o[t, i] *= sigmoid(g[t * g_stride + i]),  i < n. */
int qsv_sigmoid_gate(void* o, const void* g, int64_t g_stride, int n_tokens, int n, int dtype, void* stream);

/* Grouped top-k router: scores = softmax(router . h[t]) over n_experts; the experts form n_groups equal groups of neighbours,
 * a group's score is its largest score, only experts of the best keep_groups groups are eligible; the top_k eligible experts
 * with the largest scores are chosen.  idx [T, top_k] int32, weight [T, top_k] float = their scores (not renormalised). */
int qsv_moe_route(int32_t* idx, float* weight, const void* h, const void* router, int n_tokens, int width, int n_experts,
                  int top_k, int n_groups, int keep_groups, int dtype, void* stream);

/* act[t, k] = relu(up[idx[t, k]] . h[t])^2     up: [E, ff, width] -> act [T, top_k, ff] (storage type). */
int qsv_moe_up(void* act, const void* h, const void* up, const int32_t* idx, int n_tokens, int top_k, int width, int ff,
               int dtype, void* stream);

/* y[t] = sum_k weight[t, k] * down[idx[t, k]] . act[t, k]     down: [E, width, ff] -> y [T, width] (storage type). */
int qsv_moe_down(void* y, const void* act, const void* down, const int32_t* idx, const float* weight, int n_tokens,
                 int top_k, int width, int ff, int dtype, void* stream);

/* Expert-sorted form for many tokens: slots (t, k) are sorted by expert on the host side of the ABI, the expert products run
 * as ordinary matrix products over contiguous runs of sorted slots, and these kernels do the rest:
 *   out[i] = src[order[i] / div]                                   (rows into sorted order)
 *   a[i]   = relu(a[i])^2                                           (in place)
 *   y[t]   = sum_k weight[t, k] * ys[inv[t * top_k + k]]            (sorted rows back, weighted; float accumulation) */
/* Expert-major form (bfloat16): out[s, r] = act(W[e][r, :] . X[x_index ? x_index[s] / div : s, :]) for the sorted slots
 * s in [offsets[e], offsets[e + 1]) of every expert e; W [n_experts, rows, K]; act = relu^2 (relu_sq != 0) or none.  Every
 * weight is read once per launch.  K a multiple of 8, at most 4096. */
int qsv_expert_rows(void* out, const void* X, const int64_t* x_index, int div, const void* W, const int64_t* offsets,
                    int n_experts, int rows, int K, int relu_sq, void* stream);
/* Grouped expert product on the bf16 matrix cores (prompt phase): the same out[s, n] for work tiles (expert, first sorted slot,
 * slots <= qsv_grouped_gemm_tile_slots()) listed in tiles int32 [n_tiles, 3]; K a multiple of qsv_grouped_gemm_k_step(), n_rows
 * a multiple of 4, n_tiles <= 65535. */
int qsv_grouped_gemm_tile_slots(void);
int qsv_grouped_gemm_k_step(void);
int qsv_grouped_gemm(void* out, const void* X, const int64_t* x_index, int div, const void* W, const int32_t* tiles,
                     int n_tiles, int n_rows, int K, int relu_sq, void* stream);
int qsv_gather_rows(void* out, const void* src, const int64_t* order, int div, int n_rows, int width, int dtype, void* stream);
int qsv_relu_sq(void* a, int64_t n, int dtype, void* stream);
int qsv_moe_combine(void* y, const void* ys, const int64_t* inv, const float* weight, int n_tokens, int top_k, int width,
                    int dtype, void* stream);

#ifdef __cplusplus
}
#endif
