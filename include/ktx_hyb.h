/* ktx_hyb.h — C ABI of the hybrid-decoder kernels (libktx_hip.so / libktx_seq.so): what a decoder needs whose layers alternate a
 * gated delta-rule recurrence (short causal convolutions in front, state slots behind) with a sliding-window softmax attention over a
 * paged LATENT cache (normed latent + one rotated key part per token, a per-head sink in the denominator), under layer norms with
 * bias, a sigmoid-gated post-normed residual, a PolyNorm feed-forward and a sigmoid-routed mixture of GLU experts.
 *
 * Batching contract: that of ktx_seq.h — the T tokens of all scheduled requests are flattened, request b owns rows
 * q_indptr[b] .. q_indptr[b+1]; a token knows its request, its position and the cache row of its key.  The residual stream, norms,
 * scores, softmax, router, gates, decays and the recurrent state are fp32 whatever the storage type (KTX_SEQ_BF16 / KTX_SEQ_F32 of
 * ktx_seq.h).  DEVICE pointers, enqueue-only on `stream`, 0 = success (ktx_last_error() for the message). */
#ifndef KTX_HYB_H
#define KTX_HYB_H
#include <stddef.h>
#include <stdint.h>

#include "ktx_seq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* x[t] += (x0 ? x0[t] : 0) + (vec ? vec : 0): fp32 rows of width W (what a repeated block adds in front of a pass). */
int ktx_rows_add(int T, int W, float* d_x, const float* d_x0, const float* d_vec, ktx_stream_t stream);

/* out[t] = (x[r] - mean) / sqrt(var + eps) * w + b, var = mean of squared deviations, r = rows ? rows[t] : t.  x fp32 [.][W];
 * w, b fp32 [W] (b may be NULL); out [T][W] of out_dtype. */
int ktx_layer_norm(int T, int W, const float* d_x, const float* d_w, const float* d_b, float eps, const int32_t* d_rows, void* d_out,
                   int out_dtype, ktx_stream_t stream);

/* The gated, post-normed residual update of one sublayer, one launch:
 *   z[t] = (y ? y[t] : 0) + (ybias ? ybias : 0) + sum_{k < top} topk_w[t][k] * ey[pair_pos[t * top + k]]     (ey NULL: no such term)
 *   z   *= sigmoid(gl[t] + gbias)                                                                            (gl NULL: no gate)
 *   x[t] += layer_norm(z; wn, bn, eps)
 *   next_out[t] = layer_norm(x[t]; next_w, next_b, next_eps)      (next_w NULL: not written) — the pre-norm of the sublayer that follows
 * y fp32 rows of stride ldy, ey fp32 [pairs][W], gl fp32 rows of stride ldg, all vectors fp32 [W]; x fp32 [T][W] in place;
 * next_out [T][W] of next_dtype. */
int ktx_gated_norm_add(int T, int W, const float* d_y, int64_t ldy, const float* d_ybias, const float* d_ey, const int32_t* d_pair_pos,
                       const float* d_topk_w, int top, const float* d_gl, int64_t ldg, const float* d_gbias, const float* d_wn,
                       const float* d_bn, float eps, float* d_x, const float* d_next_w, const float* d_next_b, float next_eps,
                       void* d_next_out, int next_dtype, ktx_stream_t stream);

/* The post-normed residual update of one sublayer with a scaled residual, and the depth-weighted average behind a layer, one launch:
 *   v[t] = layer_norm(alpha * x_in[t] + (y ? y[t] : 0) + (ybias ? ybias : 0); w, b, eps)
 *   stack (fp32, level l at stack + l * stack_stride, [T][W] each; optional): level `level` receives v[t]
 *   dwa (fp32 [level + 1], needs stack): x_out[t] = sum_{j <= level} dwa[j] * stack level j [t]; otherwise x_out[t] = v[t]
 *   out_lp (optional, [T][W] of out_dtype): a copy of x_out for the products that follow.
 * x_in and x_out may be the same rows (in place) or not (x_in may be a level of the stack). */
typedef struct ktx_postnorm_args {
  const float* y;
  int64_t ldy;
  const float* ybias;
  float alpha;
  const float* w;
  const float* b;
  float eps;
  float* stack;
  int64_t stack_stride;
  int32_t level;
  const float* dwa;
  void* out_lp;
  int32_t out_dtype;
} ktx_postnorm_args;
int ktx_postnorm_mix(int T, int W, const float* d_x_in, float* d_x_out, const ktx_postnorm_args* a, ktx_stream_t stream);

/* PolyNorm: with u(v) = v / sqrt(mean(v^2) + eps) over a row of F values and z = in[t] + bias,
 * out[t] = c[0] u(z) + c[1] u(z^2) + c[2] u(z^3) + c[3] (powers element-wise).  in fp32 rows of stride ldz; coef fp32 [4] on the device. */
int ktx_poly_norm(int T, int F, const float* d_z, int64_t ldz, const float* d_bias, const float* d_coef, float eps, void* d_out,
                  int out_dtype, ktx_stream_t stream);

/* out[r][f] = silu(in[r][f]) * in[r][F + f]: fp32 rows of 2F (stride ldi) -> [R][F] of out_dtype. */
int ktx_silu_mul_rows(int R, int F, const float* d_in, int64_t ldi, void* d_out, int out_dtype, ktx_stream_t stream);

/* out[r][f] = g * sigmoid(slope * g) * (u + up_shift) with g = min(gate, limit), u = clamp(up, -limit, limit): the activation of a GLU
 * whose gate is capped from above and whose linear half is clamped (limit = INFINITY: neither); fp32 rows of 2F (stride ldi) holding
 * gate = in[r][f], up = in[r][F + f], or — paired != 0 — gate = in[r][2f], up = in[r][2f + 1]; -> [R][F] of out_dtype. */
int ktx_glu_clamp_rows(int R, int F, const float* d_in, int64_t ldi, float limit, float slope, float up_shift, int paired, void* d_out,
                       int out_dtype, ktx_stream_t stream);

/* out[r][c] = o[r][c] * sigmoid(gate[r][c]): o [R][N] of o_dtype, gate fp32 rows of stride ldg -> [R][N] of out_dtype (an output gate
 * on an attention's concatenated heads). */
int ktx_sigmoid_gate_rows(int R, int N, const void* d_o, int o_dtype, const float* d_gate, int64_t ldg, void* d_out, int out_dtype,
                          ktx_stream_t stream);

/* out[t][h][v] = o[t][h][v] / sqrt(mean_v(o[t][h]^2) + eps) * w[(w_per_head ? h * vdim : 0) + v] * act(gate[t][h * vdim + v]);
 * act = sigmoid (0) or silu (1).  o fp32 [T][heads * vdim]; gate fp32 rows of stride ldg. */
int ktx_head_gate_norm(int T, int heads, int vdim, float eps, const float* d_o, const float* d_gate, int64_t ldg, const float* d_w,
                       int w_per_head, int act, void* d_out, int out_dtype, ktx_stream_t stream);

/* ---- gated delta rule ------------------------------------------------------------------------------------------------------ */
typedef struct ktx_delta_config {
  int32_t heads, kv_heads, dim, vdim; /* value heads, query / key heads (heads % kv_heads == 0), sizes per head */
  int32_t taps;                       /* of the causal convolutions in front of q, k, v (>= 1; 1 = a plain per-channel scale) */
  float unit_eps;                     /* q, k -> v / sqrt(sum(v^2) + unit_eps) per head; q also times dim^-1/2 */
} ktx_delta_config;

/* Per token, between the input projection and the recurrence: the convolution over time (channels = q | k | v, C = 2 kv_heads dim +
 * heads vdim; taps fp32 [C][taps], last column = the current token; inputs before a request's first NEW token come from its slot of
 * conv_state fp32 [slots][taps - 1][C] when pos0 > 0 and are zero otherwise), silu, the unit vectors -> qkv fp32 [T][C]; and per head
 * decay g = exp(-exp(A_log) softplus(a + dt_bias)) and step beta = sigmoid(b), per key head k . q -> gb fp32 [T][2 heads + kv_heads]
 * (g | beta | k . q).
 * proj: fp32 rows of stride ldp with q, k, v, b, a at their offsets.  Then ktx_delta_conv_update moves the state on (second launch). */
int ktx_delta_prep(const ktx_delta_config* cfg, int B, int T, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                   const int32_t* d_tok_req, const float* d_proj, int64_t ldp, int q_off, int k_off, int v_off, int b_off, int a_off,
                   const float* d_taps, const float* d_A_log, const float* d_dt_bias, float* d_conv_state, float* d_qkv, float* d_gb,
                   ktx_stream_t stream);

/* Per head, token by token from the slot's state S fp32 [slots][heads][dim][vdim] (zero when pos0 == 0, whatever the slot holds):
 *   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q       (q, k of head h / (heads / kv_heads))
 * (evaluated as o = (g S)^T q + u (k . q): both read-outs of the decayed state are taken before the write).
 * o fp32 [T][heads * vdim].  dim <= 256. */
int ktx_delta_forward(const ktx_delta_config* cfg, int B, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                      const float* d_qkv, const float* d_gb, float* d_S, float* d_o, ktx_stream_t stream);

/* ---- sliding-window softmax attention over a latent cache, with a sink ------------------------------------------------------- */
typedef struct ktx_latattn_config {
  int32_t heads, dim, rot_dim, vdim, kv_rank; /* per head: dim un-rotated + rot_dim rotated query / key entries; latent size */
  int32_t rot_dims;                           /* the first rot_dims entries of the rotated part turn (pairs 2i, 2i+1); even, <= rot_dim */
  float scale;                                /* score = scale * (q . k) */
  int32_t window;                             /* position i sees j with 0 <= i - j < window; <= 0: no window */
  float eps;                                  /* of the latent's RMS norm */
  int32_t page_size, cache_dtype;             /* cache rows [rows][kv_rank + rot_dim] of KTX_SEQ_* */
  int32_t rot_half;                           /* != 0: the turning pairs are (i, i + rot_dims / 2) instead of (2i, 2i + 1) */
} ktx_latattn_config;

/* Per token: the first kv_rank entries of the down projection, RMS-normed with weight wn, and the last rot_dim, rotated at the token's
 * position (angle = pos * inv_freq[i], fp64 [rot_dims / 2]), go to cache row cache_loc[t]; each head's rotated query part goes, rotated,
 * to q_out[t][h][kv_rank ..] (q_out fp32 [T][heads][kv_rank + rot_dim]; the first kv_rank entries per head are written by the caller:
 * the un-rotated query part times W_uk of the head).  proj fp32 rows of stride ldp: q at q_off [heads][dim + rot_dim], the down
 * projection at c_off [kv_rank + rot_dim].  d_cache NULL: nothing is appended (a layer that reads the rows another layer of equal
 * kv_rank, rot_dim and rotation cached); only the queries' rotated parts are written. */
int ktx_latattn_prep(const ktx_latattn_config* cfg, int T, const float* d_proj, int64_t ldp, int q_off, int c_off, const float* d_wn,
                     const double* d_inv_freq, const int32_t* d_pos, const int32_t* d_cache_loc, void* d_cache, float* d_q_out,
                     ktx_stream_t stream);

/* out[t][h] = sum_j w_j c_j over the keys j in the window of token t, w = softmax over {scale q[t][h] . row_j} u {sink[h]} with the
 * sink's weight dropped (it has no value; d_sink NULL: an ordinary softmax over the keys).  q fp32 [T][heads][kv_rank + rot_dim]; out [T][heads][kv_rank] of out_dtype.
 * nsplit workgroups share a token's keys: scratch fp32 [nsplit][T][heads][kv_rank + 2] when nsplit > 1. */
int ktx_latattn_forward(const ktx_latattn_config* cfg, int T, const float* d_q, const void* d_cache, const int32_t* d_tok_req,
                        const int32_t* d_pos, const int32_t* d_page_indptr, const int32_t* d_page_indices, const float* d_sink,
                        int nsplit, float* d_scratch, void* d_out, int out_dtype, ktx_stream_t stream);

/* The same operator on the matrix cores, for prompts, portions and decode steps: request b's query rows q_indptr[b] .. q_indptr[b+1]
 * (at most max_q_len tokens; T in all) start at position pos0[b].  The (token, head) pairs of a request are the rows of one query
 * matrix against the shared latent rows; workgroups of 64 rows walk 32-key tiles: bf16 MFMA for q . row and for weights x rows (q
 * rounded to bf16), scores / mask / softmax in fp32.  nsplit key ranges per workgroup row (scratch as above), then merged with the sink.
 * Eligible: bf16 cache, kv_rank 64 / 128 / 256 / 512, rot_dim a multiple of 8 up to 128; ktx_latattn_forward serves everything else. */
int ktx_latattn_mfma_eligible(const ktx_latattn_config* cfg);
int ktx_latattn_mfma(const ktx_latattn_config* cfg, int B, int T, int max_q_len, const float* d_q, const void* d_cache,
                     const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_page_indptr, const int32_t* d_page_indices,
                     const float* d_sink, int nsplit, float* d_scratch, void* d_out, int out_dtype, ktx_stream_t stream);

/* ---- mixture of experts ---------------------------------------------------------------------------------------------------- */
/* s = sigmoid(logits[t]) (fp32 rows of stride ldl, E experts); the `top` largest (lowest index first on ties) ->
 * topk_idx int32 [T][top], topk_w fp32 [T][top] = s / (sum of the chosen s + sum_eps) * scale. */
int ktx_moe_route(int T, int E, int top, float scale, float sum_eps, const float* d_logits, int64_t ldl, int32_t* d_topk_idx,
                  float* d_topk_w, ktx_stream_t stream);

/* Sort the T * top (token, choice) pairs by expert: group_off int32 [E + 1]; sorted_tok int32 [pairs] = the token of each sorted row;
 * pair_pos int32 [pairs] = the sorted row of pair t * top + k; sorted_group int32 [pairs] = the expert of each sorted row; tiles of
 * tile_m rows that never span two experts:
 * tile_group / tile_row0 int32 [pairs / tile_m + E + 1], their number in num_tiles[0].  One workgroup; E <= 4096. */
int ktx_moe_plan(int T, int E, int top, int tile_m, const int32_t* d_topk_idx, int32_t* d_group_off, int32_t* d_sorted_tok,
                 int32_t* d_pair_pos, int32_t* d_sorted_group, int32_t* d_tile_group, int32_t* d_tile_row0, int32_t* d_num_tiles,
                 ktx_stream_t stream);

enum { KTX_GG_TILE_M = 64, KTX_GG_TILE_M_WIDE = 128 };
/* epilogues of the grouped products: none; silu(gate) * up over a [2N][K] matrix (streaming form only); relu(y)^2 */
enum { KTX_GG_ACT_NONE = 0, KTX_GG_ACT_GLU_SILU = 1, KTX_GG_ACT_RELU_SQ = 2 };

/* Grouped GEMM  Y_g = A_g W_g^T  on the matrix cores (the product runs in W's type like ktx_dense_gemm; Y fp32 or bf16).
 * W: G matrices [N][K] back to back.
 * Uniform form (d_group_off NULL): every group g < G multiplies the same M rows; A_g = columns a_goff * g .. of A's rows, Y_g = columns
 *   y_goff * g .. of Y's rows (per-head products of a [T][heads][.] tensor).
 * Ragged form: sorted rows group_off[g] .. group_off[g+1] belong to group g; the A row of sorted row r is a_rows[r] (NULL: r itself), its
 *   Y row is r; tiles come from ktx_moe_plan (max_tiles bounds the launch, num_tiles[0] on the device says how many are real) and hold
 *   tile_m = 64 rows, or 128 (bf16 products only: the wide tile prompts take).  The plan may hold MORE groups than G (a router whose
 *   last outputs stand for experts without weights): their tiles are skipped and their Y rows left untouched.
 * act: KTX_GG_ACT_NONE or KTX_GG_ACT_RELU_SQ, applied to Y. */
int ktx_grouped_gemm(int G, int M, int N, int K, const void* d_A, int a_dtype, int64_t lda, int64_t a_goff, const int32_t* d_a_rows,
                     const void* d_W, int w_dtype, void* d_Y, int y_dtype, int64_t ldy, int64_t y_goff, const int32_t* d_group_off,
                     const int32_t* d_tile_group, const int32_t* d_tile_row0, const int32_t* d_num_tiles, int max_tiles, int tile_m,
                     int act, ktx_stream_t stream);

/* The ragged products for a handful of rows (decode steps), streaming each row's weights once: Y[r] = W_g A[a_rows ? a_rows[r] : r]
 * with g = row_group[r]; rows whose group is >= G (no weights) are left untouched.  act = KTX_GG_ACT_GLU_SILU: W_g is [2N][K] (gate
 * rows, then up rows) and Y[r][n] = silu(gate_n . a) * (up_n . a) — the activation of a GLU expert in the same launch;
 * KTX_GG_ACT_RELU_SQ: Y = relu(Y)^2.  fp32 accumulation on the vector ALUs; any N, K. */
int ktx_grouped_gemv(int R, int N, int K, const void* d_A, int a_dtype, int64_t lda, const int32_t* d_a_rows, const void* d_W, int w_dtype,
                     void* d_Y, int y_dtype, int64_t ldy, const int32_t* d_row_group, int act, int G, ktx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
