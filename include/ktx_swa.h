/* ktx_swa.h — C ABI of the kernels (libktx_hip.so / libktx_seq.so) for decoders on an fp32 residual stream whose layers mix tokens
 * with a grouped-query sliding-window softmax attention over paged KEY and VALUE caches (partly rotated unit-RMS queries and keys,
 * values turned by their own position and results turned back by the query's, a sink in the denominator; or un-rotated, behind a short
 * causal convolution over time on the projections, with RMS norms over the whole q and k projections, a learned bias by distance and a
 * window that keeps the sequence's first positions) or with a selective scan
 * (per-channel state, input-dependent step and read-out), behind RMS norms whose weight is one number, a causal convolution over
 * time on what every sublayer reads, a softmax-routed mixture whose last router outputs stand for experts that return their input,
 * and a per-layer input looked up by token.
 *
 * Batching contract: that of ktx_seq.h — the T tokens of all scheduled requests are flattened, request b owns rows
 * q_indptr[b] .. q_indptr[b+1], starts at position pos0[b] and keeps its state in slot slot[b]; a token knows its request, its position
 * and its cache row.  The residual stream, norms, angles, scores, softmax, router and everything in a recurrence are fp32 whatever the
 * storage type (KTX_SEQ_BF16 / KTX_SEQ_F32).  DEVICE pointers, enqueue-only on `stream`, 0 = success (ktx_last_error()). */
#ifndef KTX_SWA_H
#define KTX_SWA_H
#include <stddef.h>
#include <stdint.h>

#include "ktx_seq.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- residual update + RMS norm with a scalar weight + rows for an input convolution ---------------------------------------------- */
typedef struct ktx_resid_args {
  /* what is added to x[t] (every part optional):
   *   y[t]                                   fp32 rows of stride ldy; with y_norm_w (fp32 [W]): y[t] / sqrt(mean(y[t]^2) + y_norm_eps) * y_norm_w
   *   sum_k topk_w[t][k] * (topk_idx[t][k] < n_real ? ey[pair_pos[t * top + k]] : h_in[t])
   *                                          ey fp32 [pairs][W]; h_in [T][W] of h_dtype: the mixture's own input, what an expert
   *                                          without weights returns */
  const float* y;
  int64_t ldy;
  const float* y_norm_w;
  float y_norm_eps;
  const float* ey;
  const int32_t* pair_pos;
  const int32_t* topk_idx;
  const float* topk_w;
  int32_t top, n_real;
  const void* h_in;
  int32_t h_dtype;
  /* the norm of the updated row, out = x[t] * g / sqrt(mean(x[t]^2) + eps), g = norm_g[0] (a device scalar); norm_g NULL: no output.
   * rows (int32 [T], optional, only without an addition): out[i] = norm(x[rows[i]]).
   * halo > 0 (requires B, q_indptr, pos0, slot, tok_req, conv_state): out is fp32 [T + B * halo][W]; request b's rows are preceded by
   * `halo` rows holding conv_state[slot[b]] (fp32 [slots][halo][W]; zeros when pos0[b] == 0): token t of request b is row
   * t + (b + 1) * halo — the layout ktx_input_conv reads.
   * conv_w (fp32 [W][conv_taps], instead of halo; same batch tensors; EVERY request brings exactly one token; 2 <= conv_taps <= 9): the
   * input convolution in the same launch — out[t] = h + conv(h) of out_dtype with h = the normed row and the slot's state before it,
   * and the slot's state moves on by one token.  conv_taps == 1 (any step, no batch tensors, no state): out[t] = h + conv_w * h. */
  const float* norm_g;
  float eps;
  const int32_t* rows;
  int32_t halo, B;
  const int32_t* q_indptr;
  const int32_t* pos0;
  const int32_t* slot;
  const int32_t* tok_req;
  float* conv_state;
  const float* conv_w;
  int32_t conv_taps;
  void* out;
  int32_t out_dtype;
} ktx_resid_args;

/* x fp32 [T][W] (updated in place when anything is added); one launch. */
int ktx_resid_norm(int T, int W, float* d_x, const ktx_resid_args* a, ktx_stream_t stream);

/* out[t][c] = hx[r][c] + sum_{j < taps} w[c][j] * hx[r - taps + 1 + j][c], r = t + (b + 1) * (taps - 1) (hx as ktx_resid_norm lays it
 * out with halo = taps - 1; w fp32 [W][taps], the last column multiplies the current token), and the slot's state moves on:
 * conv_state[slot[b]] = the last taps - 1 rows of request b's segment.  out [T][W] of out_dtype.  taps >= 2. */
int ktx_input_conv(int B, int T, int W, int taps, const float* d_hx, const float* d_w, const int32_t* d_q_indptr, const int32_t* d_slot,
                   const int32_t* d_tok_req, float* d_conv_state, void* d_out, int out_dtype, ktx_stream_t stream);

/* out[t][c] = a[t][c] * table[tokens[t]][col0 + c] for c < n: fp32 rows a (stride lda) times a slice of a token-indexed table
 * (table_dtype, row stride ldt) -> [T][n] of out_dtype. */
int ktx_rows_mul_lookup(int T, int n, const float* d_a, int64_t lda, const void* d_table, int table_dtype, int64_t ldt, int col0,
                        const int32_t* d_tokens, void* d_out, int out_dtype, ktx_stream_t stream);

/* ---- grouped-query sliding-window attention over paged key and value caches ----------------------------------------------------- */
typedef struct ktx_swa_config {
  int32_t heads, kv_heads, dim, vdim; /* query heads, key / value heads (heads % kv_heads == 0), per-head sizes of q / k and of v */
  int32_t rot_dims;                   /* the first rot_dims entries of q and k heads turn with the position (pairs 2i, 2i + 1); even */
  int32_t rot_values;                 /* != 0: the value of position j is cached turned by j over all vdim entries (pairs 2m, 2m + 1)
                                         and a head's result at position i is turned back by i; vdim even */
  int32_t qk_norm;                    /* != 0: after the rotation q and k are divided by their RMS over dim (eps inside the root) */
  float eps;
  float scale;                        /* score = scale * (q . k) */
  int32_t window;                     /* position i sees j with 0 <= i - j < window; <= 0: no window */
  int32_t page_size, cache_dtype;     /* caches [rows][kv_heads][dim] and [rows][kv_heads][vdim] of KTX_SEQ_* */
  int32_t keep_first;                 /* with a window: the first keep_first positions of a sequence stay visible to every later one */
  int32_t bias_span;                  /* rows - 1 of the distance-bias table the attention calls take (distances beyond it read its last row) */
} ktx_swa_config;

/* Per token: rotate and norm q (times scale) -> q_out fp32 [T][heads][dim]; rotate and norm k, turn v -> cache rows cache_loc[t];
 * the cosines | sines of the value rotation at the token's position -> vcs fp32 [T][vdim] (read again when results are turned back).
 * Angles = pos * inv_freq[i] in fp64 (inv_freq fp64 [rot_dims / 2], v_inv_freq fp64 [vdim / 2]), rounded once.
 * proj fp32 rows of stride ldp with q, k, v at their offsets. */
int ktx_swa_prep(const ktx_swa_config* cfg, int T, const float* d_proj, int64_t ldp, int q_off, int k_off, int v_off,
                 const double* d_inv_freq, const double* d_v_inv_freq, const int32_t* d_pos, const int32_t* d_cache_loc, void* d_kcache,
                 void* d_vcache, float* d_q_out, float* d_vcs, ktx_stream_t stream);

/* The prep of the un-rotated form whose projections pass a short causal convolution over time: with u = proj[t] + bias (q | k | v, C =
 * heads dim + kv_heads (dim + vdim) channels at column 0 of fp32 rows of stride ldp; bias fp32 [C] or NULL),
 *   y[t][c] = sum_{j < taps} conv_w[c][j] u[t - taps + 1 + j][c]      (conv_w fp32 [C][taps], the last column multiplies the current token;
 *             inputs before a request's first NEW token come from its slot of conv_state fp32 [slots][taps - 1][C] when pos0 > 0 and are
 *             zero otherwise; taps <= 1: y = u, times conv_w when given)
 *   q = y_q / sqrt(mean(y_q^2) + eps) * q_norm_w * scale over ALL heads dim entries at once (q_norm_w fp32 [heads dim] or NULL: no norm),
 *   k likewise with k_norm_w over kv_heads dim entries; q -> q_out fp32 [T][heads][dim], k and v = y_v -> cache rows cache_loc[t].
 * Then (second launch) conv_state[slot[b]] = the last taps - 1 inputs u of request b; with max_q_len == 1 (no request brings more than
 * one token), 2 .. 4 taps and channel counts that are multiples of 4 the state moves on in the first launch.  cfg: rot_dims = 0,
 * rot_values = 0; taps <= 16. */
int ktx_swa_conv_prep(const ktx_swa_config* cfg, int B, int T, int max_q_len, int taps, const float* d_proj, int64_t ldp, const float* d_bias,
                      const float* d_conv_w, const float* d_q_norm_w, const float* d_k_norm_w, const int32_t* d_q_indptr,
                      const int32_t* d_pos0, const int32_t* d_slot, const int32_t* d_tok_req, float* d_conv_state,
                      const int32_t* d_cache_loc, void* d_kcache, void* d_vcache, float* d_q_out, ktx_stream_t stream);

/* out[t][h] = turn_back(sum_j p_j v_j), p = softmax over {q[t][h] . k_j + dist_bias[min(i - j, bias_span)][h] : j visible to t at
 * position i: j <= i and (i - j < window or j < keep_first)} and, with sink (fp32 [heads]), one more score sink[h] that has no value.
 * dist_bias: fp32 [bias_span + 1][heads] or NULL (not scaled: scale is folded into q).  Vector-ALU form, any sizes and either cache type: one token x the query heads of one key head x
 * one key range per workgroup; nsplit key ranges leave partial sums in scratch fp32 [nsplit][T][heads][vdim + 2], merged afterwards.
 * out [T][heads * vdim] of out_dtype. */
int ktx_swa_forward(const ktx_swa_config* cfg, int T, const float* d_q, const void* d_kcache, const void* d_vcache,
                    const int32_t* d_tok_req, const int32_t* d_pos, const int32_t* d_page_indptr, const int32_t* d_page_indices,
                    const float* d_sink, const float* d_dist_bias, const float* d_vcs, int nsplit, float* d_scratch, void* d_out,
                    int out_dtype, ktx_stream_t stream);

/* The same operator on the matrix cores for prompts, portions and decode steps: the (token, head) pairs of a request that share a key
 * head are the rows of one query matrix; workgroups of 64 rows walk 32-key tiles, bf16 MFMA for q . k and weights x values, scores /
 * mask / softmax in fp32.  Eligible: bf16 caches, dim a multiple of 32 up to 256, vdim a multiple of 16 up to 128, or 256. */
int ktx_swa_mfma_eligible(const ktx_swa_config* cfg);
int ktx_swa_mfma(const ktx_swa_config* cfg, int B, int T, int max_q_len, const float* d_q, const void* d_kcache, const void* d_vcache,
                 const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_page_indptr, const int32_t* d_page_indices,
                 const float* d_sink, const float* d_dist_bias, const float* d_vcs, int nsplit, float* d_scratch, void* d_out, int out_dtype,
                 ktx_stream_t stream);

/* ---- selective scan --------------------------------------------------------------------------------------------------------------- */
typedef struct ktx_ssm_config {
  int32_t inner, state, dt_rank; /* channels, state entries per channel, size of the step's low-rank input */
  int32_t taps;                  /* of the causal convolution in front (>= 1) */
} ktx_ssm_config;

/* xc[t][c] = silu(bias[c] + sum_j w[c][j] * xin[t - taps + 1 + j][c]): xin = proj rows (fp32, stride ldp, channel c at x_off + c) of
 * the request's own tokens, its slot of conv_state (fp32 [slots][taps - 1][inner]) before them when pos0 > 0, zeros otherwise.
 * w fp32 [inner][taps], bias fp32 [inner] or NULL.  The state is NOT moved on here (ktx_ssm_scan does it). */
int ktx_ssm_conv(const ktx_ssm_config* cfg, int B, int T, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                 const int32_t* d_tok_req, const float* d_proj, int64_t ldp, int x_off, const float* d_w, const float* d_bias,
                 const float* d_conv_state, float* d_xc, ktx_stream_t stream);

/* Token by token from the slot's state S fp32 [slots][inner][state] (zero when pos0 == 0, whatever the slot holds):
 *   dt = softplus(dt_raw[t][c] + dt_bias[c]);  S[c][n] <- exp(dt A[c][n]) S[c][n] + dt xc[t][c] Bm[t][n];  A = -exp(A_log)
 *   y = sum_n S[c][n] Cm[t][n] + D[c] xc[t][c];  out[t][c] = y * silu(z[t][c])
 * xc fp32 [T][inner]; Bm, Cm fp32 rows of stride ldbc (state entries each); dt_raw fp32 rows of stride lddt; z = proj rows (stride ldp)
 * at z_off.  Afterwards conv_state[slot] = the last taps - 1 convolution inputs (proj at x_off; older ones from the old state).
 * out [T][inner] of out_dtype.  state <= 256. */
int ktx_ssm_scan(const ktx_ssm_config* cfg, int B, int T, int max_q_len, const int32_t* d_q_indptr, const int32_t* d_pos0,
                 const int32_t* d_slot, const float* d_xc, const float* d_Bm, const float* d_Cm, int64_t ldbc, const float* d_dt_raw,
                 int64_t lddt, const float* d_dt_bias, const float* d_A_log, const float* d_D, const float* d_proj, int64_t ldp, int x_off,
                 int z_off, float* d_S, float* d_conv_state, void* d_out, int out_dtype, ktx_stream_t stream);

/* ---- softmax router --------------------------------------------------------------------------------------------------------------- */
/* s = softmax(logits[t]) over all E router outputs (fp32 rows of stride ldl); the `top` largest s + correction (fp32 [E] or NULL; lowest
 * index first on ties) -> topk_idx int32 [T][top]; topk_w fp32 [T][top] = the chosen s (without the correction) over (their sum + sum_eps). */
int ktx_softmax_route(int T, int E, int top, float sum_eps, const float* d_logits, int64_t ldl, const float* d_correction,
                      int32_t* d_topk_idx, float* d_topk_w, ktx_stream_t stream);

/* The same router followed, in the same launch, by the expert sort of ktx_moe_plan (ktx_hyb.h; same outputs, E groups): for small steps
 * (decode), T <= KTX_ROUTE_PLAN_MAX_T, where one workgroup routes and sorts. */
enum { KTX_ROUTE_PLAN_MAX_T = 256 };
int ktx_softmax_route_plan(int T, int E, int top, float sum_eps, const float* d_logits, int64_t ldl, const float* d_correction,
                           int32_t* d_topk_idx, float* d_topk_w, int tile_m, int32_t* d_group_off, int32_t* d_sorted_tok,
                           int32_t* d_pair_pos, int32_t* d_sorted_group, int32_t* d_tile_group, int32_t* d_tile_row0, int32_t* d_num_tiles,
                           ktx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
