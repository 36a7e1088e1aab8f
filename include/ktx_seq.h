/* ktx_seq.h — C ABI of the sequence-mixer kernels (libktx_hip.so): the ops a decoder needs whose token mixers are not
 * softmax attention over a latent cache — a sigmoid-weighted grouped-query attention with head mixing over a paged key
 * cache, a matrix-memory recurrence (mLSTM) over per-sequence state slots — and the fp32-residual glue around them
 * (sinusoidal embedding, RMS norms that add into the residual, a dense GEMM that takes any shape in bf16 or fp32).
 *
 * Batching contract (shared by every entry point): the T tokens of all scheduled requests are flattened, request b owns
 * rows q_indptr[b] .. q_indptr[b+1]; a token knows its request, its position in the sequence and where its key row lives.
 * The residual stream, the scores, the attention weights, the norms and the recurrent state are fp32 whatever the element
 * type of weights, activations and cache (KTX_SEQ_BF16 or KTX_SEQ_F32).
 *
 * DEVICE pointers, enqueue-only on `stream`, 0 = success (ktx_last_error() for the message). */
#ifndef KTX_SEQ_H
#define KTX_SEQ_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#ifndef KTX_STREAM_T_DEFINED
#define KTX_STREAM_T_DEFINED
typedef void* ktx_stream_t; /* hipStream_t */
#endif

enum { KTX_SEQ_F32 = 0, KTX_SEQ_BF16 = 1 };
enum { KTX_ACT_NONE = 0, KTX_ACT_GELU_TANH = 1 };

/* x[t] = embed[tokens[t]] + s(pos[t]),  s(p)[2i] = sin(p * inv_freq[i]),  s(p)[2i+1] = cos(p * inv_freq[i]).
 * inv_freq: fp64 [(width + 1) / 2]; the angle and its sine are evaluated in fp64 and rounded once.  x: fp32 [T][width].
 * d_inv_freq == NULL: x[t] = embed[tokens[t]] alone (d_pos is not read). */
int ktx_embed_sinpos(int T, int width, int vocab, const int32_t* d_tokens, const int32_t* d_pos, const void* d_embed,
                     int embed_dtype, const double* d_inv_freq, float* d_x, ktx_stream_t stream);

/* The gate | up product of a GLU and its activation in one launch, for steps of at most 16 rows: W bf16 [2F][K] with rows ALTERNATING
 * gate_f, up_f;  Y[m][f] = g sigmoid(slope g) (u + up_shift), g = min(gate_f . A[m], limit), u = clamp(up_f . A[m], -limit, limit)
 * (limit = INFINITY: unbounded).  K a multiple of 32, 16-byte aligned rows; A fp32 or bf16 (rounded to bf16 on the way in), Y fp32 or bf16. */
int ktx_dense_gemv_glu(int M, int F, int K, const void* d_A, int a_dtype, int64_t lda, const void* d_W, void* d_Y, int y_dtype, int64_t ldy,
                       float limit, float slope, float up_shift, ktx_stream_t stream);

/* Y[m][n] = act(sum_k A[m][k] * W[n][k]), any M, N, K >= 1.  The product runs in W's type: bf16 MFMA with fp32 accumulation
 * (A rounded to bf16 on the way in when it is fp32) or fp32 MFMA (A must be fp32).  Y is fp32 or bf16.  lda / ldy in elements.
 * ksplit > 1 splits K over ksplit workgroups per tile that add into a ZEROED fp32 Y with atomics (small M; act must be NONE). */
int ktx_dense_gemm(int M, int N, int K, const void* d_A, int a_dtype, int64_t lda, const void* d_W, int w_dtype, void* d_Y,
                   int y_dtype, int64_t ldy, int act, int ksplit, ktx_stream_t stream);

typedef struct ktx_sigattn_config {
  int32_t heads, kv_heads, dim;   /* query heads, key heads (heads % kv_heads == 0), per-head size of q, k and v (v = k) */
  float scale;                    /* score = scale * (q . k) */
  float temp_coef;                /* q *= 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1); 0 switches it off */
  int32_t temp_every;
  float slope_span;               /* distance bias slope_h * (i - j), slope_h = 2^(-slope_span * (h + 1) / heads); 0 = none */
  int32_t page_size;              /* tokens per page of the key cache */
  int32_t cache_dtype;            /* KTX_SEQ_* of the key cache */
} ktx_sigattn_config;

/* Between the q | k projection and the attention: per token and head RMS-norm q (weight wq) and fold the key norm's weight wk,
 * the temperature of the token's position and `scale` into it -> q_out fp32 [T][heads][dim]; store the token's UN-normed key
 * row (it is also the value row) at cache row cache_loc[t] (= page * page_size + offset) of kcache [rows][kv_heads][dim] and
 * 1 / rms(k) per key head in kinv fp32 [rows][kv_heads].  proj: fp32 [T] rows of stride ldp holding q at q_off, k at k_off. */
int ktx_sigattn_prep(const ktx_sigattn_config* cfg, int T, const float* d_proj, int64_t ldp, int q_off, int k_off,
                     const float* d_wq, const float* d_wk, float eps, const int32_t* d_pos, const int32_t* d_cache_loc,
                     void* d_kcache, float* d_kinv, float* d_q_out, ktx_stream_t stream);

/* out[t][h] = sum_{j <= pos[t]} (sum_g talk[h][g] * sigmoid(q[t][g] . k[j][kv(g)] * kinv[j] - slope_g * (pos[t] - j) + pb[g]))
 *             * k[j][kv(h)]   (weights are not normalised over keys, so key ranges simply add).
 * tok_req[t] = request of token t; key j of request b lives in page page_indices[page_indptr[b] + j / page_size].
 * nsplit workgroups share a token's keys; d_partial: fp32 [nsplit][T][heads*dim] scratch when nsplit > 1.
 * out: [T][heads*dim] of out_dtype. */
int ktx_sigattn_forward(const ktx_sigattn_config* cfg, int T, const float* d_q, const void* d_kcache, const float* d_kinv,
                        const int32_t* d_tok_req, const int32_t* d_pos, const int32_t* d_page_indptr,
                        const int32_t* d_page_indices, const float* d_pb, const float* d_talk, int nsplit, float* d_partial,
                        void* d_out, int out_dtype, ktx_stream_t stream);

/* The same operator on the matrix cores, for prompts and for decode steps: request b's query rows q_indptr[b] .. q_indptr[b+1] (at
 * most max_q_len of them; T rows in all) start at position pos0[b]; workgroups of 16 query rows x all heads walk 32-key tiles: bf16
 * MFMA for Q K^T and for weights x values (q rounded to bf16), scores / weights / head mixing in fp32.  nsplit workgroups share a row
 * tile's keys (partial sums in d_partial: fp32 [nsplit][T][heads*dim], then reduced).  out: bf16 [T][heads*dim].
 * Eligible: bf16 cache, dim % 32 == 0, dim <= 128, heads <= 16, tiles fit the LDS; ktx_sigattn_forward serves everything else. */
int ktx_sigattn_prefill_eligible(const ktx_sigattn_config* cfg);
int ktx_sigattn_prefill(const ktx_sigattn_config* cfg, int B, int T, int max_q_len, const float* d_q, const void* d_kcache,
                        const float* d_kinv, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_page_indptr,
                        const int32_t* d_page_indices, const float* d_pb, const float* d_talk, int nsplit, float* d_partial,
                        void* d_out, ktx_stream_t stream);

/* y = gelu_tanh(y) in place, n elements of `dtype` (the activation behind a GEMM that has no epilogue for it). */
int ktx_gelu_tanh(size_t n, void* d_y, int dtype, ktx_stream_t stream);

typedef struct ktx_mlstm_config {
  int32_t heads, dim, vdim;       /* per head: q, k of size dim, v of size vdim; state S [dim][vdim], n [dim], m */
  float gate_cap;                 /* log gates are soft-capped: cap * tanh(z / cap); 0 = no cap */
  float eps;                      /* of the per-head unit norm on the output */
  float denom_eps;                /* o = S^T q / (max(|n . q|, exp(-m)) + denom_eps) */
} ktx_mlstm_config;

/* The recurrence, token by token, for B requests: request b's rows q_indptr[b] .. q_indptr[b+1] of proj (fp32, stride ldp; q at
 * q_off scaled here by dim^-1/2, k at k_off, v at v_off, gate pre-activations at i_off / f_off, biases ib / fb fp32 [heads])
 * continue the state in slot slot[b] — or start from zero (S = 0, n = 0, m = 0) when pos0[b] == 0, whatever the slot holds.
 *   i = cap*tanh((z_i + ib)/cap), f = logsigmoid(cap*tanh((z_f + fb)/cap)), m' = max(f + m, i),
 *   S' = exp(f + m - m') S + exp(i - m') k v^T, n' likewise with k, o = S'^T q / (max(|n' . q|, exp(-m')) + denom_eps).
 * S: fp32 [slots][heads][dim][vdim], n: [slots][heads][dim], m: [slots][heads].  o_raw: fp32 [T][heads*vdim].
 * Two launches: the gates and the running maximum of all new tokens (a scan, off the sequential path) into d_gates, fp32 scratch of
 * (B + 8 T) * heads floats, then the state recurrence — token by token, or, when the longest request brings max_q_len >= 16 tokens,
 * 16 tokens at a time on the fp32 matrix cores (the recurrence unrolled over a chunk; same numbers up to fp32 rounding). */
int ktx_mlstm_forward(const ktx_mlstm_config* cfg, int B, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                      const float* d_proj, int64_t ldp, int q_off, int k_off, int v_off, int i_off, int f_off, const float* d_ib,
                      const float* d_fb, float* d_S, float* d_n, float* d_m, float* d_gates, float* d_o_raw, int max_q_len,
                      ktx_stream_t stream);

/* out[t][h*vdim + v] = o_raw[t][h][v] / rms_h(o_raw[t][h]) * w[h*vdim + v] * sigmoid(proj[t][g_off + h*vdim + v]). */
int ktx_mlstm_gate_norm(const ktx_mlstm_config* cfg, int T, const float* d_o_raw, const float* d_proj, int64_t ldp, int g_off,
                        const float* d_w, void* d_out, int out_dtype, ktx_stream_t stream);

/* Row-wise fp32 norm glue.  u(v) = v / sqrt(mean(v^2) + eps).
 *   z = y2 ? 0.5 * (u(y1) * w1 + u(y2) * w2) : y1        (w1 / w2 fp32 [W], plain weights; y1, y2 fp32 [T][W])
 *   r = u(z) * (one_plus ? 1 + wn : wn)                  (wn NULL: r = z)
 *   x_residual ? x_residual[t] += r : out[t] = r         (out of out_dtype)
 * rows (int32 [T], may be NULL) gathers the input rows of y1. */
int ktx_rms_combine(int T, int W, const float* d_y1, const float* d_w1, const float* d_y2, const float* d_w2, const float* d_wn,
                    int one_plus, float eps, float* d_x_residual, const int32_t* d_rows, void* d_out, int out_dtype,
                    ktx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
