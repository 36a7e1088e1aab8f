// ktx_hyb.hip — hybrid-decoder kernels behind include/ktx_hyb.h: layer norm with bias, the sigmoid-gated post-normed residual update
// (with the mixture's weighted gather folded in), the post-norm on a scaled residual with a depth-weighted average over a stack of
// layer results, PolyNorm, the bounded GLU activation and a sigmoid output gate, the gated delta rule (convolution + unit vectors + decay prep, state update,
// token-by-token recurrence on register-resident state slices), sliding-window softmax attention with a sink over a paged latent cache,
// the sigmoid top-k router with its expert sort, and a grouped GEMM (per-head products and per-expert products) on the matrix cores.
//
// Everything a recurrence, a norm, a router or a score touches is fp32; element types only select how weights, activations and the
// latent cache are stored and which MFMA multiplies them.
#include "ktx_common.h"
#include "../../include/ktx_hyb.h"

#include <math.h>

#include <algorithm>

namespace {

#include "ktx_seq_dev.inc"

__device__ __forceinline__ float silu_f32(float z) { return z / (1.0f + expf(-z)); }
// A workgroup barrier that orders LDS traffic only: the wavefront's own LDS operations have completed, global loads it has in flight
// (a prefetch for a later step) stay in flight — __syncthreads() would wait for them too.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// ---------------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256) rows_add_kernel(size_t n, int W, float* __restrict__ x, const float* __restrict__ x0,
                                                       const float* __restrict__ vec) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float v = x[i];
  if (x0) v += x0[i];
  if (vec) v += vec[i % W];
  x[i] = v;
}

// layer norm of one row per workgroup: mean, then the mean of squared deviations, then the affine map
template <typename OT>
__global__ void __launch_bounds__(256) layer_norm_kernel(int W, const float* __restrict__ x, const float* __restrict__ w,
                                                         const float* __restrict__ b, float eps, const int32_t* __restrict__ rows,
                                                         OT* __restrict__ out) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* a = x + (size_t)(rows ? rows[t] : t) * W;
  float s = 0.f;
  for (int e = tid; e < W; e += 256) s += a[e];
  const float mean = block_sum256(s, red) / (float)W;
  float q = 0.f;
  for (int e = tid; e < W; e += 256) {
    const float d = a[e] - mean;
    q += d * d;
  }
  const float r = 1.0f / sqrtf(block_sum256(q, red) / (float)W + eps);
  for (int e = tid; e < W; e += 256) st_elem(out, (size_t)t * W + e, (a[e] - mean) * r * w[e] + (b ? b[e] : 0.f));
}

// z = (y + ybias + sum_k w_k ey[pos_k]) * sigmoid(gl + gbias); x += LN(z).  The row lives in LDS between the passes.  With nw: the
// layer norm of the UPDATED row (the next sublayer's pre-norm) is written to nout in the same launch.
template <typename OT>
__global__ void __launch_bounds__(256) gated_norm_add_kernel(int W, const float* __restrict__ y, int64_t ldy,
                                                             const float* __restrict__ ybias, const float* __restrict__ ey,
                                                             const int32_t* __restrict__ pair_pos, const float* __restrict__ topk_w,
                                                             int top, const float* __restrict__ gl, int64_t ldg,
                                                             const float* __restrict__ gbias, const float* __restrict__ wn,
                                                             const float* __restrict__ bn, float eps, float* __restrict__ x,
                                                             const float* __restrict__ nw, const float* __restrict__ nb, float neps,
                                                             OT* __restrict__ nout) {
  extern __shared__ float zrow[];
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  float s = 0.f;
  for (int e = tid; e < W; e += 256) {
    float z = y ? y[(size_t)t * ldy + e] : 0.f;
    if (ybias) z += ybias[e];
    if (ey) {
      float m = 0.f;
      for (int k = 0; k < top; k++) m += topk_w[(size_t)t * top + k] * ey[(size_t)pair_pos[(size_t)t * top + k] * W + e];
      z += m;
    }
    if (gl) z *= sigmoid_f32(gl[(size_t)t * ldg + e] + (gbias ? gbias[e] : 0.f));
    zrow[e] = z;
    s += z;
  }
  const float mean = block_sum256(s, red) / (float)W;
  float q = 0.f;
  for (int e = tid; e < W; e += 256) {
    const float d = zrow[e] - mean;
    q += d * d;
  }
  const float r = 1.0f / sqrtf(block_sum256(q, red) / (float)W + eps);
  float s2 = 0.f;
  for (int e = tid; e < W; e += 256) {
    const float v = x[(size_t)t * W + e] + ((zrow[e] - mean) * r * wn[e] + (bn ? bn[e] : 0.f));
    x[(size_t)t * W + e] = v;
    zrow[e] = v;              // (each thread re-reads only what it wrote)
    s2 += v;
  }
  if (!nw) return;
  const float mean2 = block_sum256(s2, red) / (float)W;
  float q2 = 0.f;
  for (int e = tid; e < W; e += 256) {
    const float d = zrow[e] - mean2;
    q2 += d * d;
  }
  const float r2 = 1.0f / sqrtf(block_sum256(q2, red) / (float)W + neps);
  for (int e = tid; e < W; e += 256) st_elem(nout, (size_t)t * W + e, (zrow[e] - mean2) * r2 * nw[e] + (nb ? nb[e] : 0.f));
}

// v = layer_norm(alpha * x + y + ybias); with a stack: level `level` of it receives v, and with dwa the row handed on is the weighted
// sum of levels 0 .. level.  The row lives in LDS between the passes; every level's entry is requested before the sum is formed.
template <typename OT>
__global__ void __launch_bounds__(256) postnorm_mix_kernel(int W, const float* xin, float* xout,
                                                           ktx_postnorm_args a, OT* __restrict__ lp) {
  extern __shared__ float zrow[];
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const size_t ro = (size_t)t * W;
  float s = 0.f;
  for (int e = tid; e < W; e += 256) {
    float z = a.alpha * xin[ro + e];
    if (a.y) z += a.y[(size_t)t * a.ldy + e];
    if (a.ybias) z += a.ybias[e];
    zrow[e] = z;
    s += z;
  }
  const float mean = block_sum256(s, red) / (float)W;
  float q = 0.f;
  for (int e = tid; e < W; e += 256) {
    const float d = zrow[e] - mean;
    q += d * d;
  }
  const float r = 1.0f / sqrtf(block_sum256(q, red) / (float)W + a.eps);
  const int lv = a.level;
  for (int e = tid; e < W; e += 256) {
    float v = (zrow[e] - mean) * r * a.w[e] + (a.b ? a.b[e] : 0.f);
    if (a.stack) {
      a.stack[(size_t)lv * a.stack_stride + ro + e] = v;
      if (a.dwa) {
        float m = a.dwa[lv] * v;
        for (int j0 = 0; j0 < lv; j0 += 8) {
          float part[8];
#pragma unroll
          for (int i = 0; i < 8; i++) part[i] = j0 + i < lv ? a.stack[(size_t)(j0 + i) * a.stack_stride + ro + e] : 0.f;
#pragma unroll
          for (int i = 0; i < 8; i++)
            if (j0 + i < lv) m += a.dwa[j0 + i] * part[i];
        }
        v = m;
      }
    }
    xout[ro + e] = v;
    if (lp) st_elem(lp, ro + e, v);
  }
}

// The same update for rows of at most 256 * EPT entries, held in registers: a thread owns entries tid, tid + 256, ...; every load of
// a phase (x, y and the bias; then the norm's weights and the lower levels of the stack) is requested before the first is used, so a
// one-row launch (a decode step) costs a few memory round trips instead of one per entry.
template <typename OT, int EPT>
__global__ void __launch_bounds__(256) postnorm_mix_reg_kernel(int W, const float* xin, float* xout,
                                                               ktx_postnorm_args a, OT* __restrict__ lp) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const size_t ro = (size_t)t * W;
  float z[EPT], yv[EPT], bv[EPT];
#pragma unroll
  for (int i = 0; i < EPT; i++) {
    const int e = tid + i * 256;
    const bool in = e < W;
    z[i] = in ? xin[ro + e] : 0.f;
    yv[i] = in && a.y ? a.y[(size_t)t * a.ldy + e] : 0.f;
    bv[i] = in && a.ybias ? a.ybias[e] : 0.f;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < EPT; i++) {
    z[i] = (a.alpha * z[i] + yv[i]) + bv[i];
    s += z[i];                                   // (entries beyond W are 0)
  }
  const int lv = a.level;
  const bool avg = a.stack && a.dwa;
  // the norm's weights and the first lower levels of the stack are on their way while the row is reduced
  float wv[EPT], lo[EPT];
#pragma unroll
  for (int i = 0; i < EPT; i++) {
    const int e = tid + i * 256;
    const bool in = e < W;
    wv[i] = in ? a.w[e] : 0.f;
    bv[i] = in && a.b ? a.b[e] : 0.f;
    lo[i] = in && avg && lv > 0 ? a.stack[ro + e] : 0.f;
  }
  const float mean = block_sum256(s, red) / (float)W;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < EPT; i++) {
    const float d = tid + i * 256 < W ? z[i] - mean : 0.f;
    q += d * d;
  }
  const float r = 1.0f / sqrtf(block_sum256(q, red) / (float)W + a.eps);
#pragma unroll
  for (int i = 0; i < EPT; i++) z[i] = (z[i] - mean) * r * wv[i] + bv[i];
  if (a.stack) {
#pragma unroll
    for (int i = 0; i < EPT; i++) {
      const int e = tid + i * 256;
      if (e < W) a.stack[(size_t)lv * a.stack_stride + ro + e] = z[i];
    }
  }
  if (avg) {
    const float wl = a.dwa[lv];
#pragma unroll
    for (int i = 0; i < EPT; i++) z[i] *= wl;
    for (int j = 0; j < lv; j++) {               // level j is in `lo`; level j + 1 is requested before it is used
      const float wj = a.dwa[j];
      float nx[EPT];
#pragma unroll
      for (int i = 0; i < EPT; i++) {
        const int e = tid + i * 256;
        nx[i] = e < W && j + 1 < lv ? a.stack[(size_t)(j + 1) * a.stack_stride + ro + e] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < EPT; i++) {
        z[i] += wj * lo[i];
        lo[i] = nx[i];
      }
    }
  }
#pragma unroll
  for (int i = 0; i < EPT; i++) {
    const int e = tid + i * 256;
    if (e < W) {
      xout[ro + e] = z[i];
      if (lp) st_elem(lp, ro + e, z[i]);
    }
  }
}

template <typename OT>
__global__ void __launch_bounds__(256) poly_norm_kernel(int F, const float* __restrict__ zin, int64_t ldz, const float* __restrict__ bias,
                                                        const float* __restrict__ coef, float eps, OT* __restrict__ out) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* a = zin + (size_t)t * ldz;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int e = tid; e < F; e += 256) {
    const float z = a[e] + (bias ? bias[e] : 0.f), z2 = z * z;
    s1 += z2;
    s2 += z2 * z2;
    s3 += z2 * z2 * z2;
  }
  const float r1 = coef[0] / sqrtf(block_sum256(s1, red) / (float)F + eps);
  const float r2 = coef[1] / sqrtf(block_sum256(s2, red) / (float)F + eps);
  const float r3 = coef[2] / sqrtf(block_sum256(s3, red) / (float)F + eps);
  const float c3 = coef[3];
  for (int e = tid; e < F; e += 256) {
    const float z = a[e] + (bias ? bias[e] : 0.f), z2 = z * z;
    st_elem(out, (size_t)t * F + e, ((z * r1 + z2 * r2) + z2 * z * r3) + c3);
  }
}

// out[r][f] = g * sigmoid(slope * g) * (u + up_shift), g = min(gate, limit), u = clamp(up, -limit, limit); (gate, up) = in[r][f],
// in[r][F + f], or — paired — in[r][2f], in[r][2f + 1]
template <typename OT>
__global__ void __launch_bounds__(256) glu_clamp_rows_kernel(size_t n, int F, const float* __restrict__ in, int64_t ldi, float limit,
                                                             float slope, float up_shift, int paired, OT* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const size_t r = i / F;
  const int f = (int)(i % F);
  const float gv = paired ? in[r * ldi + 2 * f] : in[r * ldi + f], uv = paired ? in[r * ldi + 2 * f + 1] : in[r * ldi + F + f];
  const float g = fminf(gv, limit), u = fminf(fmaxf(uv, -limit), limit);
  st_elem(out, i, g * sigmoid_f32(slope * g) * (u + up_shift));
}

// out[r][c] = o[r][c] * sigmoid(gate[r][c])
template <typename IT, typename OT>
__global__ void __launch_bounds__(256) sigmoid_gate_rows_kernel(size_t n, int N, const IT* __restrict__ o, const float* __restrict__ gate,
                                                                int64_t ldg, OT* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  st_elem(out, i, ld_elem(o, i) * sigmoid_f32(gate[(i / N) * ldg + i % N]));
}

template <typename OT>
__global__ void __launch_bounds__(256) silu_mul_rows_kernel(size_t n, int F, const float* __restrict__ in, int64_t ldi,
                                                            OT* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const size_t r = i / F, f = i % F;
  st_elem(out, i, silu_f32(in[r * ldi + f]) * in[r * ldi + F + f]);
}

// one workgroup per token; a wavefront takes heads wave, wave + 4, ...
template <typename OT>
__global__ void __launch_bounds__(256) head_gate_norm_kernel(int heads, int vdim, float eps, const float* __restrict__ o,
                                                             const float* __restrict__ gate, int64_t ldg, const float* __restrict__ w,
                                                             int w_per_head, int act, OT* __restrict__ out) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int h = wave; h < heads; h += 4) {
    const float* a = o + ((size_t)t * heads + h) * vdim;
    float s = 0.f;
    for (int v = lane; v < vdim; v += 64) s += a[v] * a[v];
    const float r = 1.0f / sqrtf(wave_sum(s) / (float)vdim + eps);
    for (int v = lane; v < vdim; v += 64) {
      const float g = gate[(size_t)t * ldg + h * vdim + v];
      const float ga = act ? silu_f32(g) : sigmoid_f32(g);
      st_elem(out, ((size_t)t * heads + h) * vdim + v, a[v] * r * w[(w_per_head ? h * vdim : 0) + v] * ga);
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// gated delta rule: prep (one workgroup per token)
__global__ void __launch_bounds__(256) delta_prep_kernel(ktx_delta_config c, const int32_t* __restrict__ q_indptr,
                                                         const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                         const int32_t* __restrict__ tok_req, const float* __restrict__ proj, int64_t ldp,
                                                         int q_off, int k_off, int v_off, int b_off, int a_off,
                                                         const float* __restrict__ taps, const float* __restrict__ A_log,
                                                         const float* __restrict__ dt_bias, const float* __restrict__ conv_state,
                                                         float* __restrict__ qkv, float* __restrict__ gb) {
  extern __shared__ float ch[];            // [C] convolved, activated channels of this token
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int GD = c.kv_heads * c.dim, C = 2 * GD + c.heads * c.vdim, K = c.taps;
  const int b = tok_req[t], first = q_indptr[b], i = t - first;
  const bool carried = pos0[b] > 0;
  const float* st = conv_state + (size_t)slot[b] * (K - 1) * C;
  for (int e = tid; e < C; e += 256) {
    const int col = e < GD ? q_off + e : (e < 2 * GD ? k_off + e - GD : v_off + e - 2 * GD);
    float acc = 0.f;
    if (K <= 8) {                          // every load from an address that is always valid, so that none waits for another
      float v[8], w[8];
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int jj = j < K ? j : 0, ii = i - jj;
        const bool live = j < K && (ii >= 0 || carried);
        const float* src = ii >= 0 ? proj + (size_t)(first + ii) * ldp + col : (carried ? st + (size_t)(K - 1 + ii) * C + e : taps);
        v[j] = *src;
        w[j] = taps[(size_t)e * K + (K - 1 - jj)];
        if (!live) v[j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; j++) acc += w[j] * v[j];
    } else {
      for (int j = 0; j < K; j++) {        // input i - j times the tap K - 1 - j
        const int ii = i - j;
        float v = 0.f;
        if (ii >= 0) v = proj[(size_t)(first + ii) * ldp + col];
        else if (carried) v = st[(size_t)(K - 1 + ii) * C + e];
        acc += taps[(size_t)e * K + (K - 1 - j)] * v;
      }
    }
    ch[e] = silu_f32(acc);
  }
  __syncthreads();
  // unit vectors: 2 * kv_heads heads of q | k
  for (int hh = wave; hh < 2 * c.kv_heads; hh += 4) {
    float* a = ch + (size_t)hh * c.dim;
    float s = 0.f;
    for (int d = lane; d < c.dim; d += 64) s += a[d] * a[d];
    float r = 1.0f / sqrtf(wave_sum(s) + c.unit_eps);
    if (hh < c.kv_heads) r *= 1.0f / sqrtf((float)c.dim);
    for (int d = lane; d < c.dim; d += 64) a[d] *= r;
  }
  __syncthreads();
  for (int e = tid; e < C; e += 256) qkv[(size_t)t * C + e] = ch[e];
  float* gbt = gb + (size_t)t * (2 * c.heads + c.kv_heads);
  for (int h = tid; h < c.heads; h += 256) {
    const float a = proj[(size_t)t * ldp + a_off + h] + dt_bias[h];
    gbt[h] = expf(-expf(A_log[h]) * softplus_f32(a));
    gbt[c.heads + h] = sigmoid_f32(proj[(size_t)t * ldp + b_off + h]);
  }
  for (int j = wave; j < c.kv_heads; j += 4) {      // k . q per key head: the recurrence's read-out of the token's own write
    float s = 0.f;
    for (int d = lane; d < c.dim; d += 64) s += ch[(size_t)j * c.dim + d] * ch[GD + (size_t)j * c.dim + d];
    s = wave_sum(s);
    if (lane == 0) gbt[2 * c.heads + j] = s;
  }
}

// the last taps - 1 inputs of every request of the step become its slot's convolution state (thread = request x channel; the old
// entries it still needs lie ahead of the ones it overwrites)
__global__ void __launch_bounds__(256) delta_conv_update_kernel(ktx_delta_config c, const int32_t* __restrict__ q_indptr,
                                                                const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                                const float* __restrict__ proj, int64_t ldp, int q_off, int k_off,
                                                                int v_off, float* __restrict__ conv_state) {
  const int GD = c.kv_heads * c.dim, C = 2 * GD + c.heads * c.vdim, K = c.taps;
  const int b = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
  if (e >= C) return;
  const int first = q_indptr[b], n = q_indptr[b + 1] - first;
  if (n <= 0) return;
  const bool carried = pos0[b] > 0;
  const int col = e < GD ? q_off + e : (e < 2 * GD ? k_off + e - GD : v_off + e - 2 * GD);
  float* st = conv_state + (size_t)slot[b] * (K - 1) * C;
  for (int j = 0; j < K - 1; j++) {
    const int ii = n - (K - 1) + j;
    float v = 0.f;
    if (ii >= 0) v = proj[(size_t)(first + ii) * ldp + col];
    else if (carried) v = st[(size_t)(j + n) * C + e];
    st[(size_t)j * C + e] = v;
  }
}

// the recurrence: workgroup = (request, head, 64 value columns); wavefront = dim / NW rows (NW = 4, 8 or 16), lane = value column; the state
// slice stays in registers; ONE barrier per token: both read-outs (S^T k and S^T q of the decayed state) are taken before the write,
// o = (g S)^T q + u (k . q).  The tokens' inputs are staged through LDS a chunk ahead.
template <int DPW, int NW>
__global__ void __launch_bounds__(NW * 64) delta_fwd_kernel(ktx_delta_config c, const int32_t* __restrict__ q_indptr,
                                                        const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                        const float* __restrict__ qkv, const float* __restrict__ gb,
                                                        float* __restrict__ Sg, float* __restrict__ o) {
  constexpr int DP = NW * DPW, NTH = NW * 64, ROW = 2 * DP + 68;      // per token in LDS: k | q of the key head, the value slice, g, beta, k . q, pad
  constexpr int CH = DPW >= 64 ? 8 : 16;               // tokens per staged chunk
  constexpr int NPER = (CH * ROW + NTH - 1) / NTH;
  __shared__ __attribute__((aligned(16))) float stage[2][CH][ROW];
  __shared__ float red[2][NW][2][64];
  const int VS = (c.vdim + 63) / 64;
  const int vs = blockIdx.x % VS, h = (blockIdx.x / VS) % c.heads, b = blockIdx.x / (VS * c.heads);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int D = c.dim, V = c.vdim, H = c.heads, GD = c.kv_heads * D, C = 2 * GD + H * V;
  const int kh = h / (H / c.kv_heads), NGB = 2 * H + c.kv_heads;
  const int col = vs * 64 + lane;
  const int t0 = q_indptr[b], t1 = q_indptr[b + 1];
  if (t1 <= t0) return;
  float S[DPW];
  float* Sp = Sg + (((size_t)slot[b] * H + h) * D) * V;
  const bool carried = pos0[b] > 0;
#pragma unroll
  for (int r = 0; r < DPW; r++) {
    const int d = wave * DPW + r;
    S[r] = (carried && d < D && col < V) ? Sp[(size_t)d * V + col] : 0.f;
  }
  // The inputs of CH tokens travel global -> registers (fetch, issued a whole chunk ahead: a memory round trip takes about as long as
  // one token's step, so it must not sit on the sequential path) -> LDS (commit, at the end of the chunk before the one that reads them).
  float pre[NPER];
  auto fetch = [&](int ch) {
    const int tc = t0 + ch * CH;
#pragma unroll
    for (int i = 0; i < NPER; i++) {
      const int idx = tid + i * NTH, tok = idx / ROW, e = idx % ROW, t = tc + tok;
      float v = 0.f;
      if (idx < CH * ROW && t < t1) {
        const float* row = qkv + (size_t)t * C;
        if (e < 2 * DP) {
          const int which = e / DP, d = e % DP;          // 0: k, 1: q
          if (d < D) v = row[(which ? 0 : GD) + kh * D + d];
        } else {
          const int m = e - 2 * DP;
          if (m < 64) v = (vs * 64 + m) < V ? row[2 * GD + h * V + vs * 64 + m] : 0.f;
          else if (m < 67) v = gb[(size_t)t * NGB + (m == 64 ? h : (m == 65 ? H + h : 2 * H + kh))];
        }
      }
      pre[i] = v;
    }
  };
  auto commit = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NPER; i++) {
      const int idx = tid + i * NTH;
      if (idx < CH * ROW) (&stage[buf][0][0])[idx] = pre[i];
    }
  };
  const int nch = (t1 - t0 + CH - 1) / CH;
  fetch(0);
  commit(0);
  if (nch > 1) fetch(1);
  __syncthreads();
  for (int ch = 0; ch < nch; ch++) {
    const int buf = ch & 1, tc = t0 + ch * CH, n = min(CH, t1 - tc);
    for (int i = 0; i < n; i++) {
      const int par = i & 1, t = tc + i;
      const float* kq = stage[buf][i];
      const float g = kq[2 * DP + 64], beta = kq[2 * DP + 65], kdq = kq[2 * DP + 66], val = kq[2 * DP + lane];
      float kr[DPW];
      float pk = 0.f, pq = 0.f, pk1 = 0.f, pq1 = 0.f;
      const float4* k4p = reinterpret_cast<const float4*>(kq + wave * DPW);       // 16-byte LDS reads, the same address in every lane
      const float4* q4p = reinterpret_cast<const float4*>(kq + DP + wave * DPW);
#pragma unroll
      for (int r4 = 0; r4 < DPW / 4; r4++) {
        const float4 k4 = k4p[r4], q4 = q4p[r4];
        const int r = r4 * 4;
        kr[r] = k4.x; kr[r + 1] = k4.y; kr[r + 2] = k4.z; kr[r + 3] = k4.w;
        S[r] *= g; S[r + 1] *= g; S[r + 2] *= g; S[r + 3] *= g;
        pk = fmaf(k4.x, S[r], pk); pk1 = fmaf(k4.y, S[r + 1], pk1); pk = fmaf(k4.z, S[r + 2], pk); pk1 = fmaf(k4.w, S[r + 3], pk1);
        pq = fmaf(q4.x, S[r], pq); pq1 = fmaf(q4.y, S[r + 1], pq1); pq = fmaf(q4.z, S[r + 2], pq); pq1 = fmaf(q4.w, S[r + 3], pq1);
      }
      pk += pk1;
      pq += pq1;
      red[par][wave][0][lane] = pk;
      red[par][wave][1][lane] = pq;
      lds_barrier();
      float kS = 0.f, qS = 0.f;
#pragma unroll
      for (int w = 0; w < NW; w++) {
        kS += red[par][w][0][lane];
        qS += red[par][w][1][lane];
      }
      const float u = beta * (val - kS);
#pragma unroll
      for (int r = 0; r < DPW; r++) S[r] = fmaf(kr[r], u, S[r]);
      if (wave == 0 && col < V) o[((size_t)t * H + h) * V + col] = fmaf(u, kdq, qS);
    }
    if (ch + 1 < nch) {
      commit(buf ^ 1);          // (every wavefront has passed the last barrier of chunk ch - 1, whose tokens this buffer held)
      if (ch + 2 < nch) fetch(ch + 2);
      lds_barrier();
    }
  }
#pragma unroll
  for (int r = 0; r < DPW; r++) {
    const int d = wave * DPW + r;
    if (d < D && col < V) Sp[(size_t)d * V + col] = S[r];
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// latent attention: prep (one workgroup per token)
template <typename KT>
__global__ void __launch_bounds__(256) latattn_prep_kernel(ktx_latattn_config c, const float* __restrict__ proj, int64_t ldp, int q_off,
                                                           int c_off, const float* __restrict__ wn, const double* __restrict__ inv_freq,
                                                           const int32_t* __restrict__ pos, const int32_t* __restrict__ cache_loc,
                                                           KT* __restrict__ cache, float* __restrict__ q_out) {
  extern __shared__ float cs[];            // cos | sin of the rot_dims / 2 angles
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int L = c.kv_rank, R = c.rot_dim, E = L + R, NP = c.rot_dims / 2;
  const double p = (double)pos[t];
  for (int i = tid; i < NP; i += 256) {
    const double a = p * inv_freq[i];
    cs[i] = (float)cos(a);
    cs[NP + i] = (float)sin(a);
  }
  // rotated parts: entry j of a rotated vector; j < rot_dims turns with its partner — its neighbour (pairs 2i, 2i + 1), or, in the
  // half layout, the entry rot_dims / 2 further on (pairs i, i + rot_dims / 2)
  const bool half = c.rot_half != 0;
  auto turned = [&](const float* v, int j) -> float {
    if (j >= 2 * NP) return v[j];
    if (half) {
      const int i = j < NP ? j : j - NP;
      const float a = v[i], bb = v[i + NP];
      return j < NP ? a * cs[i] - bb * cs[NP + i] : bb * cs[i] + a * cs[NP + i];
    }
    const int i = j >> 1;
    const float a = v[2 * i], bb = v[2 * i + 1];
    return (j & 1) ? bb * cs[i] + a * cs[NP + i] : a * cs[i] - bb * cs[NP + i];
  };
  if (cache) {                               // (a layer that reads another layer's latent rows has none of its own to append)
    const float* lat = proj + (size_t)t * ldp + c_off;
    float s = 0.f;
    for (int e = tid; e < L; e += 256) s += lat[e] * lat[e];
    const float r = 1.0f / sqrtf(block_sum256(s, red) / (float)L + c.eps);      // (its barriers also publish cs)
    KT* row = cache + (size_t)cache_loc[t] * E;
    for (int e = tid; e < L; e += 256) st_elem(row, e, lat[e] * r * wn[e]);
    for (int j = tid; j < R; j += 256) st_elem(row, L + j, turned(lat + L, j));
  } else {
    __syncthreads();
  }
  const int D = c.dim;
  for (int e = tid; e < c.heads * R; e += 256) {
    const int h = e / R, j = e % R;
    q_out[((size_t)t * c.heads + h) * E + L + j] = turned(proj + (size_t)t * ldp + q_off + (size_t)h * (D + R) + D, j);
  }
}

// attention of ONE token (blockIdx.x) x a group of HG heads (blockIdx.y) x one key range (blockIdx.z) on the vector ALUs: tiles of
// KTN <= 64 keys staged in LDS as fp32; scores thread = (head, key); running maximum / sum per head by wavefronts; outputs thread =
// (head, latent entry) in registers.
constexpr int LA_NACC = 32;
template <typename KT, typename OT>
__global__ void __launch_bounds__(256) latattn_fwd_kernel(ktx_latattn_config c, int T, int HG, int KTN, const float* __restrict__ q,
                                                          const KT* __restrict__ cache, const int32_t* __restrict__ tok_req,
                                                          const int32_t* __restrict__ pos, const int32_t* __restrict__ page_indptr,
                                                          const int32_t* __restrict__ page_indices, const float* __restrict__ sink,
                                                          int nsplit, float* __restrict__ scratch, OT* __restrict__ out) {
  extern __shared__ float lds[];
  const int L = c.kv_rank, E = L + c.rot_dim, EP = E + 1;
  float* qs = lds;                         // [HG][E]
  float* kt = qs + (size_t)HG * E;         // [KTN][EP]
  float* sc = kt + (size_t)KTN * EP;       // [HG][KTN]
  float* mrow = sc + (size_t)HG * KTN;     // [HG] running maximum
  float* lrow = mrow + HG;                 // [HG] running sum
  float* crow = lrow + HG;                 // [HG] correction of this tile
  int* rowidx = reinterpret_cast<int*>(crow + HG);   // [KTN]
  const int t = blockIdx.x, h0 = blockIdx.y * HG, z = blockIdx.z;
  const int nh = min(HG, c.heads - h0);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int p = pos[t], b = tok_req[t];
  const int jlo = c.window > 0 ? max(0, p - c.window + 1) : 0, jhi = p + 1;
  const int per = (jhi - jlo + nsplit - 1) / nsplit;
  const int j0 = jlo + z * per, j1 = min(jhi, j0 + per);
  for (int e = tid; e < nh * E; e += 256) qs[e] = q[((size_t)t * c.heads + h0) * E + e];
  for (int h = tid; h < HG; h += 256) {
    mrow[h] = -INFINITY;
    lrow[h] = 0.f;
  }
  float acc[LA_NACC];
#pragma unroll
  for (int i = 0; i < LA_NACC; i++) acc[i] = 0.f;
  const int nout = nh * L;
  const int32_t* pages = page_indices + page_indptr[b];
  for (int jt = j0; jt < j1; jt += KTN) {
    const int nk = min(KTN, j1 - jt);
    __syncthreads();
    if (tid < nk) {
      const int j = jt + tid;
      rowidx[tid] = pages[j / c.page_size] * c.page_size + j % c.page_size;
    }
    __syncthreads();
    for (int e = tid; e < nk * E; e += 256) {
      const int j = e / E, d = e % E;
      kt[(size_t)j * EP + d] = ld_elem(cache, (size_t)rowidx[j] * E + d);
    }
    __syncthreads();
    for (int e = tid; e < nh * KTN; e += 256) {
      const int h = e / KTN, j = e % KTN;
      if (j < nk) {
        const float* qh = qs + (size_t)h * E;
        const float* kj = kt + (size_t)j * EP;
        float s = 0.f;
        for (int d = 0; d < E; d++) s += qh[d] * kj[d];
        sc[(size_t)h * KTN + j] = s * c.scale;
      }
    }
    __syncthreads();
    for (int h = wave; h < nh; h += 4) {
      const float s = lane < nk ? sc[(size_t)h * KTN + lane] : -INFINITY;
      const float mo = mrow[h];
      const float mn = fmaxf(mo, wave_max(s));
      const float w = lane < nk ? expf(s - mn) : 0.f;
      const float sum = wave_sum(w);
      if (lane < nk) sc[(size_t)h * KTN + lane] = w;
      if (lane == 0) {
        const float cr = mo == -INFINITY ? 0.f : expf(mo - mn);
        crow[h] = cr;
        mrow[h] = mn;
        lrow[h] = lrow[h] * cr + sum;
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < LA_NACC; i++) {
      const int e = tid + i * 256;
      if (e < nout) {
        const int h = e / L, l = e % L;
        float a = acc[i] * crow[h];
        const float* w = sc + (size_t)h * KTN;
        for (int j = 0; j < nk; j++) a += w[j] * kt[(size_t)j * EP + l];
        acc[i] = a;
      }
    }
  }
  __syncthreads();
  if (nsplit == 1) {
#pragma unroll
    for (int i = 0; i < LA_NACC; i++) {
      const int e = tid + i * 256;
      if (e < nout) {
        const int h = e / L, l = e % L;
        const float m = mrow[h];
        if (sink) {
          const float sk = sink[h0 + h], M = fmaxf(m, sk);
          const float f = m == -INFINITY ? 0.f : expf(m - M);
          st_elem(out, ((size_t)t * c.heads + h0 + h) * L + l, acc[i] * f / (lrow[h] * f + expf(sk - M)));
        } else {
          st_elem(out, ((size_t)t * c.heads + h0 + h) * L + l, lrow[h] > 0.f ? acc[i] / lrow[h] : 0.f);
        }
      }
    }
    return;
  }
  float* part = scratch + (((size_t)z * T + t) * c.heads + h0) * (L + 2);
#pragma unroll
  for (int i = 0; i < LA_NACC; i++) {
    const int e = tid + i * 256;
    if (e < nout) part[(size_t)(e / L) * (L + 2) + e % L] = acc[i];
  }
  for (int h = tid; h < nh; h += 256) {
    part[(size_t)h * (L + 2) + L] = mrow[h];
    part[(size_t)h * (L + 2) + L + 1] = lrow[h];
  }
}

// merge the key ranges of one (token, head): thread = latent entry; the ranges' (maximum, sum) pairs are fetched in parallel first
template <typename OT>
__global__ void __launch_bounds__(256) latattn_merge_kernel(int T, int H, int L, int nsplit, const float* __restrict__ scratch,
                                                            const float* __restrict__ sink, OT* __restrict__ out) {
  extern __shared__ float mw[];            // [nsplit] maxima, then [nsplit] weights exp(m_z - M) (0 for an empty range)
  float* ws = mw + nsplit;
  const int t = blockIdx.x, h = blockIdx.y;
  const size_t stride = (size_t)T * H * (L + 2);
  const float* base = scratch + ((size_t)t * H + h) * (L + 2);
  for (int z = threadIdx.x; z < nsplit; z += 256) {
    mw[z] = base[z * stride + L];
    ws[z] = base[z * stride + L + 1];
  }
  __syncthreads();
  float M = sink ? sink[h] : -INFINITY;
  for (int z = 0; z < nsplit; z++) M = fmaxf(M, mw[z]);
  float den = sink ? expf(sink[h] - M) : 0.f;
  for (int z = 0; z < nsplit; z++) den += mw[z] == -INFINITY ? 0.f : ws[z] * expf(mw[z] - M);
  __syncthreads();
  for (int z = threadIdx.x; z < nsplit; z += 256) ws[z] = mw[z] == -INFINITY ? 0.f : expf(mw[z] - M);
  __syncthreads();
  const float inv = den > 0.f ? 1.0f / den : 0.f;
  for (int l = threadIdx.x; l < L; l += 256) {
    float a = 0.f;
#pragma unroll 4
    for (int z = 0; z < nsplit; z++) a = fmaf(base[z * stride + l], ws[z], a);
    st_elem(out, ((size_t)t * H + h) * L + l, a * inv);
  }
}

// The same attention on the matrix cores (bf16 latent cache).  The latent rows are keys AND values of every head, so the (token, head)
// pairs of a request are the rows of one long query matrix against shared keys: a workgroup takes 64 consecutive rows (its four
// wavefronts one 16-row MFMA tile each, query fragments resident in registers) and walks 32-key tiles of the union of its rows'
// windows: the tile is staged once in LDS row-major (scores) and transposed (values); scores, mask, running maximum and sum in fp32
// (DPP reductions inside the 16-lane column groups), weights through a per-wavefront LDS tile into the second product.  Key ranges
// (blockIdx.z) leave unnormalised partial sums that latattn_merge_kernel joins with the sink.
constexpr int LM_KT = 32, LM_PST = LM_KT + 8;
template <int NT, typename OT>
__global__ void __launch_bounds__(256) latattn_mfma_kernel(ktx_latattn_config c, int T, int row_tiles, const float* __restrict__ q,
                                                           const bf16_t* __restrict__ cache, const int32_t* __restrict__ q_indptr,
                                                           const int32_t* __restrict__ pos0, const int32_t* __restrict__ page_indptr,
                                                           const int32_t* __restrict__ page_indices, const float* __restrict__ sink,
                                                           int nsplit, float* __restrict__ scratch, OT* __restrict__ out) {
  constexpr int L = NT * 16, KSMAX = NT / 2 + 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char lm_raw[];
  const int H = c.heads, E = L + c.rot_dim, EP = (E + 31) & ~31, EPP = EP + 8, KS = EP / 32;
  bf16_t* Ks = reinterpret_cast<bf16_t*>(lm_raw);            // [LM_KT][EPP]
  bf16_t* Vt = Ks + (size_t)LM_KT * EPP;                      // [L][LM_PST]
  bf16_t* Ps = Vt + (size_t)L * LM_PST;                       // [4][16][LM_PST]
  int* rowidx = reinterpret_cast<int*>(Ps + 4 * 16 * LM_PST); // [LM_KT]
  const int b = blockIdx.x / row_tiles, rt = blockIdx.x % row_tiles, z = blockIdx.z;
  const int t0 = q_indptr[b], rows_total = (q_indptr[b + 1] - t0) * H, r0 = rt * 64;
  if (r0 >= rows_total) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
  const int p0 = pos0[b];
  const int tok_lo = r0 / H, tok_hi = (min(rows_total, r0 + 64) - 1) / H;
  const int klo = c.window > 0 ? max(0, p0 + tok_lo - c.window + 1) : 0, khi = p0 + tok_hi + 1;
  const int per = (((khi - klo + nsplit - 1) / nsplit) + LM_KT - 1) / LM_KT * LM_KT;
  const int j0 = klo + z * per, j1 = min(khi, j0 + per);
  const int rw0 = r0 + wave * 16;
  const bool active = rw0 < rows_total;
  // query fragments: lane = (row l16, 8 consecutive entries lq * 8 ..) of every 32-entry step
  sq_v8bf qf[KSMAX];
  {
    const int ar = rw0 + l16;
    const bool live = ar < rows_total;
    const float* qrow = q + ((size_t)t0 * H + (live ? ar : rows_total - 1)) * E;       // (E % 8 == 0: 16-byte pieces stay inside the row)
#pragma unroll
    for (int kk = 0; kk < KSMAX; kk++) {
      float v[8];
      const int e0 = kk * 32 + lq * 8;
      if (kk < KS && e0 < E) {
        const float4 x = *reinterpret_cast<const float4*>(qrow + e0), y = *reinterpret_cast<const float4*>(qrow + e0 + 4);
        v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w; v[4] = y.x; v[5] = y.y; v[6] = y.z; v[7] = y.w;
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = 0.f;
      }
      if (!live) {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = 0.f;
      }
      union { uint4 u; sq_v8bf f; } cv;
      cv.u.x = ktx_pk_bf16(v[0], v[1]); cv.u.y = ktx_pk_bf16(v[2], v[3]); cv.u.z = ktx_pk_bf16(v[4], v[5]); cv.u.w = ktx_pk_bf16(v[6], v[7]);
      qf[kk] = cv.f;
    }
  }
  // the four rows this lane holds of the score / output tiles (C layout: row lq * 4 + r, column l16)
  int prow[4], lorow[4], hrow[4];
  bool vrow[4];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int cr = rw0 + lq * 4 + r;
    vrow[r] = cr < rows_total;
    prow[r] = p0 + cr / H;
    hrow[r] = cr % H;
    lorow[r] = c.window > 0 ? max(0, prow[r] - c.window + 1) : 0;
  }
  float mrun[4], lrun[4];
  v4f acc[NT];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    mrun[r] = -INFINITY;
    lrun[r] = 0.f;
  }
#pragma unroll
  for (int n = 0; n < NT; n++) acc[n] = (v4f){0.f, 0.f, 0.f, 0.f};
  const int32_t* pages = page_indices + page_indptr[b];
  const int segs = EP / 8;
  bf16_t* Pw = Ps + (size_t)wave * 16 * LM_PST;
  for (int jt = j0; jt < j1; jt += LM_KT) {
    const int nk = min(LM_KT, j1 - jt);
    __syncthreads();
    if (tid < LM_KT) {
      const int j = jt + tid;
      rowidx[tid] = tid < nk ? pages[j / c.page_size] * c.page_size + j % c.page_size : -1;
    }
    __syncthreads();
    for (int idx = tid; idx < LM_KT * segs; idx += 256) {
      const int key = idx / segs, e0 = (idx % segs) * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      const int row = rowidx[key];
      if (row >= 0 && e0 < E) v = *reinterpret_cast<const uint4*>(cache + (size_t)row * E + e0);
      *reinterpret_cast<uint4*>(Ks + (size_t)key * EPP + e0) = v;
      if (e0 < L) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 8; i++) Vt[(size_t)(e0 + i) * LM_PST + key] = (bf16_t)((w[i >> 1] >> ((i & 1) * 16)) & 0xffffu);
      }
    }
    __syncthreads();
    if (active) {
      v4f s0 = (v4f){0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
      for (int kk = 0; kk < KSMAX; kk++) {
        if (kk < KS) {
          const sq_v8bf b0 = *reinterpret_cast<const sq_v8bf*>(Ks + (size_t)l16 * EPP + kk * 32 + lq * 8);
          const sq_v8bf b1 = *reinterpret_cast<const sq_v8bf*>(Ks + (size_t)(16 + l16) * EPP + kk * 32 + lq * 8);
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[kk], b0, s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[kk], b1, s1, 0, 0, 0);
        }
      }
      const int ja = jt + l16, jb = ja + 16;
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const bool oka = vrow[r] && ja < j1 && ja >= lorow[r] && ja <= prow[r];
        const bool okb = vrow[r] && jb < j1 && jb >= lorow[r] && jb <= prow[r];
        const float sa = oka ? s0[r] * c.scale : -INFINITY, sb = okb ? s1[r] * c.scale : -INFINITY;
        const float mt = row16_max(fmaxf(sa, sb));
        const float mn = fmaxf(mrun[r], mt);
        const float base = mn == -INFINITY ? 0.f : mn;
        const float wa = oka ? __expf(sa - base) : 0.f, wb = okb ? __expf(sb - base) : 0.f;
        const float cr = mrun[r] == -INFINITY ? 0.f : __expf(mrun[r] - base);
        lrun[r] = lrun[r] * cr + row16_sum(wa + wb);
        mrun[r] = mn;
#pragma unroll
        for (int n = 0; n < NT; n++) acc[n][r] *= cr;
        Pw[(lq * 4 + r) * LM_PST + l16] = to_bf16_rne(wa);
        Pw[(lq * 4 + r) * LM_PST + 16 + l16] = to_bf16_rne(wb);
      }
    }
    __syncthreads();
    if (active) {
      const sq_v8bf pf = *reinterpret_cast<const sq_v8bf*>(Pw + (size_t)l16 * LM_PST + lq * 8);
#pragma unroll
      for (int n = 0; n < NT; n++) {
        const sq_v8bf vb = *reinterpret_cast<const sq_v8bf*>(Vt + (size_t)(n * 16 + l16) * LM_PST + lq * 8);
        acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vb, acc[n], 0, 0, 0);
      }
    }
  }
  if (!active) return;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    if (!vrow[r]) continue;
    const int cr = rw0 + lq * 4 + r;
    const size_t grow = (size_t)t0 * H + cr;             // (token, head) row of q / out
    if (nsplit == 1) {
      float inv;
      if (sink) {
        const float sk = sink[hrow[r]], M = fmaxf(mrun[r], sk);
        const float f = mrun[r] == -INFINITY ? 0.f : expf(mrun[r] - M);
        inv = f / (lrun[r] * f + expf(sk - M));
      } else {
        inv = lrun[r] > 0.f ? 1.0f / lrun[r] : 0.f;
      }
#pragma unroll
      for (int n = 0; n < NT; n++) st_elem(out, grow * L + n * 16 + l16, acc[n][r] * inv);
    } else {
      float* part = scratch + ((size_t)z * T * H + grow) * (L + 2);
#pragma unroll
      for (int n = 0; n < NT; n++) part[n * 16 + l16] = acc[n][r];
      if (l16 == 0) {
        part[L] = mrun[r];
        part[L + 1] = lrun[r];
      }
    }
  }
}

size_t latattn_mfma_lds(const ktx_latattn_config& c) {
  const int E = c.kv_rank + c.rot_dim, EP = (E + 31) & ~31;
  return ((size_t)LM_KT * (EP + 8) + (size_t)c.kv_rank * LM_PST + 4 * 16 * LM_PST) * 2 + LM_KT * 4;
}

// ---------------------------------------------------------------------------------------------------------------------
// router: one wavefront per token; lane holds experts lane, lane + 64, ... (E <= 64 * RE)
constexpr int MOE_RE = 16;
__global__ void __launch_bounds__(256) moe_route_kernel(int T, int E, int top, float scale, float sum_eps,
                                                        const float* __restrict__ logits, int64_t ldl, int32_t* __restrict__ idx,
                                                        float* __restrict__ wts) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= T) return;
  float s[MOE_RE];
#pragma unroll
  for (int i = 0; i < MOE_RE; i++) {
    const int e = lane + i * 64;
    s[i] = e < E ? sigmoid_f32(logits[(size_t)t * ldl + e]) : -1.f;
  }
  float sum = 0.f, mine = 0.f;      // lane k keeps the k-th choice's score
  int mine_e = 0;
  for (int k = 0; k < top; k++) {
    float bv = -1.f;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MOE_RE; i++) {
      const int e = lane + i * 64;
      if (s[i] > bv) {
        bv = s[i];
        be = e;
      }
    }
    for (int off = 32; off; off >>= 1) {
      const float ov = __shfl_xor(bv, off);
      const int oe = __shfl_xor(be, off);
      if (ov > bv || (ov == bv && oe < be)) {
        bv = ov;
        be = oe;
      }
    }
#pragma unroll
    for (int i = 0; i < MOE_RE; i++)
      if (lane + i * 64 == be) s[i] = -1.f;
    sum += bv;
    if ((k & 63) == lane) {
      mine = bv;
      mine_e = be;
    }
    if ((k & 63) == 63 || k == top - 1) {      // flush up to 64 choices
      const int base = k & ~63;
      if (base + lane <= k) {
        idx[(size_t)t * top + base + lane] = mine_e;
        wts[(size_t)t * top + base + lane] = mine;     // normalised below
      }
    }
  }
  const float f = scale / (sum + sum_eps);
  for (int k = lane; k < top; k += 64) wts[(size_t)t * top + k] *= f;
}

// one workgroup sorts the pairs by expert (counting sort in LDS) and lays the row tiles out (moe_plan_block, ktx_seq_dev.inc)
__global__ void __launch_bounds__(1024) moe_plan_kernel(int pairs, int E, int top, int tile_m, const int32_t* __restrict__ idx,
                                                        int32_t* __restrict__ group_off, int32_t* __restrict__ sorted_tok,
                                                        int32_t* __restrict__ pair_pos, int32_t* __restrict__ sorted_group,
                                                        int32_t* __restrict__ tile_group, int32_t* __restrict__ tile_row0,
                                                        int32_t* __restrict__ num_tiles) {
  extern __shared__ int32_t pl[];          // counts [E] | offsets [E + 1] | cursor [E]
  moe_plan_block(pairs, E, top, tile_m, idx, group_off, sorted_tok, pair_pos, sorted_group, tile_group, tile_row0, num_tiles, pl);
}

// ---------------------------------------------------------------------------------------------------------------------
// grouped GEMM: the 64 x 64 x 32 tile of the dense kernel; a tile belongs to one group (its weights), rows may be gathered
template <typename AT, typename CT>
__device__ __forceinline__ void gg_stage_rows(CT* dst, const AT* __restrict__ src, int64_t ld, const int32_t* __restrict__ rows,
                                              int row0, int row_end, int k0, int K, bool vec) {
  const int r = threadIdx.x >> 2, seg = (threadIdx.x & 3) * 8;
  const int gr = row0 + r;
  CT* d = dst + r * GemmTraits<CT>::LDS_LD + seg;
  const bool live = gr < row_end;
  const size_t srow = live ? (size_t)(rows ? rows[gr] : gr) : 0;
  if (live && vec && k0 + seg + 8 <= K) {
    const AT* s = src + srow * ld + k0 + seg;
    if constexpr (sizeof(AT) == 2 && sizeof(CT) == 2) {
      *reinterpret_cast<uint4*>(d) = *reinterpret_cast<const uint4*>(s);
    } else if constexpr (sizeof(AT) == 4 && sizeof(CT) == 2) {
      const float4 a = *reinterpret_cast<const float4*>(s), b = *reinterpret_cast<const float4*>(s + 4);
      uint4 o;
      o.x = ktx_pk_bf16(a.x, a.y); o.y = ktx_pk_bf16(a.z, a.w); o.z = ktx_pk_bf16(b.x, b.y); o.w = ktx_pk_bf16(b.z, b.w);
      *reinterpret_cast<uint4*>(d) = o;
    } else {
      const float4 a = *reinterpret_cast<const float4*>(s), b = *reinterpret_cast<const float4*>(s + 4);
      d[0] = a.x; d[1] = a.y; d[2] = a.z; d[3] = a.w; d[4] = b.x; d[5] = b.y; d[6] = b.z; d[7] = b.w;
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int k = k0 + seg + i;
    float v = 0.f;
    if (live && k < K) v = ld_elem(src, srow * ld + k);
    if constexpr (sizeof(CT) == 2) d[i] = to_bf16_rne(v);
    else d[i] = v;
  }
}

// epilogue of the grouped products: KTX_GG_ACT_RELU_SQ squares the positive part
__device__ __forceinline__ float gg_act(float v, int act) {
  if (act == KTX_GG_ACT_RELU_SQ) {
    const float r = fmaxf(v, 0.f);
    return r * r;
  }
  return v;
}

template <typename AT, typename CT, typename YT>
__global__ void __launch_bounds__(256) grouped_gemm_kernel(int M, int N, int K, const AT* __restrict__ A, int64_t lda, int64_t a_goff,
                                                           const int32_t* __restrict__ a_rows, const CT* __restrict__ W,
                                                           YT* __restrict__ Y, int64_t ldy, int64_t y_goff,
                                                           const int32_t* __restrict__ group_off, const int32_t* __restrict__ tile_group,
                                                           const int32_t* __restrict__ tile_row0, const int32_t* __restrict__ num_tiles,
                                                           bool vec_a, bool vec_w, int G, int act) {
  constexpr int LD = GemmTraits<CT>::LDS_LD;
  __shared__ __attribute__((aligned(16))) CT As[64 * LD];
  __shared__ __attribute__((aligned(16))) CT Ws[64 * LD];
  int g, m0, m_end;
  if (group_off) {
    if ((int)blockIdx.y >= num_tiles[0]) return;
    g = tile_group[blockIdx.y];
    if (g >= G) return;                  // a group without weights (its rows are the caller's to fill)
    m0 = tile_row0[blockIdx.y];
    m_end = group_off[g + 1];
  } else {
    g = blockIdx.z;
    m0 = blockIdx.y * 64;
    m_end = M;
    A += a_goff * g;
    Y += y_goff * g;
  }
  const CT* Wg = W + (size_t)g * N * K;
  const int n0 = blockIdx.x * 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  const int l16 = lane & 15, lq = lane >> 4;
  v4f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    __syncthreads();
    gg_stage_rows<AT, CT>(As, A, lda, a_rows, m0, m_end, k0, K, vec_a);
    gemm_stage<CT, CT>(Ws, Wg, (int64_t)K, n0, N, k0, K, vec_w);
    __syncthreads();
    if constexpr (sizeof(CT) == 2) {
      sq_v8bf af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; i++) {
        af[i] = *reinterpret_cast<const sq_v8bf*>(As + (wm + i * 16 + l16) * LD + lq * 8);
        bf[i] = *reinterpret_cast<const sq_v8bf*>(Ws + (wn + i * 16 + l16) * LD + lq * 8);
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    } else {
#pragma unroll
      for (int kk = 0; kk < 32; kk += 4) {
        float af[2], bf[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
          af[i] = As[(wm + i * 16 + l16) * LD + kk + lq];
          bf[i] = Ws[(wn + i * 16 + l16) * LD + kk + lq];
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[i], bf[j], acc[i][j], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int m = m0 + wm + i * 16 + lq * 4 + r, n = n0 + wn + j * 16 + l16;
        if (m < m_end && n < N) st_elem(Y, (size_t)m * ldy + n, gg_act(acc[i][j][r], act));
      }
}

// the ragged form for prompts: a 128 x 128 x 32 tile (bf16 MFMA), four wavefronts of 64 x 64 = 4 x 4 MFMA tiles — four times the
// products per LDS fragment read of the 64 x 64 tile; tiles of 128 sorted rows come from ktx_moe_plan(tile_m = 128)
template <typename AT, typename YT>
__global__ void __launch_bounds__(256) grouped_gemm128_kernel(int N, int K, const AT* __restrict__ A, int64_t lda,
                                                              const int32_t* __restrict__ a_rows, const bf16_t* __restrict__ W,
                                                              YT* __restrict__ Y, int64_t ldy, const int32_t* __restrict__ group_off,
                                                              const int32_t* __restrict__ tile_group, const int32_t* __restrict__ tile_row0,
                                                              const int32_t* __restrict__ num_tiles, bool vec_a, bool vec_w, int G,
                                                              int act) {
  constexpr int LD = GemmTraits<bf16_t>::LDS_LD;
  __shared__ __attribute__((aligned(16))) bf16_t As[128 * LD];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[128 * LD];
  if ((int)blockIdx.y >= num_tiles[0]) return;
  const int g = tile_group[blockIdx.y];
  if (g >= G) return;
  const int m0 = tile_row0[blockIdx.y], m_end = group_off[g + 1];
  const bf16_t* Wg = W + (size_t)g * N * K;
  const int n0 = blockIdx.x * 128;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int l16 = lane & 15, lq = lane >> 4;
  v4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += 32) {
    __syncthreads();
    gg_stage_rows<AT, bf16_t>(As, A, lda, a_rows, m0, m_end, k0, K, vec_a);
    gg_stage_rows<AT, bf16_t>(As + 64 * LD, A, lda, a_rows, m0 + 64, m_end, k0, K, vec_a);
    gemm_stage<bf16_t, bf16_t>(Ws, Wg, (int64_t)K, n0, N, k0, K, vec_w);
    gemm_stage<bf16_t, bf16_t>(Ws + 64 * LD, Wg, (int64_t)K, n0 + 64, N, k0, K, vec_w);
    __syncthreads();
    sq_v8bf af[4], bf[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
      af[i] = *reinterpret_cast<const sq_v8bf*>(As + (wm + i * 16 + l16) * LD + lq * 8);
      bf[i] = *reinterpret_cast<const sq_v8bf*>(Ws + (wn + i * 16 + l16) * LD + lq * 8);
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int m = m0 + wm + i * 16 + lq * 4 + r, n = n0 + wn + j * 16 + l16;
        if (m < m_end && n < N) st_elem(Y, (size_t)m * ldy + n, gg_act(acc[i][j][r], act));
      }
}

// the same products for a handful of rows (decode steps): no tile, the weights stream once per row.  Workgroup = (8 output columns,
// one sorted row); a wavefront owns two columns and its lanes stride over K in 16-byte pieces.  glu: column f pairs rows f and
// F + f of the group's [2F][K] matrix and writes silu(first) * second.
template <typename AT, typename CT, typename YT>
__global__ void __launch_bounds__(256) grouped_gemv_kernel(int N, int K, const AT* __restrict__ A, int64_t lda,
                                                           const int32_t* __restrict__ a_rows, const CT* __restrict__ W, int w_rows,
                                                           YT* __restrict__ Y, int64_t ldy, const int32_t* __restrict__ row_group,
                                                           int act, bool vec, int G) {
  const int r = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (row_group[r] >= G) return;         // a group without weights
  const bool glu = act == KTX_GG_ACT_GLU_SILU;
  const AT* a = A + (size_t)(a_rows ? a_rows[r] : r) * lda;
  const CT* Wg = W + (size_t)row_group[r] * w_rows * K;
#pragma unroll
  for (int c2 = 0; c2 < 2; c2++) {
    const int n = blockIdx.x * 8 + wave * 2 + c2;
    if (n >= N) continue;
    const CT* w0 = Wg + (size_t)n * K;
    const CT* w1 = Wg + (size_t)(N + n) * K;
    float s0 = 0.f, s1 = 0.f;
    if (vec) {
      for (int k = lane * 8; k < K; k += 512) {
        float av[8], wv[8], uv[8];
#pragma unroll
        for (int i = 0; i < 8; i++) av[i] = ld_elem(a, k + i);
        if constexpr (sizeof(CT) == 2) {
          const uint4 p = *reinterpret_cast<const uint4*>(w0 + k);
          const uint32_t pw[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
          for (int i = 0; i < 4; i++) {
            wv[2 * i] = ktx_lo_f32(pw[i]);
            wv[2 * i + 1] = ktx_hi_f32(pw[i]);
          }
          if (glu) {
            const uint4 p1 = *reinterpret_cast<const uint4*>(w1 + k);
            const uint32_t pu[4] = {p1.x, p1.y, p1.z, p1.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
              uv[2 * i] = ktx_lo_f32(pu[i]);
              uv[2 * i + 1] = ktx_hi_f32(pu[i]);
            }
          }
        } else {
#pragma unroll
          for (int i = 0; i < 8; i++) {
            wv[i] = w0[k + i];
            if (glu) uv[i] = w1[k + i];
          }
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
          s0 = fmaf(av[i], wv[i], s0);
          if (glu) s1 = fmaf(av[i], uv[i], s1);
        }
      }
    } else {
      for (int k = lane; k < K; k += 64) {
        const float av = ld_elem(a, k);
        s0 = fmaf(av, ld_elem(w0, k), s0);
        if (glu) s1 = fmaf(av, ld_elem(w1, k), s1);
      }
    }
    s0 = wave_sum(s0);
    if (glu) s1 = wave_sum(s1);
    if (lane == 0) st_elem(Y, (size_t)r * ldy + n, glu ? silu_f32(s0) * s1 : gg_act(s0, act));
  }
}

int dtype_ok(int d) { return d == KTX_SEQ_F32 || d == KTX_SEQ_BF16; }

}  // namespace

extern "C" {

int ktx_rows_add(int T, int W, float* d_x, const float* d_x0, const float* d_vec, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && W > 0 && d_x, "ktx_rows_add: T >= 0, W > 0, x");
  if (T == 0 || (!d_x0 && !d_vec)) return 0;
  const size_t n = (size_t)T * W;
  rows_add_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(n, W, d_x, d_x0, d_vec);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_layer_norm(int T, int W, const float* d_x, const float* d_w, const float* d_b, float eps, const int32_t* d_rows, void* d_out,
                   int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && W > 0 && d_x && d_w && d_out && dtype_ok(out_dtype), "ktx_layer_norm: arguments");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KTX_SEQ_F32) layer_norm_kernel<float><<<T, 256, 0, st>>>(W, d_x, d_w, d_b, eps, d_rows, (float*)d_out);
  else layer_norm_kernel<bf16_t><<<T, 256, 0, st>>>(W, d_x, d_w, d_b, eps, d_rows, (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_gated_norm_add(int T, int W, const float* d_y, int64_t ldy, const float* d_ybias, const float* d_ey, const int32_t* d_pair_pos,
                       const float* d_topk_w, int top, const float* d_gl, int64_t ldg, const float* d_gbias, const float* d_wn,
                       const float* d_bn, float eps, float* d_x, const float* d_next_w, const float* d_next_b, float next_eps,
                       void* d_next_out, int next_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && W > 0 && d_wn && d_x && (d_y || d_ey), "ktx_gated_norm_add: arguments");
  KTX_REQUIRE(!d_ey || (d_pair_pos && d_topk_w && top > 0), "ktx_gated_norm_add: the gathered term needs pair_pos, topk_w and top");
  KTX_REQUIRE(!d_next_w || (d_next_out && dtype_ok(next_dtype)), "ktx_gated_norm_add: the following norm needs its output");
  KTX_REQUIRE((size_t)W * 4 <= 64 * 1024, "ktx_gated_norm_add: rows up to 16384 entries");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (d_next_w && next_dtype == KTX_SEQ_BF16)
    gated_norm_add_kernel<bf16_t><<<T, 256, (size_t)W * 4, st>>>(W, d_y, ldy, d_ybias, d_ey, d_pair_pos, d_topk_w, top, d_gl, ldg, d_gbias, d_wn,
                                                                 d_bn, eps, d_x, d_next_w, d_next_b, next_eps, (bf16_t*)d_next_out);
  else
    gated_norm_add_kernel<float><<<T, 256, (size_t)W * 4, st>>>(W, d_y, ldy, d_ybias, d_ey, d_pair_pos, d_topk_w, top, d_gl, ldg, d_gbias, d_wn,
                                                                d_bn, eps, d_x, d_next_w, d_next_b, next_eps, (float*)d_next_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_poly_norm(int T, int F, const float* d_z, int64_t ldz, const float* d_bias, const float* d_coef, float eps, void* d_out,
                  int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && F > 0 && d_z && d_coef && d_out && dtype_ok(out_dtype) && ldz >= F, "ktx_poly_norm: arguments");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KTX_SEQ_F32) poly_norm_kernel<float><<<T, 256, 0, st>>>(F, d_z, ldz, d_bias, d_coef, eps, (float*)d_out);
  else poly_norm_kernel<bf16_t><<<T, 256, 0, st>>>(F, d_z, ldz, d_bias, d_coef, eps, (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_postnorm_mix(int T, int W, const float* d_x_in, float* d_x_out, const ktx_postnorm_args* a, ktx_stream_t stream) {
  KTX_REQUIRE(a && T >= 0 && W > 0 && d_x_in && d_x_out && a->w && (a->out_lp == nullptr || a->out_dtype == KTX_SEQ_BF16 || a->out_dtype == KTX_SEQ_F32),
              "ktx_postnorm_mix: T >= 0, W > 0, x, a norm weight");
  KTX_REQUIRE(!a->y || a->ldy >= W, "ktx_postnorm_mix: ldy >= W");
  KTX_REQUIRE(!a->stack || (a->level >= 0 && a->stack_stride >= (int64_t)T * W), "ktx_postnorm_mix: level >= 0, stack_stride >= T * W");
  KTX_REQUIRE(!a->dwa || a->stack, "ktx_postnorm_mix: the average needs the stack");
  KTX_REQUIRE((size_t)W * 4 <= 150 * 1024, "ktx_postnorm_mix: a row must fit the LDS");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const bool lp16 = a->out_lp && a->out_dtype == KTX_SEQ_BF16;
  if (W <= 256 * 16) {
#define KTX_PN_GO(EPT)                                                                                                    \
  do {                                                                                                                    \
    if (lp16) postnorm_mix_reg_kernel<bf16_t, EPT><<<T, 256, 0, st>>>(W, d_x_in, d_x_out, *a, (bf16_t*)a->out_lp);        \
    else postnorm_mix_reg_kernel<float, EPT><<<T, 256, 0, st>>>(W, d_x_in, d_x_out, *a, (float*)a->out_lp);               \
  } while (0)
    if (W <= 256 * 4) KTX_PN_GO(4);
    else if (W <= 256 * 8) KTX_PN_GO(8);
    else KTX_PN_GO(16);
#undef KTX_PN_GO
    KTX_HIP(hipGetLastError());
    return 0;
  }
  if (a->out_lp && a->out_dtype == KTX_SEQ_BF16) {
    KTX_HIP(ktx_set_max_lds((const void*)postnorm_mix_kernel<bf16_t>, 150 * 1024));
    postnorm_mix_kernel<bf16_t><<<T, 256, (size_t)W * 4, st>>>(W, d_x_in, d_x_out, *a, (bf16_t*)a->out_lp);
  } else {
    KTX_HIP(ktx_set_max_lds((const void*)postnorm_mix_kernel<float>, 150 * 1024));
    postnorm_mix_kernel<float><<<T, 256, (size_t)W * 4, st>>>(W, d_x_in, d_x_out, *a, (float*)a->out_lp);
  }
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_glu_clamp_rows(int R, int F, const float* d_in, int64_t ldi, float limit, float slope, float up_shift, int paired, void* d_out,
                       int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(R >= 0 && F > 0 && d_in && d_out && dtype_ok(out_dtype) && ldi >= 2 * (int64_t)F && limit > 0.f, "ktx_glu_clamp_rows: arguments");
  if (R == 0) return 0;
  const size_t n = (size_t)R * F;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KTX_SEQ_F32)
    glu_clamp_rows_kernel<float><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(n, F, d_in, ldi, limit, slope, up_shift, paired, (float*)d_out);
  else
    glu_clamp_rows_kernel<bf16_t><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(n, F, d_in, ldi, limit, slope, up_shift, paired, (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_sigmoid_gate_rows(int R, int N, const void* d_o, int o_dtype, const float* d_gate, int64_t ldg, void* d_out, int out_dtype,
                          ktx_stream_t stream) {
  KTX_REQUIRE(R >= 0 && N > 0 && d_o && d_gate && d_out && dtype_ok(o_dtype) && dtype_ok(out_dtype) && ldg >= N, "ktx_sigmoid_gate_rows: arguments");
  if (R == 0) return 0;
  const size_t n = (size_t)R * N;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
#define KTX_SG_GO(IT, OT) sigmoid_gate_rows_kernel<IT, OT><<<blocks, 256, 0, st>>>(n, N, (const IT*)d_o, d_gate, ldg, (OT*)d_out)
  if (o_dtype == KTX_SEQ_F32) {
    if (out_dtype == KTX_SEQ_F32) KTX_SG_GO(float, float);
    else KTX_SG_GO(float, bf16_t);
  } else {
    if (out_dtype == KTX_SEQ_F32) KTX_SG_GO(bf16_t, float);
    else KTX_SG_GO(bf16_t, bf16_t);
  }
#undef KTX_SG_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_silu_mul_rows(int R, int F, const float* d_in, int64_t ldi, void* d_out, int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(R >= 0 && F > 0 && d_in && d_out && dtype_ok(out_dtype) && ldi >= 2 * (int64_t)F, "ktx_silu_mul_rows: arguments");
  if (R == 0) return 0;
  const size_t n = (size_t)R * F;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KTX_SEQ_F32) silu_mul_rows_kernel<float><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(n, F, d_in, ldi, (float*)d_out);
  else silu_mul_rows_kernel<bf16_t><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(n, F, d_in, ldi, (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_head_gate_norm(int T, int heads, int vdim, float eps, const float* d_o, const float* d_gate, int64_t ldg, const float* d_w,
                       int w_per_head, int act, void* d_out, int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && heads > 0 && vdim > 0 && d_o && d_gate && d_w && d_out && dtype_ok(out_dtype), "ktx_head_gate_norm: arguments");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KTX_SEQ_F32)
    head_gate_norm_kernel<float><<<T, 256, 0, st>>>(heads, vdim, eps, d_o, d_gate, ldg, d_w, w_per_head, act, (float*)d_out);
  else
    head_gate_norm_kernel<bf16_t><<<T, 256, 0, st>>>(heads, vdim, eps, d_o, d_gate, ldg, d_w, w_per_head, act, (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

static int delta_check(const ktx_delta_config* c, const char* who) {
  if (!c || c->heads <= 0 || c->kv_heads <= 0 || c->heads % c->kv_heads || c->dim <= 0 || c->vdim <= 0 || c->taps < 1)
    return ktx_fail(std::string(who) + ": heads % kv_heads == 0, dim, vdim > 0, taps >= 1");
  return 0;
}

int ktx_delta_prep(const ktx_delta_config* cfg, int B, int T, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                   const int32_t* d_tok_req, const float* d_proj, int64_t ldp, int q_off, int k_off, int v_off, int b_off, int a_off,
                   const float* d_taps, const float* d_A_log, const float* d_dt_bias, float* d_conv_state, float* d_qkv, float* d_gb,
                   ktx_stream_t stream) {
  if (delta_check(cfg, "ktx_delta_prep")) return -1;
  KTX_REQUIRE(B >= 0 && T >= 0 && d_q_indptr && d_pos0 && d_slot && d_tok_req && d_proj && d_taps && d_A_log && d_dt_bias && d_qkv && d_gb,
              "ktx_delta_prep: null pointer");
  KTX_REQUIRE(cfg->taps == 1 || d_conv_state, "ktx_delta_prep: a convolution over time needs its state");
  if (T == 0 || B == 0) return 0;
  const int C = 2 * cfg->kv_heads * cfg->dim + cfg->heads * cfg->vdim;
  const size_t lds = (size_t)C * 4;
  KTX_REQUIRE(lds <= 128 * 1024, "ktx_delta_prep: q | k | v of one token must fit 128 KB of LDS");
  hipStream_t st = (hipStream_t)stream;
  KTX_HIP(ktx_set_max_lds((const void*)delta_prep_kernel, 128 * 1024));
  delta_prep_kernel<<<T, 256, lds, st>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_tok_req, d_proj, ldp, q_off, k_off, v_off, b_off, a_off,
                                         d_taps, d_A_log, d_dt_bias, d_conv_state, d_qkv, d_gb);
  KTX_HIP(hipGetLastError());
  if (cfg->taps > 1) {
    delta_conv_update_kernel<<<dim3((C + 255) / 256, B), 256, 0, st>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_proj, ldp, q_off, k_off, v_off,
                                                                       d_conv_state);
    KTX_HIP(hipGetLastError());
  }
  return 0;
}

int ktx_delta_forward(const ktx_delta_config* cfg, int B, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                      const float* d_qkv, const float* d_gb, float* d_S, float* d_o, ktx_stream_t stream) {
  if (delta_check(cfg, "ktx_delta_forward")) return -1;
  KTX_REQUIRE(B >= 0 && d_q_indptr && d_pos0 && d_slot && d_qkv && d_gb && d_S && d_o, "ktx_delta_forward: null pointer");
  KTX_REQUIRE(cfg->dim <= 256, "ktx_delta_forward: dim <= 256");
  if (B == 0) return 0;
  const unsigned blocks = (unsigned)B * cfg->heads * ((cfg->vdim + 63) / 64);
  hipStream_t st = (hipStream_t)stream;
  // more wavefronts per workgroup as dim grows: a token's step costs a fixed latency plus a term per row a wavefront owns (at dim 128
  // sixteen wavefronts of 8 rows are no faster than eight of 16: the wider barrier and reduction eat the gain)
#define KTX_DL_GO(DPW, NW) delta_fwd_kernel<DPW, NW><<<blocks, NW * 64, 0, st>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_qkv, d_gb, d_S, d_o)
  const int D = cfg->dim;
  if (D <= 16) KTX_DL_GO(4, 4);
  else if (D <= 32) KTX_DL_GO(8, 4);
  else if (D <= 64) KTX_DL_GO(8, 8);
  else if (D <= 128) KTX_DL_GO(16, 8);
  else KTX_DL_GO(16, 16);
#undef KTX_DL_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

static int latattn_check(const ktx_latattn_config* c, const char* who) {
  if (!c || c->heads <= 0 || c->dim <= 0 || c->rot_dim < 0 || c->vdim <= 0 || c->kv_rank <= 0 || c->rot_dims < 0 || (c->rot_dims & 1) ||
      c->rot_dims > c->rot_dim || c->page_size <= 0 || !dtype_ok(c->cache_dtype))
    return ktx_fail(std::string(who) + ": sizes > 0, rot_dims even and <= rot_dim, a known cache type");
  return 0;
}

int ktx_latattn_prep(const ktx_latattn_config* cfg, int T, const float* d_proj, int64_t ldp, int q_off, int c_off, const float* d_wn,
                     const double* d_inv_freq, const int32_t* d_pos, const int32_t* d_cache_loc, void* d_cache, float* d_q_out,
                     ktx_stream_t stream) {
  if (latattn_check(cfg, "ktx_latattn_prep")) return -1;
  KTX_REQUIRE(T >= 0 && d_proj && (d_inv_freq || cfg->rot_dims == 0) && d_pos && d_q_out && (!d_cache || (d_wn && d_cache_loc)),
              "ktx_latattn_prep: null pointer");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)std::max(cfg->rot_dims, 2) * 4;
  if (cfg->cache_dtype == KTX_SEQ_F32)
    latattn_prep_kernel<float><<<T, 256, lds, st>>>(*cfg, d_proj, ldp, q_off, c_off, d_wn, d_inv_freq, d_pos, d_cache_loc, (float*)d_cache, d_q_out);
  else
    latattn_prep_kernel<bf16_t><<<T, 256, lds, st>>>(*cfg, d_proj, ldp, q_off, c_off, d_wn, d_inv_freq, d_pos, d_cache_loc, (bf16_t*)d_cache, d_q_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_latattn_forward(const ktx_latattn_config* cfg, int T, const float* d_q, const void* d_cache, const int32_t* d_tok_req,
                        const int32_t* d_pos, const int32_t* d_page_indptr, const int32_t* d_page_indices, const float* d_sink,
                        int nsplit, float* d_scratch, void* d_out, int out_dtype, ktx_stream_t stream) {
  if (latattn_check(cfg, "ktx_latattn_forward")) return -1;
  KTX_REQUIRE(T >= 0 && d_q && d_cache && d_tok_req && d_pos && d_page_indptr && d_page_indices && d_out && dtype_ok(out_dtype),
              "ktx_latattn_forward: null pointer");
  KTX_REQUIRE(nsplit >= 1 && nsplit <= 4096 && (nsplit == 1 || d_scratch), "ktx_latattn_forward: 1 <= nsplit <= 4096, scratch when > 1");
  if (T == 0) return 0;
  const int L = cfg->kv_rank, E = L + cfg->rot_dim;
  KTX_REQUIRE(L <= 256 * LA_NACC, "ktx_latattn_forward: kv_rank <= 8192");
  // heads per workgroup: outputs fit the registers, queries + one key tile fit the LDS
  const size_t budget = 96 * 1024;
  int HG = std::min(cfg->heads, std::max(1, 256 * LA_NACC / L));
  int KTN = 64;
  auto lds_of = [&](int hg, int ktn) { return ((size_t)hg * E + (size_t)ktn * (E + 1) + (size_t)hg * ktn + 3 * (size_t)hg + ktn) * 4; };
  while (KTN > 8 && lds_of(1, KTN) > budget) KTN /= 2;
  while (HG > 1 && lds_of(HG, KTN) > budget) HG = (HG + 1) / 2;
  KTX_REQUIRE(lds_of(HG, KTN) <= 150 * 1024, "ktx_latattn_forward: one head's query and 8 keys do not fit the LDS");
  const size_t lds = lds_of(HG, KTN);
  const dim3 grid(T, (cfg->heads + HG - 1) / HG, nsplit);
  hipStream_t st = (hipStream_t)stream;
#define KTX_LA_GO(KT, OT)                                                                                                     \
  do {                                                                                                                        \
    KTX_HIP(ktx_set_max_lds((const void*)latattn_fwd_kernel<KT, OT>, 150 * 1024));                                            \
    latattn_fwd_kernel<KT, OT><<<grid, 256, lds, st>>>(*cfg, T, HG, KTN, d_q, (const KT*)d_cache, d_tok_req, d_pos, d_page_indptr, \
                                                       d_page_indices, d_sink, nsplit, d_scratch, (OT*)d_out);               \
  } while (0)
  if (cfg->cache_dtype == KTX_SEQ_F32) {
    if (out_dtype == KTX_SEQ_F32) KTX_LA_GO(float, float);
    else KTX_LA_GO(float, bf16_t);
  } else {
    if (out_dtype == KTX_SEQ_F32) KTX_LA_GO(bf16_t, float);
    else KTX_LA_GO(bf16_t, bf16_t);
  }
#undef KTX_LA_GO
  KTX_HIP(hipGetLastError());
  if (nsplit > 1) {
    const dim3 mg(T, cfg->heads);
    if (out_dtype == KTX_SEQ_F32) latattn_merge_kernel<float><<<mg, 256, (size_t)nsplit * 8, st>>>(T, cfg->heads, L, nsplit, d_scratch, d_sink, (float*)d_out);
    else latattn_merge_kernel<bf16_t><<<mg, 256, (size_t)nsplit * 8, st>>>(T, cfg->heads, L, nsplit, d_scratch, d_sink, (bf16_t*)d_out);
    KTX_HIP(hipGetLastError());
  }
  return 0;
}

int ktx_latattn_mfma_eligible(const ktx_latattn_config* c) {
  if (!c || c->cache_dtype != KTX_SEQ_BF16) return 0;
  const int L = c->kv_rank, E = L + c->rot_dim;
  if (!(L == 64 || L == 128 || L == 256 || L == 512) || E % 8 != 0) return 0;
  if (((E + 31) / 32) > (L / 16) / 2 + 4) return 0;
  return latattn_mfma_lds(*c) <= 150 * 1024;
}

int ktx_latattn_mfma(const ktx_latattn_config* cfg, int B, int T, int max_q_len, const float* d_q, const void* d_cache,
                     const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_page_indptr, const int32_t* d_page_indices,
                     const float* d_sink, int nsplit, float* d_scratch, void* d_out, int out_dtype, ktx_stream_t stream) {
  if (latattn_check(cfg, "ktx_latattn_mfma")) return -1;
  KTX_REQUIRE(ktx_latattn_mfma_eligible(cfg), "ktx_latattn_mfma: bf16 cache, kv_rank 64 / 128 / 256 / 512, rot_dim a multiple of 8 up to 128");
  KTX_REQUIRE(B >= 0 && T >= 0 && max_q_len >= 0 && d_q && d_cache && d_q_indptr && d_pos0 && d_page_indptr && d_page_indices &&
                  d_out && dtype_ok(out_dtype),
              "ktx_latattn_mfma: null pointer");
  KTX_REQUIRE(nsplit >= 1 && nsplit <= 4096 && (nsplit == 1 || d_scratch), "ktx_latattn_mfma: 1 <= nsplit <= 4096, scratch when > 1");
  if (B == 0 || T == 0 || max_q_len == 0) return 0;
  const int row_tiles = (int)(((int64_t)max_q_len * cfg->heads + 63) / 64);
  const dim3 grid((unsigned)B * row_tiles, 1, nsplit);
  const size_t lds = latattn_mfma_lds(*cfg);
  hipStream_t st = (hipStream_t)stream;
  const int L = cfg->kv_rank;
#define KTX_LM_GO(NT, OT)                                                                                                       \
  do {                                                                                                                          \
    KTX_HIP(ktx_set_max_lds((const void*)latattn_mfma_kernel<NT, OT>, 150 * 1024));                                             \
    latattn_mfma_kernel<NT, OT><<<grid, 256, lds, st>>>(*cfg, T, row_tiles, d_q, (const bf16_t*)d_cache, d_q_indptr, d_pos0,    \
                                                        d_page_indptr, d_page_indices, d_sink, nsplit, d_scratch, (OT*)d_out);  \
  } while (0)
#define KTX_LM_NT(OT)             \
  do {                            \
    if (L == 64) KTX_LM_GO(4, OT);  \
    else if (L == 128) KTX_LM_GO(8, OT); \
    else if (L == 256) KTX_LM_GO(16, OT); \
    else KTX_LM_GO(32, OT);       \
  } while (0)
  if (out_dtype == KTX_SEQ_F32) KTX_LM_NT(float);
  else KTX_LM_NT(bf16_t);
#undef KTX_LM_NT
#undef KTX_LM_GO
  KTX_HIP(hipGetLastError());
  if (nsplit > 1) {
    const dim3 mg(T, cfg->heads);
    if (out_dtype == KTX_SEQ_F32) latattn_merge_kernel<float><<<mg, 256, (size_t)nsplit * 8, st>>>(T, cfg->heads, L, nsplit, d_scratch, d_sink, (float*)d_out);
    else latattn_merge_kernel<bf16_t><<<mg, 256, (size_t)nsplit * 8, st>>>(T, cfg->heads, L, nsplit, d_scratch, d_sink, (bf16_t*)d_out);
    KTX_HIP(hipGetLastError());
  }
  return 0;
}

int ktx_moe_route(int T, int E, int top, float scale, float sum_eps, const float* d_logits, int64_t ldl, int32_t* d_topk_idx,
                  float* d_topk_w, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && E <= 64 * MOE_RE && d_logits && d_topk_idx && d_topk_w && ldl >= E,
              "ktx_moe_route: 0 < top <= experts <= 1024");
  if (T == 0) return 0;
  moe_route_kernel<<<(T + 3) / 4, 256, 0, (hipStream_t)stream>>>(T, E, top, scale, sum_eps, d_logits, ldl, d_topk_idx, d_topk_w);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_moe_plan(int T, int E, int top, int tile_m, const int32_t* d_topk_idx, int32_t* d_group_off, int32_t* d_sorted_tok,
                 int32_t* d_pair_pos, int32_t* d_sorted_group, int32_t* d_tile_group, int32_t* d_tile_row0, int32_t* d_num_tiles,
                 ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && E > 0 && E <= 4096 && top > 0 && tile_m > 0 && d_topk_idx && d_group_off && d_sorted_tok && d_pair_pos &&
                  d_sorted_group && d_tile_group && d_tile_row0 && d_num_tiles,
              "ktx_moe_plan: arguments");
  moe_plan_kernel<<<1, 1024, (size_t)(3 * E + 1) * 4, (hipStream_t)stream>>>(T * top, E, top, tile_m, d_topk_idx, d_group_off, d_sorted_tok,
                                                                              d_pair_pos, d_sorted_group, d_tile_group, d_tile_row0,
                                                                              d_num_tiles);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_grouped_gemm(int G, int M, int N, int K, const void* d_A, int a_dtype, int64_t lda, int64_t a_goff, const int32_t* d_a_rows,
                     const void* d_W, int w_dtype, void* d_Y, int y_dtype, int64_t ldy, int64_t y_goff, const int32_t* d_group_off,
                     const int32_t* d_tile_group, const int32_t* d_tile_row0, const int32_t* d_num_tiles, int max_tiles, int tile_m,
                     int act, ktx_stream_t stream) {
  KTX_REQUIRE(G > 0 && M >= 0 && N > 0 && K > 0 && d_A && d_W && d_Y, "ktx_grouped_gemm: G, N, K > 0, pointers");
  KTX_REQUIRE(act == KTX_GG_ACT_NONE || act == KTX_GG_ACT_RELU_SQ, "ktx_grouped_gemm: epilogue none or relu^2");
  KTX_REQUIRE(dtype_ok(a_dtype) && dtype_ok(w_dtype) && dtype_ok(y_dtype), "ktx_grouped_gemm: unknown element type");
  KTX_REQUIRE(!(w_dtype == KTX_SEQ_F32 && (a_dtype != KTX_SEQ_F32 || y_dtype != KTX_SEQ_F32)),
              "ktx_grouped_gemm: an fp32 product takes and writes fp32");
  const bool ragged = d_group_off != nullptr;
  KTX_REQUIRE(!ragged || (d_tile_group && d_tile_row0 && d_num_tiles && max_tiles >= 0), "ktx_grouped_gemm: the ragged form needs its tiles");
  KTX_REQUIRE(ragged || (G <= 65535 && !d_a_rows), "ktx_grouped_gemm: the uniform form takes up to 65535 groups and no gather");
  const int ytiles = ragged ? max_tiles : (M + 63) / 64;
  if (ytiles == 0) return 0;
  if (ragged && tile_m == 128) {
    KTX_REQUIRE(w_dtype == KTX_SEQ_BF16, "ktx_grouped_gemm: 128-row tiles are the bf16 product's");
    KTX_REQUIRE(ytiles <= 65535, "ktx_grouped_gemm: too many row tiles");
    const dim3 grid128((N + 127) / 128, ytiles, 1);
    const size_t asz1 = a_dtype == KTX_SEQ_F32 ? 4 : 2;
    const bool va = aligned16(d_A) && (lda * asz1) % 16 == 0 && K % 8 == 0;
    const bool vw = aligned16(d_W) && ((size_t)K * 2) % 16 == 0 && K % 8 == 0 && ((size_t)N * K * 2) % 16 == 0;
    hipStream_t st1 = (hipStream_t)stream;
#define KTX_GG128_GO(AT, YT)                                                                                                       \
  grouped_gemm128_kernel<AT, YT><<<grid128, 256, 0, st1>>>(N, K, (const AT*)d_A, lda, d_a_rows, (const bf16_t*)d_W, (YT*)d_Y, ldy, \
                                                           d_group_off, d_tile_group, d_tile_row0, d_num_tiles, va, vw, G, act)
    if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32) KTX_GG128_GO(float, float);
    else if (a_dtype == KTX_SEQ_F32) KTX_GG128_GO(float, bf16_t);
    else if (y_dtype == KTX_SEQ_F32) KTX_GG128_GO(bf16_t, float);
    else KTX_GG128_GO(bf16_t, bf16_t);
#undef KTX_GG128_GO
    KTX_HIP(hipGetLastError());
    return 0;
  }
  KTX_REQUIRE(!ragged || tile_m == 64, "ktx_grouped_gemm: tiles of 64 or 128 rows");
  KTX_REQUIRE(ytiles <= 65535, "ktx_grouped_gemm: too many row tiles");
  const dim3 grid((N + 63) / 64, ytiles, ragged ? 1 : G);
  const size_t asz = a_dtype == KTX_SEQ_F32 ? 4 : 2, wsz = w_dtype == KTX_SEQ_F32 ? 4 : 2;
  const bool vec_a = aligned16(d_A) && (lda * asz) % 16 == 0 && ((size_t)a_goff * asz) % 16 == 0 && K % 8 == 0;
  const bool vec_w = aligned16(d_W) && ((size_t)K * wsz) % 16 == 0 && K % 8 == 0 && ((size_t)N * K * wsz) % 16 == 0;
  hipStream_t st = (hipStream_t)stream;
#define KTX_GG_GO(AT, CT, YT)                                                                                                  \
  grouped_gemm_kernel<AT, CT, YT><<<grid, 256, 0, st>>>(M, N, K, (const AT*)d_A, lda, a_goff, d_a_rows, (const CT*)d_W, (YT*)d_Y, ldy, \
                                                        y_goff, d_group_off, d_tile_group, d_tile_row0, d_num_tiles, vec_a, vec_w, G, act)
  if (w_dtype == KTX_SEQ_BF16) {
    if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32) KTX_GG_GO(float, bf16_t, float);
    else if (a_dtype == KTX_SEQ_F32) KTX_GG_GO(float, bf16_t, bf16_t);
    else if (y_dtype == KTX_SEQ_F32) KTX_GG_GO(bf16_t, bf16_t, float);
    else KTX_GG_GO(bf16_t, bf16_t, bf16_t);
  } else {
    KTX_GG_GO(float, float, float);
  }
#undef KTX_GG_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_grouped_gemv(int R, int N, int K, const void* d_A, int a_dtype, int64_t lda, const int32_t* d_a_rows, const void* d_W, int w_dtype,
                     void* d_Y, int y_dtype, int64_t ldy, const int32_t* d_row_group, int act, int G, ktx_stream_t stream) {
  KTX_REQUIRE(R >= 0 && N > 0 && K > 0 && G > 0 && d_A && d_W && d_Y && d_row_group, "ktx_grouped_gemv: N, K, G > 0, pointers");
  KTX_REQUIRE(act == KTX_GG_ACT_NONE || act == KTX_GG_ACT_GLU_SILU || act == KTX_GG_ACT_RELU_SQ, "ktx_grouped_gemv: unknown epilogue");
  const int glu = act == KTX_GG_ACT_GLU_SILU;
  KTX_REQUIRE(dtype_ok(a_dtype) && dtype_ok(w_dtype) && dtype_ok(y_dtype), "ktx_grouped_gemv: unknown element type");
  KTX_REQUIRE(R <= 65535, "ktx_grouped_gemv: up to 65535 rows");
  if (R == 0) return 0;
  const size_t asz = a_dtype == KTX_SEQ_F32 ? 4 : 2, wsz = w_dtype == KTX_SEQ_F32 ? 4 : 2;
  const bool vec = aligned16(d_W) && ((size_t)K * wsz) % 16 == 0 && K % 8 == 0 && aligned16(d_A) && (lda * asz) % 16 == 0;
  const dim3 grid((N + 7) / 8, R);
  const int w_rows = glu ? 2 * N : N;
  hipStream_t st = (hipStream_t)stream;
#define KTX_GV_GO(AT, CT, YT)                                                                                                          \
  grouped_gemv_kernel<AT, CT, YT><<<grid, 256, 0, st>>>(N, K, (const AT*)d_A, lda, d_a_rows, (const CT*)d_W, w_rows, (YT*)d_Y, ldy, \
                                                        d_row_group, act, vec, G)
  if (w_dtype == KTX_SEQ_BF16) {
    if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32) KTX_GV_GO(float, bf16_t, float);
    else if (a_dtype == KTX_SEQ_F32) KTX_GV_GO(float, bf16_t, bf16_t);
    else if (y_dtype == KTX_SEQ_F32) KTX_GV_GO(bf16_t, bf16_t, float);
    else KTX_GV_GO(bf16_t, bf16_t, bf16_t);
  } else {
    KTX_REQUIRE(a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32, "ktx_grouped_gemv: an fp32 product takes and writes fp32");
    KTX_GV_GO(float, float, float);
  }
#undef KTX_GV_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
