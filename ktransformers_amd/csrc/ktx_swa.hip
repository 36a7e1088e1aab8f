// ktx_swa.hip — kernels behind include/ktx_swa.h: the residual update with a scalar-weight RMS norm and the rows an input convolution
// reads, the input convolution over time, grouped-query sliding-window attention over paged key and value caches with rotated values
// and a sink (prep — rotating, or convolving the projections over time and norming them whole —, a vector-ALU form for any sizes, a
// matrix-core form for bf16 caches, both with an optional bias by distance and kept first positions, the key-range merge), the selective scan with
// its short convolution, and the softmax router with a choice correction.
//
// Everything a norm, an angle, a score, a router or a recurrence touches is fp32; element types only select how weights, activations
// and the caches are stored and which MFMA multiplies them.
#include "ktx_common.h"
#include "../../include/ktx_swa.h"

#include <math.h>

#include <algorithm>

namespace {

#include "ktx_seq_dev.inc"

__device__ __forceinline__ float silu_f32(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f32(float z) { return z > 20.f ? z : log1pf(expf(z)); }

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }
int dtype_ok(int d) { return d == KTX_SEQ_F32 || d == KTX_SEQ_BF16; }

// ---------------------------------------------------------------------------------------------------------------------
// one row per workgroup; the row lives in LDS between the passes
constexpr int RN_MAX_HALO = 8, RN_TOP = 8;
template <typename OT, typename HT>
__global__ void __launch_bounds__(256) resid_norm_kernel(int W, float* __restrict__ x, ktx_resid_args a) {
  extern __shared__ float row[];
  __shared__ float red[4];
  const int i = blockIdx.x, tid = threadIdx.x;
  const int t = a.rows ? a.rows[i] : i;
  float* xr = x + (size_t)t * W;
  const bool adds = a.y || a.ey;
  if (adds) {
    for (int e = tid; e < W; e += 256) row[e] = 0.f;
    if (a.y) {
      const float* y = a.y + (size_t)t * a.ldy;
      float r = 1.0f;
      if (a.y_norm_w) {
        float s = 0.f;
        for (int e = tid; e < W; e += 256) s += y[e] * y[e];
        r = 1.0f / sqrtf(block_sum256(s, red) / (float)W + a.y_norm_eps);
      }
      for (int e = tid; e < W; e += 256) row[e] = a.y_norm_w ? y[e] * r * a.y_norm_w[e] : y[e];
    }
    if (a.ey) {
      // a step of one token is one workgroup: the choices' indices, weights and row numbers are fetched side by side, then the rows
      // (a chain of dependent loads per choice would cost a memory round trip each)
      const HT* h = reinterpret_cast<const HT*>(a.h_in) + (size_t)t * W;
      for (int k0 = 0; k0 < a.top; k0 += RN_TOP) {
        int g[RN_TOP];
        float w[RN_TOP];
        const float* src[RN_TOP];
#pragma unroll
        for (int j = 0; j < RN_TOP; j++) {
          const bool ok = k0 + j < a.top;
          const size_t at = (size_t)t * a.top + (ok ? k0 + j : 0);
          g[j] = ok ? a.topk_idx[at] : a.n_real;
          w[j] = ok ? a.topk_w[at] : 0.f;
          src[j] = a.ey + (size_t)a.pair_pos[at] * W;
        }
        for (int e = tid; e < W; e += 256) {
          const float hv = ld_elem(h, e);
          float v[RN_TOP];
#pragma unroll
          for (int j = 0; j < RN_TOP; j++) v[j] = g[j] < a.n_real ? src[j][e] : hv;
          float acc = row[e];
#pragma unroll
          for (int j = 0; j < RN_TOP; j++) acc += w[j] * v[j];
          row[e] = acc;
        }
      }
    }
    for (int e = tid; e < W; e += 256) {
      const float v = xr[e] + row[e];
      row[e] = v;
      xr[e] = v;
    }
  } else {
    for (int e = tid; e < W; e += 256) row[e] = xr[e];
  }
  if (!a.norm_g) return;
  float s = 0.f;
  for (int e = tid; e < W; e += 256) s += row[e] * row[e];
  const float r = a.norm_g[0] / sqrtf(block_sum256(s, red) / (float)W + a.eps);
  OT* out = reinterpret_cast<OT*>(a.out);
  if (a.conv_w) {                // one new token per request: the convolution and the state's move happen here
    const int taps = a.conv_taps, halo = taps - 1;             // (one tap: no neighbours, no state)
    const int b = halo > 0 ? a.tok_req[t] : 0;
    const bool cont = halo > 0 && a.pos0[b] > 0;
    float* st = halo > 0 ? a.conv_state + (size_t)a.slot[b] * halo * W : nullptr;
    // four channels per thread at a time, every load of the batch in front of its first store: the state is read and written through
    // the same pointer, and a store in front of the next channel's loads would make each channel wait for a memory round trip
    constexpr int RN_CB = 4;
    const float* __restrict__ cw = a.conv_w;
    for (int e0 = tid; e0 < W; e0 += 256 * RN_CB) {
      float prev[RN_CB][RN_MAX_HALO], wv[RN_CB][RN_MAX_HALO + 1];
#pragma unroll
      for (int u = 0; u < RN_CB; u++) {
        const int e = e0 + u * 256;
#pragma unroll
        for (int j = 0; j < RN_MAX_HALO; j++) {
          const bool ok = e < W && j < halo;
          prev[u][j] = ok && cont ? st[(size_t)j * W + e] : 0.f;
          wv[u][j] = ok ? cw[(size_t)e * taps + j] : 0.f;
        }
        wv[u][RN_MAX_HALO] = e < W ? cw[(size_t)e * taps + halo] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < RN_CB; u++) {
        const int e = e0 + u * 256;
        if (e < W) {
          const float hn = row[e] * r;
          float acc = 0.f;
#pragma unroll
          for (int j = 0; j < RN_MAX_HALO; j++)
            if (j < halo) acc += wv[u][j] * prev[u][j];
          acc += wv[u][RN_MAX_HALO] * hn;
          st_elem(out, (size_t)t * W + e, hn + acc);
#pragma unroll
          for (int j = 0; j < RN_MAX_HALO; j++)
            if (j < halo) st[(size_t)j * W + e] = j + 1 < halo ? prev[u][(j + 1) % RN_MAX_HALO] : hn;
        }
      }
    }
    return;
  }
  if (a.halo <= 0) {
    for (int e = tid; e < W; e += 256) st_elem(out, (size_t)i * W + e, row[e] * r);
    return;
  }
  const int b = a.tok_req[t];
  for (int e = tid; e < W; e += 256) st_elem(out, ((size_t)t + (size_t)(b + 1) * a.halo) * W + e, row[e] * r);
  if (t == a.q_indptr[b]) {      // the request's first new token also lays the rows in front of it
    const bool cont = a.pos0[b] > 0;
    const float* st = a.conv_state + (size_t)a.slot[b] * a.halo * W;
    for (int e = tid; e < a.halo * W; e += 256) st_elem(out, ((size_t)t + (size_t)b * a.halo) * W + e, cont ? st[e] : 0.f);
  }
}

// thread = (token, channel)
template <typename OT>
__global__ void __launch_bounds__(256) input_conv_kernel(int W, int taps, const float* __restrict__ hx, const float* __restrict__ w,
                                                         const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ slot,
                                                         const int32_t* __restrict__ tok_req, float* __restrict__ conv_state,
                                                         OT* __restrict__ out) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int halo = taps - 1, b = tok_req[t];
  const size_t r = (size_t)t + (size_t)(b + 1) * halo;
  float acc = 0.f;
  for (int j = 0; j < taps; j++) acc += w[(size_t)c * taps + j] * hx[(r - halo + j) * W + c];
  st_elem(out, (size_t)t * W + c, hx[r * W + c] + acc);
  if (t == q_indptr[b + 1] - 1) {
    float* st = conv_state + (size_t)slot[b] * halo * W;
    for (int i = 0; i < halo; i++) st[(size_t)i * W + c] = hx[(r - halo + 1 + i) * W + c];
  }
}

template <typename TT, typename OT>
__global__ void __launch_bounds__(256) rows_mul_lookup_kernel(size_t total, int n, const float* __restrict__ a, int64_t lda,
                                                              const TT* __restrict__ table, int64_t ldt, int col0,
                                                              const int32_t* __restrict__ tokens, OT* __restrict__ out) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const size_t t = i / n;
  const int c = (int)(i % n);
  st_elem(out, i, a[t * lda + c] * ld_elem(table, (size_t)tokens[t] * ldt + col0 + c));
}

// ---------------------------------------------------------------------------------------------------------------------
// attention prep: one token per workgroup, a wavefront per head
template <typename KT>
__global__ void __launch_bounds__(256) swa_prep_kernel(ktx_swa_config c, const float* __restrict__ proj, int64_t ldp, int q_off, int k_off,
                                                       int v_off, const double* __restrict__ inv_freq, const double* __restrict__ v_inv_freq,
                                                       const int32_t* __restrict__ pos, const int32_t* __restrict__ cache_loc,
                                                       KT* __restrict__ kcache, KT* __restrict__ vcache, float* __restrict__ q_out,
                                                       float* __restrict__ vcs) {
  extern __shared__ float cs[];            // cos | sin of the rot_dims / 2 key angles, cos | sin of the vdim / 2 value angles, the token's q | k | v
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int NP = c.rot_dims / 2, NV = c.rot_values ? c.vdim / 2 : 0;
  const int D = c.dim, V = c.vdim, H = c.heads, G = c.kv_heads;
  float* vc = cs + 2 * NP;
  float* row = vc + 2 * NV;                // [H * D | G * D | G * V]: read once, coalesced; the heads' passes below stay in LDS
  const float* base = proj + (size_t)t * ldp;
  const int nq = H * D, nk = G * D, nv = G * V;
  for (int i = tid; i < nq + nk + nv; i += 256)
    row[i] = base[i < nq ? q_off + i : i < nq + nk ? k_off + (i - nq) : v_off + (i - nq - nk)];
  const double p = (double)pos[t];
  for (int i = tid; i < NP; i += 256) {
    double si, co;
    sincos(p * inv_freq[i], &si, &co);
    cs[i] = (float)co;
    cs[NP + i] = (float)si;
  }
  for (int i = tid; i < NV; i += 256) {
    double sd, cd;
    sincos(p * v_inv_freq[i], &sd, &cd);
    const float co = (float)cd, si = (float)sd;
    vc[i] = co;
    vc[NV + i] = si;
    vcs[(size_t)t * c.vdim + i] = co;
    vcs[(size_t)t * c.vdim + NV + i] = si;
  }
  __syncthreads();
  // entry j of a vector whose first 2 * np entries turn in pairs (2i, 2i + 1)
  auto turned = [](const float* v, int j, int np, const float* tab) -> float {
    if (j >= 2 * np) return v[j];
    const int i = j >> 1;
    const float a = v[2 * i], bb = v[2 * i + 1];
    return (j & 1) ? bb * tab[i] + a * tab[np + i] : a * tab[i] - bb * tab[np + i];
  };
  const size_t loc = (size_t)cache_loc[t];
  for (int u = wave; u < H + 2 * G; u += 4) {
    if (u < H + G) {        // a query or key head: rotate, then norm
      const bool isq = u < H;
      const float* v = row + (size_t)u * D;      // (key heads follow the query heads in the row)
      float r = 1.0f;
      if (c.qk_norm) {
        float s = 0.f;
        for (int j = lane; j < D; j += 64) {
          const float x = turned(v, j, NP, cs);
          s += x * x;
        }
        r = 1.0f / sqrtf(wave_sum(s) / (float)D + c.eps);
      }
      if (isq) {
        r *= c.scale;
        float* o = q_out + ((size_t)t * H + u) * D;
        for (int j = lane; j < D; j += 64) o[j] = turned(v, j, NP, cs) * r;
      } else {
        KT* o = kcache + (loc * G + (u - H)) * D;
        for (int j = lane; j < D; j += 64) st_elem(o, j, turned(v, j, NP, cs) * r);
      }
    } else {
      const int g = u - H - G;
      const float* v = row + nq + nk + (size_t)g * V;
      KT* o = vcache + (loc * G + g) * V;
      for (int j = lane; j < V; j += 64) st_elem(o, j, turned(v, j, NV, vc));
    }
  }
}

// The prep of an attention whose projections pass a short causal convolution over time and whose q and k are RMS-normed over the WHOLE
// projection (all heads at once) with a weight: one workgroup per token, the convolved q | k | v row in LDS between the passes.
// Input u[c] at relative token ii of the request: this step's projection (+ bias) for ii >= 0, the slot's state row taps - 1 + ii for
// ii < 0 when the request has a past, zero otherwise.
constexpr int CP_MAX_TAPS = 16;
template <typename KT>
__global__ void __launch_bounds__(256) swa_conv_prep_kernel(ktx_swa_config c, int taps, const float* __restrict__ proj, int64_t ldp,
                                                            const float* __restrict__ bias, const float* __restrict__ cw,
                                                            const float* __restrict__ qw, const float* __restrict__ kw,
                                                            const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ pos0,
                                                            const int32_t* __restrict__ slot, const int32_t* __restrict__ tok_req,
                                                            const float* __restrict__ conv_state, const int32_t* __restrict__ cache_loc,
                                                            KT* __restrict__ kcache, KT* __restrict__ vcache, float* __restrict__ q_out) {
  extern __shared__ float row[];           // [H * D | G * D | G * V]
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int nq = c.heads * c.dim, nk = c.kv_heads * c.dim, nv = c.kv_heads * c.vdim, C = nq + nk + nv;
  const int b = tok_req[t], i = t - q_indptr[b];
  const bool carried = pos0[b] > 0;
  const float* st = conv_state ? conv_state + (size_t)slot[b] * (taps - 1) * C : nullptr;
  float sq = 0.f, sk = 0.f;
  for (int e = tid; e < C; e += 256) {
    const float be = bias ? bias[e] : 0.f;
    float y;
    if (taps <= 1) {
      y = (proj[(size_t)t * ldp + e] + be) * (cw ? cw[e] : 1.0f);
    } else {
      float u[CP_MAX_TAPS];
#pragma unroll
      for (int j = 0; j < CP_MAX_TAPS; j++) {
        u[j] = 0.f;
        if (j < taps) {
          const int ii = i - (taps - 1) + j;
          if (ii >= 0) u[j] = proj[(size_t)(t - (taps - 1) + j) * ldp + e] + be;
          else if (carried) u[j] = st[(size_t)(taps - 1 + ii) * C + e];
        }
      }
      y = 0.f;
#pragma unroll
      for (int j = 0; j < CP_MAX_TAPS; j++)
        if (j < taps) y += cw[(size_t)e * taps + j] * u[j];
    }
    row[e] = y;
    if (e < nq) sq += y * y;
    else if (e < nq + nk) sk += y * y;
  }
  const float rq = qw ? 1.0f / sqrtf(block_sum256(sq, red) / (float)nq + c.eps) : 1.0f;
  const float rk = kw ? 1.0f / sqrtf(block_sum256(sk, red) / (float)nk + c.eps) : 1.0f;
  const size_t loc = (size_t)cache_loc[t];
  for (int e = tid; e < C; e += 256) {      // (each thread re-reads only what it wrote)
    const float y = row[e];
    if (e < nq) q_out[(size_t)t * nq + e] = y * rq * (qw ? qw[e] : 1.0f) * c.scale;
    else if (e < nq + nk) st_elem(kcache, loc * nk + (e - nq), y * rk * (kw ? kw[e - nq] : 1.0f));
    else st_elem(vcache, loc * nv + (e - nq - nk), y);
  }
}

// The same prep for 2 .. 4 taps and channel counts that are multiples of 4 (q, k and v each): a thread owns FOUR neighbouring channels
// (16-byte loads of the projections, the state rows and the taps), requests everything a group needs before it uses any of it, and —
// in steps where every request brings exactly one token (`one_token`) — moves the slot's state on itself: the token's workgroup is the
// only reader of its slot, and a thread reads and writes only its own channels.
template <typename KT, int TAPS>
__global__ void __launch_bounds__(256) swa_conv_prep_vec_kernel(ktx_swa_config c, const float* __restrict__ proj, int64_t ldp,
                                                                const float* __restrict__ bias, const float* __restrict__ cw,
                                                                const float* __restrict__ qw, const float* __restrict__ kw,
                                                                const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ pos0,
                                                                const int32_t* __restrict__ slot, const int32_t* __restrict__ tok_req,
                                                                float* __restrict__ conv_state, int one_token,
                                                                const int32_t* __restrict__ cache_loc, KT* __restrict__ kcache,
                                                                KT* __restrict__ vcache, float* __restrict__ q_out) {
  extern __shared__ __attribute__((aligned(16))) float row[];      // [H * D | G * D | G * V]
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int nq = c.heads * c.dim, nk = c.kv_heads * c.dim, nv = c.kv_heads * c.vdim, C = nq + nk + nv;
  const int b = tok_req[t], i = t - q_indptr[b];
  const bool carried = pos0[b] > 0;
  float* st = conv_state + (size_t)slot[b] * (TAPS - 1) * C;
  const float4 zero4 = make_float4(0.f, 0.f, 0.f, 0.f);
  float sq = 0.f, sk = 0.f;
  for (int e = tid * 4; e < C; e += 1024) {
    float4 u[TAPS], w[4];
    const float4 be = bias ? *reinterpret_cast<const float4*>(bias + e) : zero4;
#pragma unroll
    for (int j = 0; j < TAPS; j++) {
      const int ii = i - (TAPS - 1) + j;
      if (ii >= 0) u[j] = *reinterpret_cast<const float4*>(proj + (size_t)(t - (TAPS - 1) + j) * ldp + e);
      else if (carried) u[j] = *reinterpret_cast<const float4*>(st + (size_t)(TAPS - 1 + ii) * C + e);
      else u[j] = zero4;
    }
#pragma unroll
    for (int n = 0; n < 4; n++) {      // the taps of channel e + n: TAPS consecutive floats
      if constexpr (TAPS == 4) {
        w[n] = *reinterpret_cast<const float4*>(cw + (size_t)(e + n) * 4);
      } else {
        const float* wp = cw + (size_t)(e + n) * TAPS;
        w[n] = make_float4(wp[0], wp[1], TAPS > 2 ? wp[2] : 0.f, 0.f);
      }
    }
#pragma unroll
    for (int j = 0; j < TAPS; j++) {
      const int ii = i - (TAPS - 1) + j;
      if (ii >= 0) {
        u[j].x += be.x; u[j].y += be.y; u[j].z += be.z; u[j].w += be.w;
      }
    }
    auto tap = [](const float4& v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; };
    float4 y = zero4;
#pragma unroll
    for (int j = 0; j < TAPS; j++) {
      y.x += tap(w[0], j) * u[j].x;
      y.y += tap(w[1], j) * u[j].y;
      y.z += tap(w[2], j) * u[j].z;
      y.w += tap(w[3], j) * u[j].w;
    }
    *reinterpret_cast<float4*>(row + e) = y;
    const float ss = (y.x * y.x + y.y * y.y) + (y.z * y.z + y.w * y.w);
    if (e < nq) sq += ss;
    else if (e < nq + nk) sk += ss;
    if (one_token) {
#pragma unroll
      for (int j = 0; j < TAPS - 1; j++) *reinterpret_cast<float4*>(st + (size_t)j * C + e) = u[j + 1];
    }
  }
  const float rq = qw ? 1.0f / sqrtf(block_sum256(sq, red) / (float)nq + c.eps) : 1.0f;
  const float rk = kw ? 1.0f / sqrtf(block_sum256(sk, red) / (float)nk + c.eps) : 1.0f;
  const size_t loc = (size_t)cache_loc[t];
  for (int e = tid * 4; e < C; e += 1024) {      // (each thread re-reads only what it wrote)
    float4 y = *reinterpret_cast<const float4*>(row + e);
    if (e < nq) {
      const float4 g = qw ? *reinterpret_cast<const float4*>(qw + e) : make_float4(1.f, 1.f, 1.f, 1.f);
      const float r = rq * c.scale;
      *reinterpret_cast<float4*>(q_out + (size_t)t * nq + e) = make_float4(y.x * r * g.x, y.y * r * g.y, y.z * r * g.z, y.w * r * g.w);
    } else {
      const bool isk = e < nq + nk;
      if (isk) {
        const float4 g = kw ? *reinterpret_cast<const float4*>(kw + (e - nq)) : make_float4(1.f, 1.f, 1.f, 1.f);
        y = make_float4(y.x * rk * g.x, y.y * rk * g.y, y.z * rk * g.z, y.w * rk * g.w);
      }
      KT* dst = isk ? kcache + loc * nk + (e - nq) : vcache + loc * nv + (e - nq - nk);
      if constexpr (sizeof(KT) == 2) {
        *reinterpret_cast<uint2*>(dst) = make_uint2(ktx_pk_bf16(y.x, y.y), ktx_pk_bf16(y.z, y.w));
      } else {
        *reinterpret_cast<float4*>(dst) = y;
      }
    }
  }
}

// the state of a causal convolution over C channels moves on behind a step: the slot's rows become the last taps - 1 inputs (this step's
// projections + bias; older ones from the old state when the request brought fewer).  thread = channel, rows oldest first
__global__ void __launch_bounds__(256) conv_state_update_kernel(int C, int taps, const int32_t* __restrict__ q_indptr,
                                                                const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                                const float* __restrict__ proj, int64_t ldp, const float* __restrict__ bias,
                                                                float* __restrict__ conv_state) {
  const int b = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
  if (e >= C) return;
  const int first = q_indptr[b], n = q_indptr[b + 1] - first;
  if (n <= 0) return;
  const bool carried = pos0[b] > 0;
  const float be = bias ? bias[e] : 0.f;
  float* st = conv_state + (size_t)slot[b] * (taps - 1) * C;
  for (int j = 0; j < taps - 1; j++) {      // row j takes the input n - (taps - 1) + j; an old row it may need lies further on (j + n > j)
    const int ii = n - (taps - 1) + j;
    float v = 0.f;
    if (ii >= 0) v = proj[(size_t)(first + ii) * ldp + e] + be;
    else if (carried) v = st[(size_t)(j + n) * C + e];
    st[(size_t)j * C + e] = v;
  }
}

// attention of ONE token (blockIdx.x) x HG query heads of one key head (blockIdx.y) x one key range (blockIdx.z) on the vector ALUs:
// tiles of KTN <= 64 keys and values staged in LDS as fp32; scores thread = (head, key); running maximum / sum per head by wavefronts;
// outputs thread = (head, value entry) in registers.
constexpr int SW_NACC = 32;
template <typename KT, typename OT>
__global__ void __launch_bounds__(256) swa_fwd_kernel(ktx_swa_config c, int T, int HG, int parts, int KTN, const float* __restrict__ q,
                                                      const KT* __restrict__ kcache, const KT* __restrict__ vcache,
                                                      const int32_t* __restrict__ tok_req, const int32_t* __restrict__ pos,
                                                      const int32_t* __restrict__ page_indptr, const int32_t* __restrict__ page_indices,
                                                      const float* __restrict__ sink, const float* __restrict__ dist_bias,
                                                      const float* __restrict__ vcs, int nsplit, float* __restrict__ scratch,
                                                      OT* __restrict__ out) {
  extern __shared__ float lds[];
  const int D = c.dim, V = c.vdim, DP = D + 1, VP = V + 1, G = c.kv_heads, HPG = c.heads / G;
  float* qs = lds;                         // [HG][D]
  float* kt = qs + (size_t)HG * D;         // [KTN][DP]
  float* vt = kt + (size_t)KTN * DP;       // [KTN][VP]
  float* sc = vt + (size_t)KTN * VP;       // [HG][KTN]
  float* mrow = sc + (size_t)HG * KTN;     // [HG] running maximum
  float* lrow = mrow + HG;                 // [HG] running sum
  float* crow = lrow + HG;                 // [HG] correction of this tile
  int* rowidx = reinterpret_cast<int*>(crow + HG);   // [KTN]
  int* jpos = rowidx + KTN;                          // [KTN] the keys' positions
  const int t = blockIdx.x, g = blockIdx.y / parts, part = blockIdx.y % parts, z = blockIdx.z;
  const int h0 = g * HPG + part * HG;
  const int nh = min(HG, HPG - part * HG);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int p = pos[t], b = tok_req[t];
  const int jlo = c.window > 0 ? max(0, p - c.window + 1) : 0, jhi = p + 1;
  // the keys the token sees, as one list: the kept first positions that lie in front of the window, then the window
  const int nfront = min(c.keep_first, jlo), nvis = nfront + (jhi - jlo);
  const int per = (nvis + nsplit - 1) / nsplit;
  const int j0 = z * per, j1 = min(nvis, j0 + per);
  for (int e = tid; e < nh * D; e += 256) qs[e] = q[((size_t)t * c.heads + h0) * D + e];
  for (int h = tid; h < HG; h += 256) {
    mrow[h] = -INFINITY;
    lrow[h] = 0.f;
  }
  float acc[SW_NACC];
#pragma unroll
  for (int i = 0; i < SW_NACC; i++) acc[i] = 0.f;
  const int nout = nh * V;
  const int32_t* pages = page_indices + page_indptr[b];
  for (int jt = j0; jt < j1; jt += KTN) {
    const int nk = min(KTN, j1 - jt);
    __syncthreads();
    if (tid < nk) {
      const int u = jt + tid, j = u < nfront ? u : jlo + (u - nfront);
      rowidx[tid] = pages[j / c.page_size] * c.page_size + j % c.page_size;
      jpos[tid] = j;
    }
    __syncthreads();
    for (int e = tid; e < nk * D; e += 256) {
      const int j = e / D, d = e % D;
      kt[(size_t)j * DP + d] = ld_elem(kcache, ((size_t)rowidx[j] * G + g) * D + d);
    }
    for (int e = tid; e < nk * V; e += 256) {
      const int j = e / V, d = e % V;
      vt[(size_t)j * VP + d] = ld_elem(vcache, ((size_t)rowidx[j] * G + g) * V + d);
    }
    __syncthreads();
    for (int e = tid; e < nh * KTN; e += 256) {
      const int h = e / KTN, j = e % KTN;
      if (j < nk) {
        const float* qh = qs + (size_t)h * D;
        const float* kj = kt + (size_t)j * DP;
        float s = 0.f;
        for (int d = 0; d < D; d++) s += qh[d] * kj[d];
        if (dist_bias) s += dist_bias[(size_t)min(p - jpos[j], c.bias_span) * c.heads + h0 + h];
        sc[(size_t)h * KTN + j] = s;      // (scale is folded into q)
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
    for (int i = 0; i < SW_NACC; i++) {
      const int e = tid + i * 256;
      if (e < nout) {
        const int h = e / V, l = e % V;
        float a = acc[i] * crow[h];
        const float* w = sc + (size_t)h * KTN;
        for (int j = 0; j < nk; j++) a += w[j] * vt[(size_t)j * VP + l];
        acc[i] = a;
      }
    }
  }
  __syncthreads();
  if (nsplit == 1) {
    const int NV = V / 2;
#pragma unroll
    for (int i = 0; i < SW_NACC; i++) {
      const int e = tid + i * 256;
      const bool live = e < nout;
      const int h = live ? e / V : 0, l = live ? e % V : 0;
      float o = 0.f;
      if (live) {
        const float m = mrow[h];
        if (sink) {
          const float sk = sink[h0 + h], M = fmaxf(m, sk);
          const float f = m == -INFINITY ? 0.f : expf(m - M);
          o = acc[i] * f / (lrow[h] * f + expf(sk - M));
        } else {
          o = lrow[h] > 0.f ? acc[i] / lrow[h] : 0.f;
        }
      }
      if (c.rot_values) {      // turn the pair (2m, 2m + 1) back by the token's own angle; the partner sits in the neighbouring thread
        const float other = __shfl_xor(o, 1);
        if (live) {
          const float co = vcs[(size_t)t * V + (l >> 1)], si = vcs[(size_t)t * V + NV + (l >> 1)];
          o = (l & 1) ? o * co - other * si : o * co + other * si;
        }
      }
      if (live) st_elem(out, ((size_t)t * c.heads + h0 + h) * V + l, o);
    }
    return;
  }
  float* partial = scratch + (((size_t)z * T + t) * c.heads + h0) * (V + 2);
#pragma unroll
  for (int i = 0; i < SW_NACC; i++) {
    const int e = tid + i * 256;
    if (e < nout) partial[(size_t)(e / V) * (V + 2) + e % V] = acc[i];
  }
  for (int h = tid; h < nh; h += 256) {
    partial[(size_t)h * (V + 2) + V] = mrow[h];
    partial[(size_t)h * (V + 2) + V + 1] = lrow[h];
  }
}

// merge the key ranges of one (token, head): thread = value entry; normalise with the sink, then turn the result back
template <typename OT>
__global__ void __launch_bounds__(256) swa_merge_kernel(int T, int H, int V, int nsplit, int rot_values, const float* __restrict__ scratch,
                                                        const float* __restrict__ sink, const float* __restrict__ vcs,
                                                        OT* __restrict__ out) {
  extern __shared__ float mw[];            // [nsplit] maxima, then [nsplit] weights exp(m_z - M) (0 for an empty range)
  float* ws = mw + nsplit;
  const int t = blockIdx.x, h = blockIdx.y;
  const size_t stride = (size_t)T * H * (V + 2);
  const float* base = scratch + ((size_t)t * H + h) * (V + 2);
  for (int z = threadIdx.x; z < nsplit; z += 256) {
    mw[z] = base[z * stride + V];
    ws[z] = base[z * stride + V + 1];
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
  const int NV = V / 2;
  for (int l0 = 0; l0 < V; l0 += 256) {
    const int l = l0 + threadIdx.x;
    const bool live = l < V;
    float a = 0.f;
    if (live) {
#pragma unroll 4
      for (int z = 0; z < nsplit; z++) a = fmaf(base[z * stride + l], ws[z], a);
      a *= inv;
    }
    if (rot_values) {
      const float other = __shfl_xor(a, 1);
      if (live) {
        const float co = vcs[(size_t)t * V + (l >> 1)], si = vcs[(size_t)t * V + NV + (l >> 1)];
        a = (l & 1) ? a * co - other * si : a * co + other * si;
      }
    }
    if (live) st_elem(out, ((size_t)t * H + h) * V + l, a);
  }
}

// The same attention on the matrix cores (bf16 caches).  The (token, head) pairs of a request that share key head g (blockIdx.y) are the
// rows of one query matrix: a workgroup takes 64 consecutive rows (its four wavefronts one 16-row MFMA tile each, query fragments
// resident in registers) and walks 32-key tiles of the union of its rows' windows: keys staged row-major, values transposed; scores,
// mask, running maximum and sum in fp32 (DPP reductions inside the 16-lane column groups), weights through a per-wavefront LDS tile
// into the second product.  Key ranges (blockIdx.z) leave unnormalised partial sums that swa_merge_kernel joins.
constexpr int SM_KT = 32, SM_PST = SM_KT + 8, SM_KSMAX = 8;
template <int NT, typename OT>
__global__ void __launch_bounds__(256) swa_mfma_kernel(ktx_swa_config c, int T, int row_tiles, const float* __restrict__ q,
                                                       const bf16_t* __restrict__ kcache, const bf16_t* __restrict__ vcache,
                                                       const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ pos0,
                                                       const int32_t* __restrict__ page_indptr, const int32_t* __restrict__ page_indices,
                                                       const float* __restrict__ sink, const float* __restrict__ dist_bias,
                                                       const float* __restrict__ vcs, int nsplit, float* __restrict__ scratch,
                                                       OT* __restrict__ out) {
  constexpr int V = NT * 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char sm_raw[];
  const int H = c.heads, G = c.kv_heads, HPG = H / G, D = c.dim, DPP = D + 8, KS = D / 32;
  bf16_t* Ks = reinterpret_cast<bf16_t*>(sm_raw);            // [SM_KT][DPP]
  bf16_t* Vt = Ks + (size_t)SM_KT * DPP;                      // [V][SM_PST]
  bf16_t* Ps = Vt + (size_t)V * SM_PST;                       // [4][16][SM_PST]
  int* rowidx = reinterpret_cast<int*>(Ps + 4 * 16 * SM_PST); // [SM_KT]
  const int b = blockIdx.x / row_tiles, rt = blockIdx.x % row_tiles, g = blockIdx.y, z = blockIdx.z;
  const int t0 = q_indptr[b], rows_total = (q_indptr[b + 1] - t0) * HPG, r0 = rt * 64;
  if (r0 >= rows_total) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
  const int p0 = pos0[b];
  const int tok_lo = r0 / HPG, tok_hi = (min(rows_total, r0 + 64) - 1) / HPG;
  const int klo = c.window > 0 ? max(0, p0 + tok_lo - c.window + 1) : 0, khi = p0 + tok_hi + 1;
  // the keys any of the rows sees, as one list: the kept first positions in front of the rows' windows, then the union of the windows
  const int nfront = min(c.keep_first, klo), nvis = nfront + (khi - klo);
  const int per = (((nvis + nsplit - 1) / nsplit) + SM_KT - 1) / SM_KT * SM_KT;
  const int j0 = z * per, j1 = min(nvis, j0 + per);
  const int rw0 = r0 + wave * 16;
  const bool active = rw0 < rows_total;
  // query fragments: lane = (row l16, 8 consecutive entries lq * 8 ..) of every 32-entry step
  sq_v8bf qf[SM_KSMAX];
  {
    const int ar = min(rw0 + l16, rows_total - 1);
    const bool live = rw0 + l16 < rows_total;
    const float* qrow = q + ((size_t)(t0 + ar / HPG) * H + g * HPG + ar % HPG) * D;
#pragma unroll
    for (int kk = 0; kk < SM_KSMAX; kk++) {
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; i++) v[i] = 0.f;
      if (kk < KS && live) {
        const int e0 = kk * 32 + lq * 8;
        const float4 x = *reinterpret_cast<const float4*>(qrow + e0), y = *reinterpret_cast<const float4*>(qrow + e0 + 4);
        v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w; v[4] = y.x; v[5] = y.y; v[6] = y.z; v[7] = y.w;
      }
      union { uint4 u; sq_v8bf f; } cv;
      cv.u.x = ktx_pk_bf16(v[0], v[1]); cv.u.y = ktx_pk_bf16(v[2], v[3]); cv.u.z = ktx_pk_bf16(v[4], v[5]); cv.u.w = ktx_pk_bf16(v[6], v[7]);
      qf[kk] = cv.f;
    }
  }
  // the four rows this lane holds of the score / output tiles (C layout: row lq * 4 + r, column l16)
  int prow[4], lorow[4];
  bool vrow[4];
  const float* brow[4];                    // the distance-bias column of the row's head
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int cr = rw0 + lq * 4 + r;
    vrow[r] = cr < rows_total;
    prow[r] = p0 + cr / HPG;
    lorow[r] = c.window > 0 ? max(0, prow[r] - c.window + 1) : 0;
    brow[r] = dist_bias ? dist_bias + g * HPG + cr % HPG : nullptr;
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
  const int ksegs = D / 8, vsegs = V / 8;
  bf16_t* Pw = Ps + (size_t)wave * 16 * SM_PST;
  for (int jt = j0; jt < j1; jt += SM_KT) {
    const int nk = min(SM_KT, j1 - jt);
    __syncthreads();
    if (tid < SM_KT) {
      const int u = jt + tid, j = u < nfront ? u : klo + (u - nfront);
      rowidx[tid] = tid < nk ? pages[j / c.page_size] * c.page_size + j % c.page_size : -1;
    }
    __syncthreads();
    for (int idx = tid; idx < SM_KT * ksegs; idx += 256) {
      const int key = idx / ksegs, e0 = (idx % ksegs) * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      const int row = rowidx[key];
      if (row >= 0) v = *reinterpret_cast<const uint4*>(kcache + ((size_t)row * G + g) * D + e0);
      *reinterpret_cast<uint4*>(Ks + (size_t)key * DPP + e0) = v;
    }
    for (int idx = tid; idx < SM_KT * vsegs; idx += 256) {
      const int key = idx % SM_KT, e0 = (idx / SM_KT) * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      const int row = rowidx[key];
      if (row >= 0) v = *reinterpret_cast<const uint4*>(vcache + ((size_t)row * G + g) * V + e0);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int i = 0; i < 8; i++) Vt[(size_t)(e0 + i) * SM_PST + key] = (bf16_t)((w[i >> 1] >> ((i & 1) * 16)) & 0xffffu);
    }
    __syncthreads();
    if (active) {
      v4f s0 = (v4f){0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
      for (int kk = 0; kk < SM_KSMAX; kk++) {
        if (kk < KS) {
          const sq_v8bf b0 = *reinterpret_cast<const sq_v8bf*>(Ks + (size_t)l16 * DPP + kk * 32 + lq * 8);
          const sq_v8bf b1 = *reinterpret_cast<const sq_v8bf*>(Ks + (size_t)(16 + l16) * DPP + kk * 32 + lq * 8);
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[kk], b0, s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[kk], b1, s1, 0, 0, 0);
        }
      }
      const int ua = jt + l16, ub = ua + 16;
      const int ja = ua < nfront ? ua : klo + (ua - nfront), jb = ub < nfront ? ub : klo + (ub - nfront);
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const bool oka = vrow[r] && ua < j1 && (ja >= lorow[r] || ja < c.keep_first) && ja <= prow[r];
        const bool okb = vrow[r] && ub < j1 && (jb >= lorow[r] || jb < c.keep_first) && jb <= prow[r];
        float sa = -INFINITY, sb = -INFINITY;      // (scale is folded into q)
        if (oka) sa = s0[r] + (brow[r] ? brow[r][(size_t)min(prow[r] - ja, c.bias_span) * H] : 0.f);
        if (okb) sb = s1[r] + (brow[r] ? brow[r][(size_t)min(prow[r] - jb, c.bias_span) * H] : 0.f);
        const float mt = row16_max(fmaxf(sa, sb));
        const float mn = fmaxf(mrun[r], mt);
        const float mb = mn == -INFINITY ? 0.f : mn;
        const float wa = oka ? __expf(sa - mb) : 0.f, wb = okb ? __expf(sb - mb) : 0.f;
        const float cr = mrun[r] == -INFINITY ? 0.f : __expf(mrun[r] - mb);
        lrun[r] = lrun[r] * cr + row16_sum(wa + wb);
        mrun[r] = mn;
#pragma unroll
        for (int n = 0; n < NT; n++) acc[n][r] *= cr;
        Pw[(lq * 4 + r) * SM_PST + l16] = to_bf16_rne(wa);
        Pw[(lq * 4 + r) * SM_PST + 16 + l16] = to_bf16_rne(wb);
      }
    }
    __syncthreads();
    if (active) {
      const sq_v8bf pf = *reinterpret_cast<const sq_v8bf*>(Pw + (size_t)l16 * SM_PST + lq * 8);
#pragma unroll
      for (int n = 0; n < NT; n++) {
        const sq_v8bf vb = *reinterpret_cast<const sq_v8bf*>(Vt + (size_t)(n * 16 + l16) * SM_PST + lq * 8);
        acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vb, acc[n], 0, 0, 0);
      }
    }
  }
  if (!active) return;
  constexpr int NV = V / 2;
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int cr = min(rw0 + lq * 4 + r, rows_total - 1);
    const int tok = t0 + cr / HPG, head = g * HPG + cr % HPG;
    const size_t grow = (size_t)tok * H + head;             // (token, head) row of out
    if (nsplit == 1) {
      float inv;
      if (sink) {
        const float sk = sink[head], M = fmaxf(mrun[r], sk);
        const float f = mrun[r] == -INFINITY ? 0.f : expf(mrun[r] - M);
        inv = f / (lrun[r] * f + expf(sk - M));
      } else {
        inv = lrun[r] > 0.f ? 1.0f / lrun[r] : 0.f;
      }
#pragma unroll
      for (int n = 0; n < NT; n++) {
        float o = acc[n][r] * inv;
        if (c.rot_values) {      // column n * 16 + l16 pairs with its neighbour column: the neighbouring lane of the quad
          const float other = ktx_dpp_f<KTX_DPP_QUAD_1032>(o);
          const int m = (n * 16 + l16) >> 1;
          const float co = vcs[(size_t)tok * V + m], si = vcs[(size_t)tok * V + NV + m];
          o = (l16 & 1) ? o * co - other * si : o * co + other * si;
        }
        if (vrow[r]) st_elem(out, grow * V + n * 16 + l16, o);
      }
    } else if (vrow[r]) {
      float* part = scratch + ((size_t)z * T * H + grow) * (V + 2);
#pragma unroll
      for (int n = 0; n < NT; n++) part[n * 16 + l16] = acc[n][r];
      if (l16 == 0) {
        part[V] = mrun[r];
        part[V + 1] = lrun[r];
      }
    }
  }
}

size_t swa_mfma_lds(const ktx_swa_config& c) {
  return ((size_t)SM_KT * (c.dim + 8) + (size_t)c.vdim * SM_PST + 4 * 16 * SM_PST) * 2 + SM_KT * 4;
}

// ---------------------------------------------------------------------------------------------------------------------
// selective scan.  thread = (token, channel) for the convolution
constexpr int SSM_MAX_TAPS = 8;
__global__ void __launch_bounds__(256) ssm_conv_kernel(ktx_ssm_config c, const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ pos0,
                                                       const int32_t* __restrict__ slot, const int32_t* __restrict__ tok_req,
                                                       const float* __restrict__ proj, int64_t ldp, int x_off, const float* __restrict__ w,
                                                       const float* __restrict__ bias, const float* __restrict__ conv_state,
                                                       float* __restrict__ xc) {
  const int t = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
  if (ch >= c.inner) return;
  const int b = tok_req[t], q0 = q_indptr[b], i = t - q0, K = c.taps;
  const bool cont = pos0[b] > 0;
  float acc = bias ? bias[ch] : 0.f;
  for (int j = 0; j < K; j++) {
    const int s = i - K + 1 + j;
    float v = 0.f;
    if (s >= 0) v = proj[(size_t)(q0 + s) * ldp + x_off + ch];
    else if (cont) v = conv_state[((size_t)slot[b] * (K - 1) + (K - 1 + s)) * c.inner + ch];
    acc += w[(size_t)ch * K + j] * v;
  }
  xc[(size_t)t * c.inner + ch] = silu_f32(acc);
}

// The recurrence: a workgroup owns 256 / LPC channels of one request; a channel's state entries are split over LPC neighbouring lanes
// (SS_NS each, in registers), their read-outs joined with DPP inside the 16-lane row (lane shuffles beyond it).  Tokens are taken SS_TC
// at a time: the chunk's B and C rows are staged in LDS once for all channels (two buffers, ONE barrier per chunk), the per-channel
// inputs of the NEXT chunk (step, x, gate) and its B | C rows are requested before the sequential part of the current one starts, and
// the steps' softplus, dt * x and the gate of a whole chunk are taken off the sequential path and shared by the lanes of a channel
// (each takes a part of the chunk's tokens; the values reach the others by DPP when they are used).
constexpr int SS_NS = 4, SS_TC = 16;
template <int LPC>
__device__ __forceinline__ float ssm_join(float y) {
  if constexpr (LPC >= 2) y += ktx_dpp_f<KTX_DPP_QUAD_1032>(y);
  if constexpr (LPC >= 4) y += ktx_dpp_f<KTX_DPP_QUAD_2301>(y);
  if constexpr (LPC >= 8) y += ktx_dpp_f<KTX_DPP_ROW_HALF_MIRROR>(y);
  if constexpr (LPC >= 16) y += ktx_dpp_f<KTX_DPP_ROW_MIRROR>(y);
  if constexpr (LPC >= 32) y += __shfl_xor(y, 16);
  if constexpr (LPC >= 64) y += __shfl_xor(y, 32);
  return y;
}

// value v of lane k of the SH lanes that share a channel's per-token work (SH = 1, 2 or 4 neighbouring lanes inside a quad)
template <int SH>
__device__ __forceinline__ float ssm_bcast(float v, int k) {
  if constexpr (SH == 1) return v;
  else if constexpr (SH == 2) return k == 0 ? ktx_dpp_f<0xA0>(v) : ktx_dpp_f<0xF5>(v);          // quad_perm [0,0,2,2] / [1,1,3,3]
  else return k == 0 ? ktx_dpp_f<0x00>(v) : k == 1 ? ktx_dpp_f<0x55>(v) : k == 2 ? ktx_dpp_f<0xAA>(v) : ktx_dpp_f<0xFF>(v);
}
// v_exp_f32 + v_rcp_f32, about 1 ulp each: the gate multiplies a read-out, it enters no recurrence
__device__ __forceinline__ float silu_fast(float z) { return z * __builtin_amdgcn_rcpf(1.0f + __expf(-z)); }

template <int LPC, typename OT>
__global__ void __launch_bounds__(256) ssm_scan_kernel(ktx_ssm_config c, const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ pos0,
                                                       const int32_t* __restrict__ slot, const float* __restrict__ xc,
                                                       const float* __restrict__ Bm, const float* __restrict__ Cm, int64_t ldbc,
                                                       const float* __restrict__ dt_raw, int64_t lddt, const float* __restrict__ dt_bias,
                                                       const float* __restrict__ A_log, const float* __restrict__ Dv,
                                                       const float* __restrict__ proj, int64_t ldp, int x_off, int z_off,
                                                       float* __restrict__ S, float* __restrict__ conv_state, OT* __restrict__ out) {
  constexpr int NP = LPC * SS_NS, CPB = 256 / LPC, CH = SS_TC * 2 * NP;     // CH floats of B | C per chunk
  constexpr int PER = (CH + 255) / 256;                                      // of them per thread
  constexpr int SH = LPC >= 4 ? 4 : LPC, MINE = SS_TC / SH;                  // lanes that share a channel's per-token work; tokens per lane
  extern __shared__ __attribute__((aligned(16))) float bc[];                 // [2][SS_TC][2][NP]
  const int b = blockIdx.y, tid = threadIdx.x;
  const int ch = blockIdx.x * CPB + tid / LPC, sl = tid % LPC, n0 = sl * SS_NS, sh = sl % SH;
  const bool live = ch < c.inner;
  const int N = c.state, q0 = q_indptr[b], q1 = q_indptr[b + 1];
  const bool cont = pos0[b] > 0;
  float A[SS_NS], st[SS_NS];
  float* Srow = S + ((size_t)slot[b] * c.inner + (live ? ch : 0)) * N;
#pragma unroll
  for (int i = 0; i < SS_NS; i++) {
    const bool ok = live && n0 + i < N;
    A[i] = ok ? -expf(A_log[(size_t)ch * N + n0 + i]) : 0.f;
    st[i] = ok && cont ? Srow[n0 + i] : 0.f;
  }
  const float dtb = live ? dt_bias[ch] : 0.f, dsk = live ? Dv[ch] : 0.f;
  // lane `sh` of a channel's sharing lanes takes the chunk's tokens sh, sh + SH, ...: their step, x and gate
  float ndt[MINE], nx[MINE], nz[MINE], nbc[PER];
  auto request = [&](int tc) {       // the chunk that starts at token tc: this lane's tokens and its share of the B | C rows
    const int nt = min(SS_TC, q1 - tc);
#pragma unroll
    for (int i = 0; i < MINE; i++) {
      const int tt = i * SH + sh;
      const bool ok = live && tt < nt;
      ndt[i] = ok ? dt_raw[(size_t)(tc + tt) * lddt + ch] : 0.f;
      nx[i] = ok ? xc[(size_t)(tc + tt) * c.inner + ch] : 0.f;
      nz[i] = ok ? proj[(size_t)(tc + tt) * ldp + z_off + ch] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < PER; k++) {
      const int e = tid + k * 256;
      const int tt = e / (2 * NP), r = e % (2 * NP), which = r / NP, n = r % NP;
      nbc[k] = e < CH && tt < nt && n < N ? (which ? Cm : Bm)[(size_t)(tc + tt) * ldbc + n] : 0.f;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int k = 0; k < PER; k++) {
      const int e = tid + k * 256;
      if (e < CH) bc[buf * CH + e] = nbc[k];
    }
  };
  if (q0 < q1) {
    request(q0);
    stage(0);
  }
  __syncthreads();
  int buf = 0;
  for (int tc = q0; tc < q1; tc += SS_TC, buf ^= 1) {
    const int nt = min(SS_TC, q1 - tc);
    float dt[MINE], dx[MINE], gz[MINE], sk[MINE];
#pragma unroll
    for (int i = 0; i < MINE; i++) {          // independent of the state: off the sequential path
      dt[i] = softplus_f32(ndt[i] + dtb);
      dx[i] = dt[i] * nx[i];
      sk[i] = dsk * nx[i];
      gz[i] = silu_fast(nz[i]);
    }
    const bool more = tc + SS_TC < q1;
    if (more) request(tc + SS_TC);           // in flight while this chunk runs
    const float* cur = bc + buf * CH;
#pragma unroll
    for (int tt = 0; tt < SS_TC; tt++) {
      if (tt < nt) {                        // (uniform over the workgroup)
        const float dtv = ssm_bcast<SH>(dt[tt / SH], tt % SH), dxv = ssm_bcast<SH>(dx[tt / SH], tt % SH);
        const float skv = ssm_bcast<SH>(sk[tt / SH], tt % SH), gzv = ssm_bcast<SH>(gz[tt / SH], tt % SH);
        const float4 Bt = *reinterpret_cast<const float4*>(cur + (size_t)tt * 2 * NP + n0);
        const float4 Ct = *reinterpret_cast<const float4*>(cur + (size_t)tt * 2 * NP + NP + n0);
        const float Bv[4] = {Bt.x, Bt.y, Bt.z, Bt.w}, Cv[4] = {Ct.x, Ct.y, Ct.z, Ct.w};
        float y = 0.f;
#pragma unroll
        for (int i = 0; i < SS_NS; i++) {
          st[i] = fmaf(__expf(dtv * A[i]), st[i], dxv * Bv[i]);
          y = fmaf(st[i], Cv[i], y);
        }
        y = ssm_join<LPC>(y);
        if (live && sl == 0) st_elem(out, (size_t)(tc + tt) * c.inner + ch, (y + skv) * gzv);
      }
    }
    if (more) stage(buf ^ 1);
    __syncthreads();
  }
  if (!live) return;
#pragma unroll
  for (int i = 0; i < SS_NS; i++)
    if (n0 + i < N) Srow[n0 + i] = st[i];
  if (sl == 0 && c.taps > 1) {             // the convolution's state moves on: its last taps - 1 inputs
    const int K1 = c.taps - 1, nn = q1 - q0;
    float* cs = conv_state + (size_t)slot[b] * K1 * c.inner + ch;
    float keep[SSM_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < SSM_MAX_TAPS; i++) {
      if (i < K1) {
        const int src = nn - K1 + i;
        keep[i] = src >= 0 ? proj[(size_t)(q0 + src) * ldp + x_off + ch] : (cont ? cs[(size_t)(nn + i) * c.inner] : 0.f);
      }
    }
#pragma unroll
    for (int i = 0; i < SSM_MAX_TAPS; i++)
      if (i < K1) cs[(size_t)i * c.inner] = keep[i];
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// router: one wavefront per token; lane holds outputs lane, lane + 64, ... (E <= 64 * SR_RE)
constexpr int SR_RE = 16;
__device__ __forceinline__ void softmax_route_token(int t, int lane, int E, int top, float sum_eps, const float* __restrict__ logits,
                                                    int64_t ldl, const float* __restrict__ corr, int32_t* idx, float* wts) {
  float s[SR_RE], ch[SR_RE];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < SR_RE; i++) {
    const int e = lane + i * 64;
    s[i] = e < E ? logits[(size_t)t * ldl + e] : -INFINITY;
    mx = fmaxf(mx, s[i]);
  }
  mx = wave_max(mx);
  float den = 0.f;
#pragma unroll
  for (int i = 0; i < SR_RE; i++) {
    s[i] = lane + i * 64 < E ? expf(s[i] - mx) : 0.f;
    den += s[i];
  }
  den = wave_sum(den);
#pragma unroll
  for (int i = 0; i < SR_RE; i++) {
    const int e = lane + i * 64;
    s[i] = s[i] / den;
    ch[i] = e < E ? s[i] + (corr ? corr[e] : 0.f) : -INFINITY;
  }
  float sum = 0.f;
  for (int k = 0; k < top; k++) {
    float bv = -INFINITY;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < SR_RE; i++) {
      const int e = lane + i * 64;
      if (e < E && ch[i] > bv) {
        bv = ch[i];
        be = e;
      }
    }
    for (int off = 32; off; off >>= 1) {
      const float ov = __shfl_xor(bv, off);
      const int oe = __shfl_xor(be, off);
      if (oe != 0x7fffffff && (be == 0x7fffffff || ov > bv || (ov == bv && oe < be))) {
        bv = ov;
        be = oe;
      }
    }
    float sv = 0.f;
#pragma unroll
    for (int i = 0; i < SR_RE; i++)
      if (lane + i * 64 == be) {
        sv = s[i];
        ch[i] = -INFINITY;
      }
    sv = wave_sum(sv);                     // the chosen output's score (its owner's value, zeros elsewhere)
    sum += sv;
    if (lane == 0) {
      idx[(size_t)t * top + k] = be;
      wts[(size_t)t * top + k] = sv;
    }
  }
  const float f = 1.0f / (sum + sum_eps);
  __builtin_amdgcn_wave_barrier();
  if (lane == 0)
    for (int k = 0; k < top; k++) wts[(size_t)t * top + k] *= f;
}

__global__ void __launch_bounds__(256) softmax_route_kernel(int T, int E, int top, float sum_eps, const float* __restrict__ logits,
                                                            int64_t ldl, const float* __restrict__ corr, int32_t* __restrict__ idx,
                                                            float* __restrict__ wts) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t < T) softmax_route_token(t, lane, E, top, sum_eps, logits, ldl, corr, idx, wts);
}

// router and expert sort of a SMALL step (decode) in one launch: the sixteen wavefronts of the one workgroup route the tokens, then the
// workgroup sorts the pairs it has just written (moe_plan_block)
__global__ void __launch_bounds__(1024) softmax_route_plan_kernel(int T, int E, int top, float sum_eps, const float* __restrict__ logits,
                                                                  int64_t ldl, const float* __restrict__ corr, int32_t* idx, float* wts,
                                                                  int tile_m, int32_t* __restrict__ group_off,
                                                                  int32_t* __restrict__ sorted_tok, int32_t* __restrict__ pair_pos,
                                                                  int32_t* __restrict__ sorted_group, int32_t* __restrict__ tile_group,
                                                                  int32_t* __restrict__ tile_row0, int32_t* __restrict__ num_tiles) {
  extern __shared__ int32_t pl[];          // counts [E] | offsets [E + 1] | cursor [E]
  for (int t = threadIdx.x >> 6; t < T; t += 16) softmax_route_token(t, threadIdx.x & 63, E, top, sum_eps, logits, ldl, corr, idx, wts);
  __threadfence_block();
  __syncthreads();
  moe_plan_block(T * top, E, top, tile_m, idx, group_off, sorted_tok, pair_pos, sorted_group, tile_group, tile_row0, num_tiles, pl);
}

}  // namespace

extern "C" {

int ktx_resid_norm(int T, int W, float* d_x, const ktx_resid_args* a, ktx_stream_t stream) {
  KTX_REQUIRE(a && T >= 0 && W > 0 && d_x, "ktx_resid_norm: T >= 0, W > 0, x");
  KTX_REQUIRE((size_t)W * 4 <= 150 * 1024, "ktx_resid_norm: a row must fit the LDS");
  const bool adds = a->y || a->ey;
  KTX_REQUIRE(!a->ey || (a->pair_pos && a->topk_idx && a->topk_w && a->top > 0 && a->h_in && dtype_ok(a->h_dtype)),
              "ktx_resid_norm: the gathered term needs pair_pos, topk_idx, topk_w, top, h_in");
  KTX_REQUIRE(!a->y_norm_w || a->y, "ktx_resid_norm: y_norm_w without y");
  KTX_REQUIRE(!a->rows || !adds, "ktx_resid_norm: a row gather only without an addition");
  KTX_REQUIRE(!a->norm_g || (a->out && dtype_ok(a->out_dtype)), "ktx_resid_norm: the norm needs its output");
  KTX_REQUIRE(a->halo <= 0 || (a->norm_g && !a->rows && a->B > 0 && a->q_indptr && a->pos0 && a->slot && a->tok_req && a->conv_state &&
                               a->out_dtype == KTX_SEQ_F32),
              "ktx_resid_norm: halo rows need the batch's tensors, the state and an fp32 output");
  KTX_REQUIRE(!a->conv_w || (a->halo <= 0 && a->norm_g && !a->rows && a->conv_taps >= 1 && a->conv_taps <= RN_MAX_HALO + 1 &&
                             (a->conv_taps == 1 || (a->q_indptr && a->pos0 && a->slot && a->tok_req && a->conv_state))),
              "ktx_resid_norm: the fused convolution needs 1 <= taps <= 9, no halo and, beyond one tap, the batch's tensors and the state");
  if (T == 0 || (!adds && !a->norm_g)) return 0;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)W * 4;
#define KTX_RN_GO(OT, HT)                                                                        \
  do {                                                                                           \
    KTX_HIP(ktx_set_max_lds((const void*)resid_norm_kernel<OT, HT>, 150 * 1024));                \
    resid_norm_kernel<OT, HT><<<T, 256, lds, st>>>(W, d_x, *a);                                  \
  } while (0)
  const bool obf = a->norm_g && a->out_dtype == KTX_SEQ_BF16, hbf = a->ey && a->h_dtype == KTX_SEQ_BF16;
  if (obf && hbf) KTX_RN_GO(bf16_t, bf16_t);
  else if (obf) KTX_RN_GO(bf16_t, float);
  else if (hbf) KTX_RN_GO(float, bf16_t);
  else KTX_RN_GO(float, float);
#undef KTX_RN_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_input_conv(int B, int T, int W, int taps, const float* d_hx, const float* d_w, const int32_t* d_q_indptr, const int32_t* d_slot,
                   const int32_t* d_tok_req, float* d_conv_state, void* d_out, int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(B >= 0 && T >= 0 && W > 0 && taps >= 2 && d_hx && d_w && d_q_indptr && d_slot && d_tok_req && d_conv_state && d_out &&
                  dtype_ok(out_dtype),
              "ktx_input_conv: taps >= 2, pointers");
  if (T == 0) return 0;
  const dim3 grid(T, (W + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (out_dtype == KTX_SEQ_F32)
    input_conv_kernel<float><<<grid, 256, 0, st>>>(W, taps, d_hx, d_w, d_q_indptr, d_slot, d_tok_req, d_conv_state, (float*)d_out);
  else
    input_conv_kernel<bf16_t><<<grid, 256, 0, st>>>(W, taps, d_hx, d_w, d_q_indptr, d_slot, d_tok_req, d_conv_state, (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_rows_mul_lookup(int T, int n, const float* d_a, int64_t lda, const void* d_table, int table_dtype, int64_t ldt, int col0,
                        const int32_t* d_tokens, void* d_out, int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && n > 0 && d_a && d_table && d_tokens && d_out && dtype_ok(table_dtype) && dtype_ok(out_dtype) && col0 >= 0 &&
                  col0 + n <= ldt && lda >= n,
              "ktx_rows_mul_lookup: arguments");
  if (T == 0) return 0;
  const size_t total = (size_t)T * n;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
#define KTX_ML_GO(TT, OT) \
  rows_mul_lookup_kernel<TT, OT><<<blocks, 256, 0, st>>>(total, n, d_a, lda, (const TT*)d_table, ldt, col0, d_tokens, (OT*)d_out)
  if (table_dtype == KTX_SEQ_F32) {
    if (out_dtype == KTX_SEQ_F32) KTX_ML_GO(float, float);
    else KTX_ML_GO(float, bf16_t);
  } else {
    if (out_dtype == KTX_SEQ_F32) KTX_ML_GO(bf16_t, float);
    else KTX_ML_GO(bf16_t, bf16_t);
  }
#undef KTX_ML_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

static int swa_check(const ktx_swa_config* c, const char* who) {
  KTX_REQUIRE(c && c->heads > 0 && c->kv_heads > 0 && c->heads % c->kv_heads == 0 && c->dim > 0 && c->vdim > 0 && c->page_size > 0 &&
                  dtype_ok(c->cache_dtype),
              std::string(who) + ": heads a multiple of kv_heads, positive sizes, a known cache type");
  KTX_REQUIRE(c->rot_dims >= 0 && c->rot_dims % 2 == 0 && c->rot_dims <= c->dim, std::string(who) + ": rot_dims even and at most dim");
  KTX_REQUIRE(!c->rot_values || c->vdim % 2 == 0, std::string(who) + ": rotated values need an even vdim");
  KTX_REQUIRE(c->keep_first >= 0 && c->bias_span >= 0, std::string(who) + ": keep_first and bias_span are not negative");
  return 0;
}

int ktx_swa_prep(const ktx_swa_config* cfg, int T, const float* d_proj, int64_t ldp, int q_off, int k_off, int v_off,
                 const double* d_inv_freq, const double* d_v_inv_freq, const int32_t* d_pos, const int32_t* d_cache_loc, void* d_kcache,
                 void* d_vcache, float* d_q_out, float* d_vcs, ktx_stream_t stream) {
  if (swa_check(cfg, "ktx_swa_prep")) return -1;
  KTX_REQUIRE(T >= 0 && d_proj && d_pos && d_cache_loc && d_kcache && d_vcache && d_q_out, "ktx_swa_prep: null pointer");
  KTX_REQUIRE(cfg->rot_dims == 0 || d_inv_freq, "ktx_swa_prep: rotation without frequencies");
  KTX_REQUIRE(!cfg->rot_values || (d_v_inv_freq && d_vcs), "ktx_swa_prep: rotated values need their frequencies and the table");
  if (T == 0) return 0;
  const size_t lds = ((size_t)cfg->rot_dims + (cfg->rot_values ? cfg->vdim : 0) + (size_t)cfg->heads * cfg->dim +
                      (size_t)cfg->kv_heads * (cfg->dim + cfg->vdim) + 2) * 4;
  KTX_REQUIRE(lds <= 150 * 1024, "ktx_swa_prep: a token's q | k | v row and the angle tables must fit the LDS");
  KTX_HIP(ktx_set_max_lds((const void*)swa_prep_kernel<float>, 150 * 1024));
  KTX_HIP(ktx_set_max_lds((const void*)swa_prep_kernel<bf16_t>, 150 * 1024));
  hipStream_t st = (hipStream_t)stream;
  if (cfg->cache_dtype == KTX_SEQ_F32)
    swa_prep_kernel<float><<<T, 256, lds, st>>>(*cfg, d_proj, ldp, q_off, k_off, v_off, d_inv_freq, d_v_inv_freq, d_pos, d_cache_loc,
                                                (float*)d_kcache, (float*)d_vcache, d_q_out, d_vcs);
  else
    swa_prep_kernel<bf16_t><<<T, 256, lds, st>>>(*cfg, d_proj, ldp, q_off, k_off, v_off, d_inv_freq, d_v_inv_freq, d_pos, d_cache_loc,
                                                 (bf16_t*)d_kcache, (bf16_t*)d_vcache, d_q_out, d_vcs);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_swa_conv_prep(const ktx_swa_config* cfg, int B, int T, int max_q_len, int taps, const float* d_proj, int64_t ldp, const float* d_bias,
                      const float* d_conv_w, const float* d_q_norm_w, const float* d_k_norm_w, const int32_t* d_q_indptr,
                      const int32_t* d_pos0, const int32_t* d_slot, const int32_t* d_tok_req, float* d_conv_state,
                      const int32_t* d_cache_loc, void* d_kcache, void* d_vcache, float* d_q_out, ktx_stream_t stream) {
  if (swa_check(cfg, "ktx_swa_conv_prep")) return -1;
  KTX_REQUIRE(B >= 0 && T >= 0 && max_q_len >= 0 && d_proj && d_q_indptr && d_pos0 && d_slot && d_tok_req && d_cache_loc && d_kcache && d_vcache && d_q_out,
              "ktx_swa_conv_prep: null pointer");
  KTX_REQUIRE(taps >= 0 && taps <= CP_MAX_TAPS && (taps <= 1 || (d_conv_w && d_conv_state)),
              "ktx_swa_conv_prep: at most 16 taps; a convolution needs its weights and state slots");
  KTX_REQUIRE(cfg->rot_dims == 0 && !cfg->rot_values, "ktx_swa_conv_prep: no rotation in this form");
  const int C = cfg->heads * cfg->dim + cfg->kv_heads * (cfg->dim + cfg->vdim);
  KTX_REQUIRE(ldp >= C, "ktx_swa_conv_prep: rows of q | k | v");
  KTX_REQUIRE((size_t)C * 4 <= 150 * 1024, "ktx_swa_conv_prep: a token's q | k | v row must fit the LDS");
  if (T == 0 || B == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = (size_t)C * 4;
  const int nq = cfg->heads * cfg->dim, nk = cfg->kv_heads * cfg->dim, nv = cfg->kv_heads * cfg->vdim;
  const bool vec = taps >= 2 && taps <= 4 && nq % 4 == 0 && nk % 4 == 0 && nv % 4 == 0 && ldp % 4 == 0 && aligned16(d_proj) &&
                   aligned16(d_conv_w) && aligned16(d_conv_state) && (!d_bias || aligned16(d_bias)) && (!d_q_norm_w || aligned16(d_q_norm_w)) &&
                   (!d_k_norm_w || aligned16(d_k_norm_w)) && aligned16(d_q_out) && aligned16(d_kcache) && aligned16(d_vcache);
  if (vec) {
    const int one = max_q_len == 1 ? 1 : 0;
#define KTX_CP_GO(KT, TAPS)                                                                                                          \
  do {                                                                                                                               \
    KTX_HIP(ktx_set_max_lds((const void*)swa_conv_prep_vec_kernel<KT, TAPS>, 150 * 1024));                                           \
    swa_conv_prep_vec_kernel<KT, TAPS><<<T, 256, lds, st>>>(*cfg, d_proj, ldp, d_bias, d_conv_w, d_q_norm_w, d_k_norm_w, d_q_indptr,  \
                                                            d_pos0, d_slot, d_tok_req, d_conv_state, one, d_cache_loc, (KT*)d_kcache, \
                                                            (KT*)d_vcache, d_q_out);                                                 \
  } while (0)
#define KTX_CP_TAPS(KT)               \
  do {                                \
    if (taps == 2) KTX_CP_GO(KT, 2);  \
    else if (taps == 3) KTX_CP_GO(KT, 3); \
    else KTX_CP_GO(KT, 4);            \
  } while (0)
    if (cfg->cache_dtype == KTX_SEQ_F32) KTX_CP_TAPS(float);
    else KTX_CP_TAPS(bf16_t);
#undef KTX_CP_TAPS
#undef KTX_CP_GO
    KTX_HIP(hipGetLastError());
    if (!one) {
      conv_state_update_kernel<<<dim3((C + 255) / 256, B), 256, 0, st>>>(C, taps, d_q_indptr, d_pos0, d_slot, d_proj, ldp, d_bias, d_conv_state);
      KTX_HIP(hipGetLastError());
    }
    return 0;
  }
  if (cfg->cache_dtype == KTX_SEQ_F32) {
    KTX_HIP(ktx_set_max_lds((const void*)swa_conv_prep_kernel<float>, 150 * 1024));
    swa_conv_prep_kernel<float><<<T, 256, lds, st>>>(*cfg, taps, d_proj, ldp, d_bias, d_conv_w, d_q_norm_w, d_k_norm_w, d_q_indptr, d_pos0,
                                                     d_slot, d_tok_req, d_conv_state, d_cache_loc, (float*)d_kcache, (float*)d_vcache, d_q_out);
  } else {
    KTX_HIP(ktx_set_max_lds((const void*)swa_conv_prep_kernel<bf16_t>, 150 * 1024));
    swa_conv_prep_kernel<bf16_t><<<T, 256, lds, st>>>(*cfg, taps, d_proj, ldp, d_bias, d_conv_w, d_q_norm_w, d_k_norm_w, d_q_indptr, d_pos0,
                                                      d_slot, d_tok_req, d_conv_state, d_cache_loc, (bf16_t*)d_kcache, (bf16_t*)d_vcache,
                                                      d_q_out);
  }
  KTX_HIP(hipGetLastError());
  if (taps > 1) {      // second launch: the state moves on only after every token of the step has read it
    conv_state_update_kernel<<<dim3((C + 255) / 256, B), 256, 0, st>>>(C, taps, d_q_indptr, d_pos0, d_slot, d_proj, ldp, d_bias, d_conv_state);
    KTX_HIP(hipGetLastError());
  }
  return 0;
}

static int swa_merge(const ktx_swa_config* cfg, int T, int nsplit, const float* d_scratch, const float* d_sink, const float* d_vcs,
                     void* d_out, int out_dtype, hipStream_t st) {
  const dim3 mg(T, cfg->heads);
  if (out_dtype == KTX_SEQ_F32)
    swa_merge_kernel<float><<<mg, 256, (size_t)nsplit * 8, st>>>(T, cfg->heads, cfg->vdim, nsplit, cfg->rot_values, d_scratch, d_sink, d_vcs,
                                                                 (float*)d_out);
  else
    swa_merge_kernel<bf16_t><<<mg, 256, (size_t)nsplit * 8, st>>>(T, cfg->heads, cfg->vdim, nsplit, cfg->rot_values, d_scratch, d_sink, d_vcs,
                                                                  (bf16_t*)d_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_swa_forward(const ktx_swa_config* cfg, int T, const float* d_q, const void* d_kcache, const void* d_vcache,
                    const int32_t* d_tok_req, const int32_t* d_pos, const int32_t* d_page_indptr, const int32_t* d_page_indices,
                    const float* d_sink, const float* d_dist_bias, const float* d_vcs, int nsplit, float* d_scratch, void* d_out,
                    int out_dtype, ktx_stream_t stream) {
  if (swa_check(cfg, "ktx_swa_forward")) return -1;
  KTX_REQUIRE(T >= 0 && d_q && d_kcache && d_vcache && d_tok_req && d_pos && d_page_indptr && d_page_indices && d_out && dtype_ok(out_dtype),
              "ktx_swa_forward: null pointer");
  KTX_REQUIRE(!cfg->rot_values || d_vcs, "ktx_swa_forward: rotated values need the table of their angles");
  KTX_REQUIRE(nsplit >= 1 && nsplit <= 4096 && (nsplit == 1 || d_scratch), "ktx_swa_forward: 1 <= nsplit <= 4096, scratch when > 1");
  if (T == 0) return 0;
  const int D = cfg->dim, V = cfg->vdim, HPG = cfg->heads / cfg->kv_heads;
  KTX_REQUIRE(V <= 256 * SW_NACC, "ktx_swa_forward: vdim <= 8192");
  const size_t budget = 96 * 1024;
  int HG = std::min(HPG, std::max(1, 256 * SW_NACC / V));
  int KTN = 64;
  auto lds_of = [&](int hg, int ktn) {
    return ((size_t)hg * D + (size_t)ktn * (D + 1) + (size_t)ktn * (V + 1) + (size_t)hg * ktn + 3 * (size_t)hg + 2 * (size_t)ktn) * 4;
  };
  while (KTN > 8 && lds_of(1, KTN) > budget) KTN /= 2;
  while (HG > 1 && lds_of(HG, KTN) > budget) HG = (HG + 1) / 2;
  KTX_REQUIRE(lds_of(HG, KTN) <= 150 * 1024, "ktx_swa_forward: one head's query and 8 keys and values do not fit the LDS");
  const size_t lds = lds_of(HG, KTN);
  const int parts = (HPG + HG - 1) / HG;
  const dim3 grid(T, cfg->kv_heads * parts, nsplit);
  hipStream_t st = (hipStream_t)stream;
#define KTX_SW_GO(KT, OT)                                                                                                          \
  do {                                                                                                                             \
    KTX_HIP(ktx_set_max_lds((const void*)swa_fwd_kernel<KT, OT>, 150 * 1024));                                                     \
    swa_fwd_kernel<KT, OT><<<grid, 256, lds, st>>>(*cfg, T, HG, parts, KTN, d_q, (const KT*)d_kcache, (const KT*)d_vcache, d_tok_req, \
                                                   d_pos, d_page_indptr, d_page_indices, d_sink, d_dist_bias, d_vcs, nsplit, d_scratch, (OT*)d_out); \
  } while (0)
  if (cfg->cache_dtype == KTX_SEQ_F32) {
    if (out_dtype == KTX_SEQ_F32) KTX_SW_GO(float, float);
    else KTX_SW_GO(float, bf16_t);
  } else {
    if (out_dtype == KTX_SEQ_F32) KTX_SW_GO(bf16_t, float);
    else KTX_SW_GO(bf16_t, bf16_t);
  }
#undef KTX_SW_GO
  KTX_HIP(hipGetLastError());
  if (nsplit > 1) return swa_merge(cfg, T, nsplit, d_scratch, d_sink, d_vcs, d_out, out_dtype, st);
  return 0;
}

int ktx_swa_mfma_eligible(const ktx_swa_config* c) {
  if (!c || c->cache_dtype != KTX_SEQ_BF16) return 0;
  if (c->dim % 32 != 0 || c->dim > 32 * SM_KSMAX) return 0;
  const int V = c->vdim;
  if (!((V % 16 == 0 && V >= 16 && V <= 128) || V == 256)) return 0;
  return swa_mfma_lds(*c) <= 150 * 1024;
}

int ktx_swa_mfma(const ktx_swa_config* cfg, int B, int T, int max_q_len, const float* d_q, const void* d_kcache, const void* d_vcache,
                 const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_page_indptr, const int32_t* d_page_indices,
                 const float* d_sink, const float* d_dist_bias, const float* d_vcs, int nsplit, float* d_scratch, void* d_out, int out_dtype,
                 ktx_stream_t stream) {
  if (swa_check(cfg, "ktx_swa_mfma")) return -1;
  KTX_REQUIRE(ktx_swa_mfma_eligible(cfg), "ktx_swa_mfma: bf16 caches, dim a multiple of 32 up to 256, vdim a multiple of 16 up to 128, or 256");
  KTX_REQUIRE(B >= 0 && T >= 0 && max_q_len >= 0 && d_q && d_kcache && d_vcache && d_q_indptr && d_pos0 && d_page_indptr &&
                  d_page_indices && d_out && dtype_ok(out_dtype),
              "ktx_swa_mfma: null pointer");
  KTX_REQUIRE(!cfg->rot_values || d_vcs, "ktx_swa_mfma: rotated values need the table of their angles");
  KTX_REQUIRE(nsplit >= 1 && nsplit <= 4096 && (nsplit == 1 || d_scratch), "ktx_swa_mfma: 1 <= nsplit <= 4096, scratch when > 1");
  KTX_REQUIRE(aligned16(d_q) && aligned16(d_kcache) && aligned16(d_vcache), "ktx_swa_mfma: 16-byte aligned q and caches");
  if (B == 0 || T == 0 || max_q_len == 0) return 0;
  const int HPG = cfg->heads / cfg->kv_heads;
  const int row_tiles = (int)(((int64_t)max_q_len * HPG + 63) / 64);
  KTX_REQUIRE(cfg->kv_heads <= 65535, "ktx_swa_mfma: up to 65535 key heads");
  const dim3 grid((unsigned)B * row_tiles, cfg->kv_heads, nsplit);
  const size_t lds = swa_mfma_lds(*cfg);
  hipStream_t st = (hipStream_t)stream;
  const int V = cfg->vdim;
#define KTX_SM_GO(NT, OT)                                                                                                             \
  do {                                                                                                                                \
    KTX_HIP(ktx_set_max_lds((const void*)swa_mfma_kernel<NT, OT>, 150 * 1024));                                                       \
    swa_mfma_kernel<NT, OT><<<grid, 256, lds, st>>>(*cfg, T, row_tiles, d_q, (const bf16_t*)d_kcache, (const bf16_t*)d_vcache,        \
                                                    d_q_indptr, d_pos0, d_page_indptr, d_page_indices, d_sink, d_dist_bias, d_vcs, nsplit, d_scratch, \
                                                    (OT*)d_out);                                                                      \
  } while (0)
#define KTX_SM_NT(OT)                  \
  do {                                 \
    if (V == 16) KTX_SM_GO(1, OT);     \
    else if (V == 32) KTX_SM_GO(2, OT); \
    else if (V == 48) KTX_SM_GO(3, OT); \
    else if (V == 64) KTX_SM_GO(4, OT); \
    else if (V == 80) KTX_SM_GO(5, OT); \
    else if (V == 96) KTX_SM_GO(6, OT); \
    else if (V == 112) KTX_SM_GO(7, OT); \
    else if (V == 128) KTX_SM_GO(8, OT); \
    else KTX_SM_GO(16, OT);            \
  } while (0)
  if (out_dtype == KTX_SEQ_F32) KTX_SM_NT(float);
  else KTX_SM_NT(bf16_t);
#undef KTX_SM_NT
#undef KTX_SM_GO
  KTX_HIP(hipGetLastError());
  if (nsplit > 1) return swa_merge(cfg, T, nsplit, d_scratch, d_sink, d_vcs, d_out, out_dtype, st);
  return 0;
}

static int ssm_check(const ktx_ssm_config* c, const char* who) {
  KTX_REQUIRE(c && c->inner > 0 && c->state > 0 && c->state <= 256 && c->dt_rank > 0 && c->taps >= 1 && c->taps <= SSM_MAX_TAPS + 1,
              std::string(who) + ": inner, dt_rank > 0, 0 < state <= 256, 1 <= taps <= 9");
  return 0;
}

int ktx_ssm_conv(const ktx_ssm_config* cfg, int B, int T, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                 const int32_t* d_tok_req, const float* d_proj, int64_t ldp, int x_off, const float* d_w, const float* d_bias,
                 const float* d_conv_state, float* d_xc, ktx_stream_t stream) {
  if (ssm_check(cfg, "ktx_ssm_conv")) return -1;
  KTX_REQUIRE(B >= 0 && T >= 0 && d_q_indptr && d_pos0 && d_slot && d_tok_req && d_proj && d_w && d_xc && (cfg->taps == 1 || d_conv_state),
              "ktx_ssm_conv: null pointer");
  if (T == 0) return 0;
  const dim3 grid(T, (cfg->inner + 255) / 256);
  ssm_conv_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_tok_req, d_proj, ldp, x_off, d_w, d_bias,
                                                         d_conv_state, d_xc);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_ssm_scan(const ktx_ssm_config* cfg, int B, int T, int max_q_len, const int32_t* d_q_indptr, const int32_t* d_pos0,
                 const int32_t* d_slot, const float* d_xc, const float* d_Bm, const float* d_Cm, int64_t ldbc, const float* d_dt_raw,
                 int64_t lddt, const float* d_dt_bias, const float* d_A_log, const float* d_D, const float* d_proj, int64_t ldp, int x_off,
                 int z_off, float* d_S, float* d_conv_state, void* d_out, int out_dtype, ktx_stream_t stream) {
  if (ssm_check(cfg, "ktx_ssm_scan")) return -1;
  KTX_REQUIRE(B >= 0 && T >= 0 && d_q_indptr && d_pos0 && d_slot && d_xc && d_Bm && d_Cm && d_dt_raw && d_dt_bias && d_A_log && d_D &&
                  d_proj && d_S && d_out && dtype_ok(out_dtype) && (cfg->taps == 1 || d_conv_state),
              "ktx_ssm_scan: null pointer");
  KTX_REQUIRE(B <= 65535, "ktx_ssm_scan: up to 65535 requests");
  if (B == 0 || T == 0) return 0;
  (void)max_q_len;
  int lpc = 1;
  while (lpc * SS_NS < cfg->state) lpc *= 2;
  hipStream_t st = (hipStream_t)stream;
#define KTX_SS_GO(LPC, OT)                                                                                                         \
  do {                                                                                                                             \
    const dim3 grid((cfg->inner + 256 / LPC - 1) / (256 / LPC), B);                                                                \
    ssm_scan_kernel<LPC, OT><<<grid, 256, (size_t)2 * SS_TC * 2 * LPC * SS_NS * 4, st>>>(                                          \
        *cfg, d_q_indptr, d_pos0, d_slot, d_xc, d_Bm, d_Cm, ldbc, d_dt_raw, lddt, d_dt_bias, d_A_log, d_D, d_proj, ldp, x_off, z_off, \
        d_S, d_conv_state, (OT*)d_out);                                                                                            \
  } while (0)
#define KTX_SS_LPC(OT)                  \
  do {                                  \
    if (lpc == 1) KTX_SS_GO(1, OT);     \
    else if (lpc == 2) KTX_SS_GO(2, OT); \
    else if (lpc == 4) KTX_SS_GO(4, OT); \
    else if (lpc == 8) KTX_SS_GO(8, OT); \
    else if (lpc == 16) KTX_SS_GO(16, OT); \
    else if (lpc == 32) KTX_SS_GO(32, OT); \
    else KTX_SS_GO(64, OT);             \
  } while (0)
  if (out_dtype == KTX_SEQ_F32) KTX_SS_LPC(float);
  else KTX_SS_LPC(bf16_t);
#undef KTX_SS_LPC
#undef KTX_SS_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_softmax_route(int T, int E, int top, float sum_eps, const float* d_logits, int64_t ldl, const float* d_correction,
                      int32_t* d_topk_idx, float* d_topk_w, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && E <= 64 * SR_RE && d_logits && d_topk_idx && d_topk_w && ldl >= E,
              "ktx_softmax_route: 0 < top <= outputs <= 1024");
  if (T == 0) return 0;
  softmax_route_kernel<<<(T + 3) / 4, 256, 0, (hipStream_t)stream>>>(T, E, top, sum_eps, d_logits, ldl, d_correction, d_topk_idx, d_topk_w);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_softmax_route_plan(int T, int E, int top, float sum_eps, const float* d_logits, int64_t ldl, const float* d_correction,
                           int32_t* d_topk_idx, float* d_topk_w, int tile_m, int32_t* d_group_off, int32_t* d_sorted_tok,
                           int32_t* d_pair_pos, int32_t* d_sorted_group, int32_t* d_tile_group, int32_t* d_tile_row0, int32_t* d_num_tiles,
                           ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && T <= KTX_ROUTE_PLAN_MAX_T && E > 0 && top > 0 && top <= E && E <= 64 * SR_RE && d_logits && d_topk_idx && d_topk_w &&
                  ldl >= E && tile_m > 0 && d_group_off && d_sorted_tok && d_pair_pos && d_sorted_group && d_tile_group && d_tile_row0 &&
                  d_num_tiles,
              "ktx_softmax_route_plan: a small step (T <= 256), 0 < top <= outputs <= 1024, pointers");
  softmax_route_plan_kernel<<<1, 1024, (size_t)(3 * E + 1) * 4, (hipStream_t)stream>>>(
      T, E, top, sum_eps, d_logits, ldl, d_correction, d_topk_idx, d_topk_w, tile_m, d_group_off, d_sorted_tok, d_pair_pos, d_sorted_group,
      d_tile_group, d_tile_row0, d_num_tiles);
  KTX_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
