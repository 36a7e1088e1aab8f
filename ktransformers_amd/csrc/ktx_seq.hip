// ktx_seq.hip — sequence-mixer kernels behind include/ktx_seq.h: sinusoidal embedding, a shape-agnostic dense GEMM (bf16 or
// fp32 MFMA) with its decode-sized streaming forms, sigmoid-weighted grouped-query attention with head mixing over a paged key cache
// (values = un-normed keys; a matrix-core kernel for prompts and decode steps, a vector-ALU kernel for every other shape and for fp32),
// the mLSTM matrix-memory recurrence over state slots (gate scan, token-by-token kernel, 16-token chunk kernel on the fp32 matrix
// cores), and the fp32 RMS-norm glue that adds into the residual stream.
//
// Everything a recurrence or a score touches is fp32: the residual, norms, scores, attention weights and their mixing, gates,
// exponentials and the state.  Element types only select how weights, activations and the key cache are stored and which MFMA
// multiplies them.
#include "ktx_common.h"
#include "../../include/ktx_seq.h"

#include <math.h>

#include <algorithm>

namespace {

#include "ktx_seq_dev.inc"

// ---------------------------------------------------------------------------------------------------------------------
// embedding + sinusoidal positions
template <typename WT>
__global__ void __launch_bounds__(256) embed_sinpos_kernel(int width, int vocab, const int32_t* __restrict__ tok,
                                                           const int32_t* __restrict__ pos, const WT* __restrict__ embed,
                                                           const double* __restrict__ inv_freq, float* __restrict__ x) {
  const int t = blockIdx.x;
  int id = tok[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  if (!inv_freq) {      // a plain table row (positions enter elsewhere)
    for (int e = threadIdx.x; e < width; e += 256) x[(size_t)t * width + e] = ld_elem(embed, (size_t)id * width + e);
    return;
  }
  const double p = (double)pos[t];
  for (int e = threadIdx.x; e < width; e += 256) {
    const double ang = p * inv_freq[e >> 1];
    const float s = (float)((e & 1) ? cos(ang) : sin(ang));
    x[(size_t)t * width + e] = ld_elem(embed, (size_t)id * width + e) + s;
  }
}

// ---------------------------------------------------------------------------------------------------------------------
// dense GEMM  Y = act(A W^T): 64 x 64 tile, BK = 32, 4 wavefronts of 32 x 32; any shape (edges zero-filled / masked).
template <typename AT, typename CT, typename YT>
__global__ void __launch_bounds__(256) dense_gemm_kernel(int M, int N, int K, const AT* __restrict__ A, int64_t lda,
                                                         const CT* __restrict__ W, YT* __restrict__ Y, int64_t ldy, int act,
                                                         int ksplit, bool vec_a, bool vec_w) {
  constexpr int LD = GemmTraits<CT>::LDS_LD;
  __shared__ __attribute__((aligned(16))) CT As[64 * LD];
  __shared__ __attribute__((aligned(16))) CT Ws[64 * LD];
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  const int l16 = lane & 15, lq = lane >> 4;
  v4f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
  // K range of this workgroup (split-K over blockIdx.z in whole 32-wide steps)
  const int ksteps = (K + 31) / 32;
  const int per = (ksteps + ksplit - 1) / ksplit;
  const int ks0 = blockIdx.z * per, ks1 = min(ksteps, ks0 + per);
  for (int ks = ks0; ks < ks1; ks++) {
    const int k0 = ks * 32;
    __syncthreads();
    gemm_stage<AT, CT>(As, A, lda, m0, M, k0, K, vec_a);
    gemm_stage<CT, CT>(Ws, W, (int64_t)K, n0, N, k0, K, vec_w);
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
        if (m < M && n < N) {
          float v = acc[i][j][r];
          if (ksplit > 1) {
            if constexpr (sizeof(YT) == 4) atomicAdd(reinterpret_cast<float*>(Y) + (size_t)m * ldy + n, v);
          } else {
            if (act == KTX_ACT_GELU_TANH) v = gelu_tanh_f32(v);
            st_elem(Y, (size_t)m * ldy + n, v);
          }
        }
      }
}

// ---------------------------------------------------------------------------------------------------------------------
// sigmoid attention: prep (q / k norms, temperature, cache append)
template <typename KT>
__global__ void __launch_bounds__(256) sigattn_prep_kernel(ktx_sigattn_config c, const float* __restrict__ proj, int64_t ldp,
                                                           int q_off, int k_off, const float* __restrict__ wq,
                                                           const float* __restrict__ wk, float eps, const int32_t* __restrict__ pos,
                                                           const int32_t* __restrict__ loc, KT* __restrict__ kcache,
                                                           float* __restrict__ kinv, float* __restrict__ q_out) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int H = c.heads, G = c.kv_heads, D = c.dim;
  const float* row = proj + (size_t)t * ldp;
  const int p = pos[t];
  float temp = 1.f;
  if (c.temp_coef != 0.f && c.temp_every > 0) temp = (float)(1.0 + (double)c.temp_coef * log((double)((p + 1) / c.temp_every) + 1.0));
  const float qmul = temp * c.scale;
  for (int u = wave; u < H + G; u += 4) {
    const bool is_q = u < H;
    const float* v = is_q ? row + q_off + (size_t)u * D : row + k_off + (size_t)(u - H) * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) ss += v[d] * v[d];
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)D + eps);
    if (is_q) {
      float* o = q_out + ((size_t)t * H + u) * D;
      for (int d = lane; d < D; d += 64) o[d] = v[d] * rinv * wq[d] * wk[d] * qmul;
    } else {
      const int g = u - H;
      const size_t r = (size_t)loc[t];
      KT* o = kcache + (r * G + g) * D;
      for (int d = lane; d < D; d += 64) st_elem(o, d, v[d]);
      if (lane == 0) kinv[r * G + g] = rinv;
    }
  }
}

// sigmoid attention, generic kernel: one query token x one key range per workgroup, fp32 on the vector ALUs.
// LDS: qs [H*D] | ks [KC][kst] | ps [H][KC] | wm [H][KC] | kv [KC]   (floats; kst = G*D | 1)
template <typename KT, typename OT, int NO>
__global__ void __launch_bounds__(256) sigattn_fwd_kernel(ktx_sigattn_config c, int T, int KC, const float* __restrict__ q,
                                                          const KT* __restrict__ kcache, const float* __restrict__ kinv,
                                                          const int32_t* __restrict__ tok_req, const int32_t* __restrict__ pos,
                                                          const int32_t* __restrict__ page_indptr,
                                                          const int32_t* __restrict__ page_indices, const float* __restrict__ pb,
                                                          const float* __restrict__ talk, float* __restrict__ partial,
                                                          OT* __restrict__ out) {
  extern __shared__ float lds[];
  const int H = c.heads, G = c.kv_heads, D = c.dim, rep = H / G, GD = G * D, HD = H * D;
  const int kst = GD | 1;
  float* qs = lds;
  float* ks = qs + HD;
  float* ps = ks + (size_t)KC * kst;
  float* wm = ps + H * KC;
  const int t = blockIdx.x, split = blockIdx.y, nsplit = gridDim.y, tid = threadIdx.x;
  const int p = pos[t], b = tok_req[t];
  const int nkeys = p + 1;
  int span = (nkeys + nsplit - 1) / nsplit;
  span = (span + KC - 1) / KC * KC;
  const int lo = split * span, hi = min(nkeys, lo + span);
  const int32_t* pages = page_indices + page_indptr[b];
  for (int e = tid; e < HD; e += 256) qs[e] = q[(size_t)t * HD + e];
  float acc[NO];
#pragma unroll
  for (int i = 0; i < NO; i++) acc[i] = 0.f;
  for (int j0 = lo; j0 < hi; j0 += KC) {
    const int nk = min(KC, hi - j0);
    __syncthreads();
    // stage nk key rows (all key heads) as fp32
    for (int e = tid; e < nk * GD; e += 256) {
      const int jj = e / GD, x = e - jj * GD;
      const int j = j0 + jj;
      const size_t r = (size_t)pages[j / c.page_size] * c.page_size + (j % c.page_size);
      ks[(size_t)jj * kst + x] = ld_elem(kcache, r * GD + x);
    }
    __syncthreads();
    // scores -> weights
    for (int e = tid; e < H * KC; e += 256) {
      const int h = e / KC, jj = e - h * KC;
      float w = 0.f;
      if (jj < nk) {
        const int g = h / rep, j = j0 + jj;
        const float* qh = qs + h * D;
        const float* kj = ks + (size_t)jj * kst + g * D;
        float s = 0.f;
        for (int d = 0; d < D; d++) s += qh[d] * kj[d];
        const size_t r = (size_t)pages[j / c.page_size] * c.page_size + (j % c.page_size);
        s *= kinv[r * G + g];
        if (c.slope_span != 0.f) s -= exp2f(-c.slope_span * (float)(h + 1) / (float)H) * (float)(p - j);
        w = sigmoid_f32(s + pb[h]);
      }
      ps[e] = w;
    }
    __syncthreads();
    // head mixing
    for (int e = tid; e < H * KC; e += 256) {
      const int h = e / KC, jj = e - h * KC;
      float w = 0.f;
      for (int g = 0; g < H; g++) w += talk[h * H + g] * ps[g * KC + jj];
      wm[e] = w;
    }
    __syncthreads();
    // weights x values (values = the staged key rows)
#pragma unroll
    for (int i = 0; i < NO; i++) {
      const int e = tid + i * 256;
      if (e < HD) {
        const int h = e / D, d = e - h * D, g = h / rep;
        const float* wr = wm + h * KC;
        const float* vc = ks + g * D + d;
        float a = acc[i];
        for (int jj = 0; jj < nk; jj++) a += wr[jj] * vc[(size_t)jj * kst];
        acc[i] = a;
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NO; i++) {
    const int e = tid + i * 256;
    if (e < HD) {
      if (nsplit > 1) partial[((size_t)split * T + t) * HD + e] = acc[i];
      else st_elem(out, (size_t)t * HD + e, acc[i]);
    }
  }
}

template <typename OT>
__global__ void __launch_bounds__(256) sigattn_reduce_kernel(int nsplit, size_t n, const float* __restrict__ partial,
                                                             OT* __restrict__ out) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= n) return;
  // eight loads in flight per round; the sum stays in range order (a0 + a1 + ...), whatever nsplit is
  float a = 0.f;
  int s = 0;
  for (; s + 8 <= nsplit; s += 8) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = partial[(size_t)(s + i) * n + e];
#pragma unroll
    for (int i = 0; i < 8; i++) a += v[i];
  }
  for (; s < nsplit; s++) a += partial[(size_t)s * n + e];
  st_elem(out, e, a);
}

// ---------------------------------------------------------------------------------------------------------------------
// mLSTM, part 1: the gates of a request's new tokens and the running maximum, off the sequential path.  Workgroup = (request, head).
//   z_i, z_f -> log gates i_t, f_t (soft cap, logsigmoid);  m_t = max(f_t + m_(t-1), i_t) is a scan of maps m -> max(m + L, Z), which
//   compose associatively ((L1, Z1) then (L2, Z2) = (L1 + L2, max(Z1 + L2, Z2))): 256 tokens per round, a wave scan on shuffles and
//   the four wave totals through LDS.  Written per token: a_t = exp(f_t + m_(t-1) - m_t), b_t = exp(i_t - m_t), e_t = exp(-m_t), and
//   the five terms the chunk kernel multiplies with; per (request, head) the maximum the call started from.
constexpr int KTX_MLSTM_GATE_FLOATS = 8;
__global__ void __launch_bounds__(256) mlstm_gates_kernel(ktx_mlstm_config c, const int32_t* __restrict__ q_indptr,
                                                          const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                          const float* __restrict__ proj, int64_t ldp, int i_off, int f_off,
                                                          const float* __restrict__ ib, const float* __restrict__ fb,
                                                          float* __restrict__ mg, float* __restrict__ gates,
                                                          float* __restrict__ minit) {
  __shared__ float wl[4], wz[4], mlast[256 + 1], lfs[256];
  __shared__ float m_carry;
  const int N = c.heads;
  const int b = blockIdx.x, hd = blockIdx.y, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int t0 = q_indptr[b], t1 = q_indptr[b + 1];
  if (t1 <= t0) return;
  const int sl = slot[b];
  if (tid == 0) {
    m_carry = pos0[b] == 0 ? 0.f : mg[(size_t)sl * N + hd];
    minit[(size_t)b * N + hd] = m_carry;
  }
  const float bi = ib[hd], bf = fb[hd], cap = c.gate_cap;
  for (int base = t0; base < t1; base += 256) {
    const int t = base + tid;
    const bool ok = t < t1;
    float L = 0.f, Z = -INFINITY, zi = 0.f;
    if (ok) {
      const float* row = proj + (size_t)t * ldp;
      zi = row[i_off + hd] + bi;
      float zf = row[f_off + hd] + bf;
      if (cap != 0.f) {
        zi = cap * tanhf(zi / cap);
        zf = cap * tanhf(zf / cap);
      }
      L = log_sigmoid_f32(zf);
      Z = zi;
    }
    const float lf = L;
    // inclusive scan inside the wavefront
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float pl = __shfl_up(L, d, 64), pz = __shfl_up(Z, d, 64);
      if (lane >= d) {
        Z = fmaxf(pz + L, Z);
        L = pl + L;
      }
    }
    __syncthreads();                        // (m_carry of the previous round has been read by everyone)
    if (lane == 63) {
      wl[wave] = L;
      wz[wave] = Z;
    }
    __syncthreads();
    float m_in = m_carry;
    for (int w = 0; w < wave; w++) m_in = fmaxf(m_in + wl[w], wz[w]);
    const float m = fmaxf(m_in + L, Z);
    mlast[tid + 1] = m;
    if (tid == 0) mlast[0] = m_carry;
    __syncthreads();
    if (ok) {
      const float m_prev = mlast[tid];
      float* g = gates + ((size_t)t * N + hd) * KTX_MLSTM_GATE_FLOATS;
      g[0] = expf(lf + m_prev - m);
      g[1] = expf(zi - m);
      g[2] = expf(-m);
    }
    // the terms of the 16-token chunk form (chunks are counted from the request's first new token; a round holds 16 whole chunks):
    // F = the chunk's summed log forget gates up to the token, m_0 = the maximum before the chunk, L = the chunk's last token
    lfs[tid] = ok ? lf : 0.f;
    __syncthreads();
    if (ok) {
      const int cb = tid & ~15, nvc = min(16, t1 - (base + cb));
      float F = 0.f, FL = 0.f;
      for (int r = 0; r < nvc; r++) {
        FL += lfs[cb + r];
        if (cb + r <= tid) F = FL;
      }
      const float m0c = mlast[cb], mL = mlast[cb + nvc];
      float* g = gates + ((size_t)t * N + hd) * KTX_MLSTM_GATE_FLOATS;
      g[3] = F - m;                          // row term of the in-chunk weights exp(F_t - F_s + i_s - m_t)
      g[4] = F - zi;                         // column term
      g[5] = expf(F + m0c - m);              // carry of the chunk's incoming state into this token
      g[6] = expf(FL - F + zi - mL);         // weight of this token in the chunk's outgoing state
      g[7] = expf(FL + m0c - mL);            // decay of the incoming state over the whole chunk
    }
    const int last = min(256, t1 - base) - 1;
    __syncthreads();
    if (tid == last) m_carry = m;
  }
  __syncthreads();
  if (tid == 0) mg[(size_t)sl * N + hd] = m_carry;
}

// mLSTM, part 2: the state recurrence.  Workgroup = (request, head, 64 value columns); wavefront w owns the rows d = w*DPG .. of the
// state slice, lane = value column; state slice and normaliser rows live in registers for the whole call.  Per token: the decay /
// input factors from part 1, k and q of the wavefront's rows (wave-uniform loads), S = a S + (b k) v, partial S^T q and n . q, ONE
// barrier, and the first wavefront adds the four partials and divides.
template <int DPG>
__global__ void __launch_bounds__(256) mlstm_fwd_kernel(ktx_mlstm_config c, const int32_t* __restrict__ q_indptr,
                                                        const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                        const float* __restrict__ proj, int64_t ldp, int q_off, int k_off,
                                                        int v_off, const float* __restrict__ gates, float* __restrict__ Sg,
                                                        float* __restrict__ ng, float* __restrict__ o_raw) {
  __shared__ float red[2][4][64];
  __shared__ float redn[2][4];
  __shared__ __attribute__((aligned(16))) float qk[2][2][4 * DPG];      // [half][q | k][rows, zero beyond dim]
  const int N = c.heads, D = c.dim, V = c.vdim;
  const int b = blockIdx.x, hd = blockIdx.y, vs = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int v = vs * 64 + lane;
  const bool vok = v < V;
  const int t0 = q_indptr[b], t1 = q_indptr[b + 1];
  if (t1 <= t0) return;
  const int sl = slot[b];
  const bool fresh = pos0[b] == 0;
  const int d0 = wave * DPG;
  float* Sp = Sg + ((size_t)sl * N + hd) * D * V;
  float* np_ = ng + ((size_t)sl * N + hd) * D;
  float S[DPG], nn[DPG];
#pragma unroll
  for (int i = 0; i < DPG; i++) {
    const int d = d0 + i;
    S[i] = (!fresh && d < D && vok) ? Sp[(size_t)d * V + v] : 0.f;
    nn[i] = (!fresh && d < D) ? np_[d] : 0.f;
  }
  for (int e = tid; e < 2 * 2 * 4 * DPG; e += 256) (&qk[0][0][0])[e] = 0.f;
  __syncthreads();
  const float qscale = 1.0f / sqrtf((float)D);
  // q and k of a token reach the wavefronts through LDS (one element per thread, broadcast reads); everything a token brings is
  // requested a step ahead: while token t is computed, token t+1's q / k go into the other LDS half and token t+2's are in flight
  float rq = 0.f, rk = 0.f, nv, na, nb, ne;
  {
    const float* row = proj + (size_t)t0 * ldp;
    const float* g = gates + ((size_t)t0 * N + hd) * KTX_MLSTM_GATE_FLOATS;
    if (tid < D) {
      qk[0][0][tid] = row[q_off + hd * D + tid] * qscale;
      qk[0][1][tid] = row[k_off + hd * D + tid];
    }
    nv = vok ? row[v_off + hd * V + v] : 0.f;
    na = g[0], nb = g[1], ne = g[2];
    if (t0 + 1 < t1 && tid < D) {
      const float* r1 = proj + (size_t)(t0 + 1) * ldp;
      rq = r1[q_off + hd * D + tid];
      rk = r1[k_off + hd * D + tid];
    }
  }
  __syncthreads();
  for (int t = t0; t < t1; t++) {
    const int buf = (t - t0) & 1;
    const float vv = nv, a = na, bb = nb, e = ne;
    if (tid < D) {
      qk[buf ^ 1][0][tid] = rq * qscale;
      qk[buf ^ 1][1][tid] = rk;
    }
    if (t + 1 < t1) {
      const float* row = proj + (size_t)(t + 1) * ldp;
      const float* g = gates + ((size_t)(t + 1) * N + hd) * KTX_MLSTM_GATE_FLOATS;
      nv = vok ? row[v_off + hd * V + v] : 0.f;
      na = g[0], nb = g[1], ne = g[2];
      if (t + 2 < t1 && tid < D) {
        const float* r2 = proj + (size_t)(t + 2) * ldp;
        rq = r2[q_off + hd * D + tid];
        rk = r2[k_off + hd * D + tid];
      }
    }
    float po = 0.f, pn = 0.f;
    const float* qb = &qk[buf][0][d0];
    const float* kb = &qk[buf][1][d0];
#pragma unroll
    for (int i = 0; i < DPG; i++) {
      const float bk = bb * kb[i], qd = qb[i];
      S[i] = a * S[i] + bk * vv;
      nn[i] = a * nn[i] + bk;
      po += S[i] * qd;
      pn += nn[i] * qd;
    }
    red[buf][wave][lane] = po;
    if (lane == 0) redn[buf][wave] = pn;
    __syncthreads();
    if (wave == 0 && vok) {
      const float num = ((red[buf][0][lane] + red[buf][1][lane]) + red[buf][2][lane]) + red[buf][3][lane];
      const float nqd = ((redn[buf][0] + redn[buf][1]) + redn[buf][2]) + redn[buf][3];
      o_raw[(size_t)t * N * V + hd * V + v] = num / (fmaxf(fabsf(nqd), e) + c.denom_eps);
    }
    // (the next token writes the other halves of `red` and `qk`; these halves are rewritten only behind the next barrier)
  }
#pragma unroll
  for (int i = 0; i < DPG; i++) {
    const int d = d0 + i;
    if (d < D) {
      if (vok) Sp[(size_t)d * V + v] = S[i];
      if (vs == 0 && lane == 0) np_[d] = nn[i];
    }
  }
}

// mLSTM, part 2 for prompts: the same recurrence 16 tokens at a time on the matrix cores (fp32 MFMA: state, gates and products stay
// fp32).  With F_t the sum of the chunk's log forget gates up to t and m_0 the maximum the chunk starts from, unrolling the recurrence
// over a chunk gives
//   S_t^T q_t = exp(F_t + m_0 - m_t) S_0^T q_t + sum_{s <= t} exp(F_t - F_s + i_s - m_t) (k_s . q_t) v_s        (n_t . q_t alike, without v)
//   S_L       = exp(F_L + m_0 - m_L) S_0 + sum_s exp(F_L - F_s + i_s - m_L) k_s v_s^T
// — every exponent is <= 0 because m is the running maximum of exactly these sums.  Workgroup = (request, head, 64 value columns), the
// state slice [dim, 64] lives in LDS for the whole call; wavefront w owns 16 columns: A = Q K^T (16 x 16), W = A o weights (lower
// triangle), O = c o (Q S_0) + W V, then its columns of S_L = decay S_0 + (u o K)^T V.  Only the staging of a chunk is shared.
constexpr int ML_CL = 16;
__global__ void __launch_bounds__(256) mlstm_chunk_kernel(ktx_mlstm_config c, const int32_t* __restrict__ q_indptr,
                                                          const int32_t* __restrict__ pos0, const int32_t* __restrict__ slot,
                                                          const float* __restrict__ proj, int64_t ldp, int q_off, int k_off,
                                                          int v_off, const float* __restrict__ gates, const float* __restrict__ minit,
                                                          float* __restrict__ Sg, float* __restrict__ ng, float* __restrict__ o_raw) {
  extern __shared__ __attribute__((aligned(16))) float cl[];
  const int N = c.heads, D = c.dim, V = c.vdim;
  const int Dp = (D + 15) & ~15, QST = Dp + 4;
  float* Ss = cl;                           // [Dp][64]
  float* Qs = Ss + (size_t)Dp * 64;         // [16][QST]
  float* Ks = Qs + ML_CL * QST;             // [16][QST]
  float* Vs = Ks + ML_CL * QST;             // [16][64]
  float* Ws = Vs + ML_CL * 64;              // [4][16][17]
  float* ns = Ws + 4 * 16 * 17;             // [2][Dp]
  float* gl = ns + 2 * Dp;                  // (48 unused) | rt[16] ct[16] cc[16] ee[16] us[16] | decay
  float* qn = gl + 8 * 16 + 2;              // [4][16]
  const int b = blockIdx.x, hd = blockIdx.y, vs = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int t0 = q_indptr[b], t1 = q_indptr[b + 1];
  if (t1 <= t0) return;
  const int sl = slot[b];
  const bool fresh = pos0[b] == 0;
  float* Sp = Sg + ((size_t)sl * N + hd) * D * V;
  float* np_ = ng + ((size_t)sl * N + hd) * D;
  for (int e = tid; e < Dp * 64; e += 256) {
    const int d = e >> 6, col = e & 63, v = vs * 64 + col;
    Ss[e] = (!fresh && d < D && v < V) ? Sp[(size_t)d * V + v] : 0.f;
  }
  for (int d = tid; d < Dp; d += 256) ns[d] = (!fresh && d < D) ? np_[d] : 0.f;
  const float qscale = 1.0f / sqrtf((float)D);
  const int vcol = 16 * wave + l16, v = vs * 64 + vcol;
  const bool vok = v < V;
  float* Ww = Ws + wave * 16 * 17;
  float* qnw = qn + wave * 16;
  // a chunk's q / k / v / gate records are requested one chunk ahead and wait in registers
  constexpr int ML_PF = 16;                   // 256 threads x 16 cover the 16 x Dp (Dp <= 256) elements of q and of k
  float rq[ML_PF], rk[ML_PF], rv[4], rg[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  auto fetch = [&](int c0) {
    const int nv = min(ML_CL, t1 - c0);
#pragma unroll
    for (int i = 0; i < ML_PF; i++) {
      const int e = tid + i * 256;
      const int t = e / Dp, d = e - t * Dp;
      const bool ok = e < ML_CL * Dp && t < nv && d < D;
      const float* row = proj + (size_t)(c0 + (ok ? t : 0)) * ldp;
      rq[i] = ok ? row[q_off + hd * D + d] : 0.f;
      rk[i] = ok ? row[k_off + hd * D + d] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int e = tid + i * 256;
      const int t = e >> 6, vv = vs * 64 + (e & 63);
      rv[i] = (t < nv && vv < V) ? proj[(size_t)(c0 + t) * ldp + v_off + hd * V + vv] : 0.f;
    }
    if (tid < ML_CL) {
      const bool okt = tid < nv;
      const float* g = gates + ((size_t)(c0 + (okt ? tid : 0)) * N + hd) * KTX_MLSTM_GATE_FLOATS;
      rg[0] = okt ? g[3] : 0.f;
      rg[1] = okt ? g[4] : 0.f;
      rg[2] = okt ? g[5] : 0.f;
      rg[3] = okt ? g[2] : 1.f;
      rg[4] = okt ? g[6] : 0.f;
      rg[5] = nv > 0 ? g[7] : 1.f;          // (token 0 of the chunk carries the chunk's decay like every other)
    }
  };
  fetch(t0);
  int par = 0;
  for (int c0 = t0; c0 < t1; c0 += ML_CL, par ^= 1) {
    const int nv = min(ML_CL, t1 - c0);
    float* n_cur = ns + par * Dp;
    float* n_nxt = ns + (par ^ 1) * Dp;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ML_PF; i++) {
      const int e = tid + i * 256;
      if (e < ML_CL * Dp) {
        const int t = e / Dp, d = e - t * Dp;
        Qs[t * QST + d] = rq[i] * qscale;
        Ks[t * QST + d] = rk[i];
      }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) Vs[tid + i * 256] = rv[i];
    if (tid < ML_CL) {
      gl[48 + tid] = rg[0];                  // row term
      gl[64 + tid] = rg[1];                  // column term
      gl[80 + tid] = rg[2];                  // carry of the incoming state into token t
      gl[96 + tid] = rg[3];                  // exp(-m_t)
      gl[112 + tid] = rg[4];                 // weight of token s in the outgoing state
      if (tid == 0) gl[128] = rg[5];
    }
    if (c0 + ML_CL < t1) fetch(c0 + ML_CL);
    __syncthreads();
    const float decay = gl[128];
    // (i) A = Q K^T, (ii) weights, row sums, relayout through the wavefront's LDS tile
    v4f A = {0.f, 0.f, 0.f, 0.f};
    {
      // four independent accumulators (Dp is a multiple of 16): the products of one chain wait on each other otherwise
      v4f a1 = A, a2 = A, a3 = A;
      const float* qr = Qs + l16 * QST + lq;
      const float* kr = Ks + l16 * QST + lq;
#pragma unroll 2
      for (int k = 0; k < Dp; k += 16) {
        A = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k], kr[k], A, 0, 0, 0);
        a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k + 4], kr[k + 4], a1, 0, 0, 0);
        a2 = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k + 8], kr[k + 8], a2, 0, 0, 0);
        a3 = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k + 12], kr[k + 12], a3, 0, 0, 0);
      }
      A = (A + a1) + (a2 + a3);
    }
    float rsum[4];
    {
      const float ctm = gl[64 + l16];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const int t = lq * 4 + r;
        float w = 0.f;
        if (l16 <= t && t < nv) w = A[r] * expf(gl[48 + t] - ctm);
        Ww[t * 17 + l16] = w;
        rsum[r] = w;
      }
      row16_sum4(rsum[0], rsum[1], rsum[2], rsum[3]);
    }
    // (iii) q_t . n_0 for the 16 tokens
    {
      float pq = 0.f;
#pragma unroll 8
      for (int k = lq; k < Dp; k += 4) pq += Qs[l16 * QST + k] * n_cur[k];
      pq += __shfl_xor(pq, 16, 64);
      pq += __shfl_xor(pq, 32, 64);
      if (lq == 0) qnw[l16] = pq;
    }
    // (iv) O = carry o (Q S_0) + W V  -> outputs
    v4f O = {0.f, 0.f, 0.f, 0.f};
    {
      v4f o1 = O, o2 = O, o3 = O;
      const float* qr = Qs + l16 * QST + lq;
      const float* sr = Ss + lq * 64 + vcol;
#pragma unroll 2
      for (int k = 0; k < Dp; k += 16) {
        O = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k], sr[k * 64], O, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k + 4], sr[(k + 4) * 64], o1, 0, 0, 0);
        o2 = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k + 8], sr[(k + 8) * 64], o2, 0, 0, 0);
        o3 = __builtin_amdgcn_mfma_f32_16x16x4f32(qr[k + 12], sr[(k + 12) * 64], o3, 0, 0, 0);
      }
      O = (O + o1) + (o2 + o3);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) O[r] *= gl[80 + lq * 4 + r];
#pragma unroll
    for (int k = 0; k < ML_CL; k += 4) O = __builtin_amdgcn_mfma_f32_16x16x4f32(Ww[l16 * 17 + k + lq], Vs[(k + lq) * 64 + vcol], O, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int t = lq * 4 + r;
      if (t < nv && vok) {
        const float nq = gl[80 + t] * qnw[t] + rsum[r];
        o_raw[(size_t)(c0 + t) * N * V + hd * V + v] = O[r] / (fmaxf(fabsf(nq), gl[96 + t]) + c.denom_eps);
      }
    }
    // (v) this wavefront's 16 columns of the outgoing state
#pragma unroll 2
    for (int dt = 0; dt < Dp; dt += 16) {
      v4f C;
#pragma unroll
      for (int r = 0; r < 4; r++) C[r] = decay * Ss[(dt + lq * 4 + r) * 64 + vcol];
#pragma unroll
      for (int k = 0; k < ML_CL; k += 4)
        C = __builtin_amdgcn_mfma_f32_16x16x4f32(Ks[(k + lq) * QST + dt + l16] * gl[112 + k + lq], Vs[(k + lq) * 64 + vcol], C, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < 4; r++) Ss[(dt + lq * 4 + r) * 64 + vcol] = C[r];
    }
    // (vi) the normaliser (into the other half: every wavefront may still be reading this chunk's)
    for (int d = tid; d < Dp; d += 256) {
      float a = decay * n_cur[d];
      for (int s2 = 0; s2 < nv; s2++) a += gl[112 + s2] * Ks[s2 * QST + d];
      n_nxt[d] = a;
    }
  }
  __syncthreads();
  for (int e = tid; e < Dp * 64; e += 256) {
    const int d = e >> 6, col = e & 63, vv = vs * 64 + col;
    if (d < D && vv < V) Sp[(size_t)d * V + vv] = Ss[e];
  }
  if (vs == 0)
    for (int d = tid; d < D; d += 256) np_[d] = ns[par * Dp + d];
}

size_t mlstm_chunk_lds(int D) {
  const size_t Dp = (D + 15) & ~15;
  return (Dp * 64 + 2 * ML_CL * (Dp + 4) + ML_CL * 64 + 4 * 16 * 17 + 2 * Dp + 8 * 16 + 2 + 4 * 16) * sizeof(float);
}

template <typename OT>
__global__ void __launch_bounds__(256) mlstm_gate_norm_kernel(ktx_mlstm_config c, int T, const float* __restrict__ o_raw,
                                                              const float* __restrict__ proj, int64_t ldp, int g_off,
                                                              const float* __restrict__ w, OT* __restrict__ out) {
  const int N = c.heads, V = c.vdim;
  const int unit = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (unit >= T * N) return;
  const int t = unit / N, hd = unit - t * N;
  const float* o = o_raw + (size_t)t * N * V + hd * V;
  float ss = 0.f;
  for (int v = lane; v < V; v += 64) ss += o[v] * o[v];
  ss = wave_sum(ss);
  const float rinv = 1.0f / sqrtf(ss / (float)V + c.eps);
  const float* g = proj + (size_t)t * ldp + g_off + hd * V;
  for (int v = lane; v < V; v += 64) st_elem(out, (size_t)t * N * V + hd * V + v, o[v] * rinv * w[hd * V + v] * sigmoid_f32(g[v]));
}

// ---------------------------------------------------------------------------------------------------------------------
// decode-sized GEMM (M <= 8 rows): Y[m][n] = act(sum_k A[m][k] W[n][k]).  Bandwidth-bound on W: the activation rows sit in LDS in the
// product's type, a wavefront owns RPW weight rows and streams them with 16-byte loads, fp32 accumulation, one wave reduction per row.
template <typename AT, typename CT, typename YT, int MM>
__global__ void __launch_bounds__(256) dense_gemv_kernel(int M, int N, int K, const AT* __restrict__ A, int64_t lda,
                                                         const CT* __restrict__ W, YT* __restrict__ Y, int64_t ldy, int act, bool vec) {
  extern __shared__ __attribute__((aligned(16))) unsigned char gv_lds[];
  CT* As = reinterpret_cast<CT*>(gv_lds);                 // [MM][Kp], Kp = K rounded up to 8
  const int Kp = (K + 7) & ~7;
  for (int e = threadIdx.x; e < MM * Kp; e += 256) {
    const int m = e / Kp, k = e - m * Kp;
    const float v = (m < M && k < K) ? ld_elem(A, (size_t)m * lda + k) : 0.f;
    if constexpr (sizeof(CT) == 2) As[e] = to_bf16_rne(v);
    else As[e] = v;
  }
  __syncthreads();
  constexpr int RPW = 2;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
#pragma unroll
  for (int rr = 0; rr < RPW; rr++) {
    const int n = (blockIdx.x * 4 + wave) * RPW + rr;
    if (n >= N) break;
    const CT* wrow = W + (size_t)n * K;
    float acc[MM];
#pragma unroll
    for (int m = 0; m < MM; m++) acc[m] = 0.f;
    for (int k = lane * 8; k < Kp; k += 512) {
      float wv[8];
      if (vec) {
        if constexpr (sizeof(CT) == 2) {
          const uint4 u = *reinterpret_cast<const uint4*>(wrow + k);
          wv[0] = ktx_lo_f32(u.x); wv[1] = ktx_hi_f32(u.x); wv[2] = ktx_lo_f32(u.y); wv[3] = ktx_hi_f32(u.y);
          wv[4] = ktx_lo_f32(u.z); wv[5] = ktx_hi_f32(u.z); wv[6] = ktx_lo_f32(u.w); wv[7] = ktx_hi_f32(u.w);
        } else {
          const float4 a = *reinterpret_cast<const float4*>(wrow + k), b = *reinterpret_cast<const float4*>(wrow + k + 4);
          wv[0] = a.x; wv[1] = a.y; wv[2] = a.z; wv[3] = a.w; wv[4] = b.x; wv[5] = b.y; wv[6] = b.z; wv[7] = b.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) wv[i] = (k + i < K) ? ld_elem(wrow, (size_t)(k + i)) : 0.f;
      }
#pragma unroll
      for (int m = 0; m < MM; m++) {
        const CT* ar = As + m * Kp + k;
        float a = acc[m];
#pragma unroll
        for (int i = 0; i < 8; i++) a = fmaf(wv[i], ld_elem(ar, (size_t)i), a);
        acc[m] = a;
      }
    }
#pragma unroll
    for (int m = 0; m < MM; m++) {
      float a = wave_sum(acc[m]);
      if (lane == 0 && m < M) {
        if (act == KTX_ACT_GELU_TANH) a = gelu_tanh_f32(a);
        st_elem(Y, (size_t)m * ldy + n, a);
      }
    }
  }
}

// decode-sized GEMM on the matrix cores (M <= 16, bf16 weights, K % 32 == 0): workgroup = 16 weight rows, its four wavefronts take a
// quarter of K each; a lane streams ITS weight row's 16-byte pieces straight from memory into the B operand (no LDS on the weight
// path), the activation rows (few, L2-resident) fill the A operand; partial tiles meet in LDS.
// GLU: W's rows alternate gate_f, up_f (N = 2F); neighbouring lanes hold a pair's two products and the even one writes
// Y[m][f] = g sigmoid(slope g) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit).
template <typename AT, typename YT, bool GLU>
__global__ void __launch_bounds__(256) dense_gemv_mfma_kernel(int M, int N, int K, const AT* __restrict__ A, int64_t lda,
                                                              const bf16_t* __restrict__ W, YT* __restrict__ Y, int64_t ldy, int act,
                                                              float limit, float slope, float shift) {
  __shared__ float red[4][64][4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
  const int n = blockIdx.x * 16 + l16;
  const int steps = K / 32, per = (steps + 3) / 4;
  const int s0 = wave * per, s1 = min(steps, s0 + per);
  const bf16_t* wrow = W + (size_t)min(n, N - 1) * K + lq * 8;
  const AT* arow = A + (size_t)min(l16, M - 1) * lda + lq * 8;
  const bool aok = l16 < M, wok = n < N;
  v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int st = s0; st < s1; st++) {
    const int k = st * 32;
    uint4 wv = *reinterpret_cast<const uint4*>(wrow + k);
    uint4 av;
    if constexpr (sizeof(AT) == 4) {
      const float4 a0 = *reinterpret_cast<const float4*>(arow + k), a1 = *reinterpret_cast<const float4*>(arow + k + 4);
      av.x = ktx_pk_bf16(a0.x, a0.y); av.y = ktx_pk_bf16(a0.z, a0.w); av.z = ktx_pk_bf16(a1.x, a1.y); av.w = ktx_pk_bf16(a1.z, a1.w);
    } else {
      av = *reinterpret_cast<const uint4*>(arow + k);
    }
    if (!aok) av = uint4{0u, 0u, 0u, 0u};
    if (!wok) wv = uint4{0u, 0u, 0u, 0u};
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sq_v8bf, av), __builtin_bit_cast(sq_v8bf, wv), acc, 0, 0, 0);
  }
#pragma unroll
  for (int r = 0; r < 4; r++) red[wave][lane][r] = acc[r];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int m = lq * 4 + r;
      float v = ((red[0][lane][r] + red[1][lane][r]) + red[2][lane][r]) + red[3][lane][r];
      if constexpr (GLU) {
        const float other = __shfl_xor(v, 1);      // (N is even: a pair is inside or outside together)
        if (wok && m < M && (l16 & 1) == 0) {
          const float g = fminf(v, limit), u = fminf(fmaxf(other, -limit), limit);
          st_elem(Y, (size_t)m * ldy + (n >> 1), g * sigmoid_f32(slope * g) * (u + shift));
        }
      } else if (wok && m < M) {
        if (act == KTX_ACT_GELU_TANH) v = gelu_tanh_f32(v);
        st_elem(Y, (size_t)m * ldy + n, v);
      }
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256) gelu_tanh_kernel(size_t n, T* __restrict__ y) {
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e < n) st_elem(y, e, gelu_tanh_f32(ld_elem(y, e)));
}

// ---------------------------------------------------------------------------------------------------------------------
// sigmoid attention on the matrix cores (prompts AND decode steps).  Workgroup = 16 consecutive query rows of one request x ALL
// heads (the head mixing needs every head's weight of a (query, key) pair in one place) x one range of the keys; wavefront w owns the
// NHW consecutive heads w*NHW .. (with grouped queries they share their key head, so its fragments are loaded once).
// Per tile of 32 keys:  S_g = Q_g K^T (bf16 MFMA, Q fragments resident in registers) -> fp32 weights sigmoid(S kinv_j - slope (i - j)
// + bias) into LDS -> every wavefront mixes its own heads' weights from all heads' (fp32 FMAs) -> bf16 -> O_h += W_h V (bf16 MFMA; the
// values are the key rows, read from the same LDS tile column-wise).  Weights are not normalised over keys, so the key ranges of a
// row (gridDim.z of them) are plain partial sums: fp32 partials + ktx's reduce kernel when gridDim.z > 1.
constexpr int SA_KN = 32;      // keys per tile
constexpr int SA_PST = 33;     // row stride of the fp32 weight tiles (words)
constexpr int SA_WST = 40;     // row stride of the bf16 mixed-weight tiles (elements)

template <int NHW, int DS>
__global__ void __launch_bounds__(256) sigattn_mfma_kernel(ktx_sigattn_config c, int T, const float* __restrict__ q,
                                                           const bf16_t* __restrict__ kcache, const float* __restrict__ kinv,
                                                           const int32_t* __restrict__ q_indptr, const int32_t* __restrict__ pos0,
                                                           const int32_t* __restrict__ page_indptr,
                                                           const int32_t* __restrict__ page_indices, const float* __restrict__ pb,
                                                           const float* __restrict__ talk, float* __restrict__ partial,
                                                           bf16_t* __restrict__ out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char sa_lds[];
  constexpr int D = DS * 32;
  const int H = c.heads, G = c.kv_heads, rep = H / G, GD = G * D, HD = H * D;
  const int KST = GD + 8;
  bf16_t* ks = reinterpret_cast<bf16_t*>(sa_lds);                       // [32][KST]
  float* ps = reinterpret_cast<float*>(ks + SA_KN * KST);                // [H][16][33] weights (fp32) ...
  bf16_t* wm = reinterpret_cast<bf16_t*>(ps);                            // ... and, once every wavefront has mixed, [H][16][40] bf16
  float* kis = ps + (size_t)H * 16 * SA_PST;                             // [32][G]
  float* tks = kis + SA_KN * G;                                          // [H][H]
  const int b = blockIdx.y, tile = gridDim.x - 1 - blockIdx.x;            // long rows first
  const int split = blockIdx.z, nsplit = gridDim.z;
  const int qb = q_indptr[b], qe = q_indptr[b + 1];
  const int row0 = qb + tile * 16;
  if (row0 >= qe) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, l16 = lane & 15, lq = lane >> 4;
  const int nrows = min(16, qe - row0);
  const int p0 = pos0[b] + tile * 16;                 // position of row 0 of the tile
  const int p_last = p0 + nrows - 1;
  // this workgroup's key range, in whole tiles
  const int ntiles = p_last / SA_KN + 1;
  const int per = (ntiles + nsplit - 1) / nsplit;
  const int jt0 = split * per, jt1 = min(ntiles, jt0 + per);
  const int32_t* pages = page_indices + page_indptr[b];
  for (int e = tid; e < H * H; e += 256) tks[e] = talk[e];
  const int h0 = wave * NHW;
  // Q fragments (A operand: row = l16, k = ds*32 + lq*8 ..)
  sq_v8bf qf[NHW][DS];
#pragma unroll
  for (int u = 0; u < NHW; u++) {
    const int g = h0 + u;
#pragma unroll
    for (int ds = 0; ds < DS; ds++) {
      uint4 pk = {0u, 0u, 0u, 0u};
      if (g < H && l16 < nrows && jt0 < jt1) {
        const float* src = q + (size_t)(row0 + l16) * HD + g * D + ds * 32 + lq * 8;
        const float4 a = *reinterpret_cast<const float4*>(src), bq = *reinterpret_cast<const float4*>(src + 4);
        pk.x = ktx_pk_bf16(a.x, a.y); pk.y = ktx_pk_bf16(a.z, a.w); pk.z = ktx_pk_bf16(bq.x, bq.y); pk.w = ktx_pk_bf16(bq.z, bq.w);
      }
      qf[u][ds] = __builtin_bit_cast(sq_v8bf, pk);
    }
  }
  v4f o[NHW][DS * 2];
#pragma unroll
  for (int u = 0; u < NHW; u++)
#pragma unroll
    for (int dn = 0; dn < DS * 2; dn++) o[u][dn] = (v4f){0.f, 0.f, 0.f, 0.f};
  float slope[NHW], bias[NHW];
#pragma unroll
  for (int u = 0; u < NHW; u++) {
    const int g = h0 + u;
    slope[u] = (g < H && c.slope_span != 0.f) ? exp2f(-c.slope_span * (float)(g + 1) / (float)H) : 0.f;
    bias[u] = g < H ? pb[g] : 0.f;
  }
  // all heads of this wavefront on one key head?  (wave-uniform)
  const bool shared_kv = (h0 / rep) == ((min(h0 + NHW, H) - 1) / rep);
  // staging: 8 threads per key row, 16-byte pieces 64 elements apart; a tile's rows are requested one tile ahead and wait in
  // registers (SA_PF pieces of 16 bytes per thread cover key rows of up to 64 * SA_PF elements; longer rows are loaded in place)
  constexpr int SA_PF = 8;
  const int sj = tid >> 3, sx = (tid & 7) * 8;
  uint4 pf[SA_PF];
  float pf_ki = 0.f;
  auto row_of = [&](int jt) -> long {      // cache row of this thread's key of tile jt, -1 when the key does not exist
    const int j = jt * SA_KN + sj;
    if (jt >= jt1 || j > p_last) return -1;
    return (long)pages[j / c.page_size] * c.page_size + (j % c.page_size);
  };
  long row_next = row_of(jt0), row_cur = -1;    // the page lookup runs one tile ahead of the row loads, which run one tile ahead of use
  auto request = [&](int jt) {
    row_cur = row_next;
    row_next = row_of(jt + 1);
    const bool ok = row_cur >= 0;
    const size_t r = ok ? (size_t)row_cur : 0;
    const bf16_t* src = kcache + r * GD;
#pragma unroll
    for (int u = 0; u < SA_PF; u++) {
      const int x = sx + u * 64;
      pf[u] = (ok && x < GD) ? *reinterpret_cast<const uint4*>(src + x) : uint4{0u, 0u, 0u, 0u};
    }
    const int g = tid & 7;                 // thread g of a row's eight fetches 1 / rms of key head g (+8, +16 ... in place below)
    pf_ki = (ok && g < G) ? kinv[r * G + g] : 0.f;
  };
  request(jt0);
  for (int jt = jt0; jt < jt1; jt++) {
    const int j0 = jt * SA_KN;
    __syncthreads();
    {
#pragma unroll
      for (int u = 0; u < SA_PF; u++) {
        const int x = sx + u * 64;
        if (x < GD) *reinterpret_cast<uint4*>(ks + sj * KST + x) = pf[u];
      }
      if ((tid & 7) < G) kis[sj * G + (tid & 7)] = pf_ki;
      if (GD > 64 * SA_PF || G > 8) {       // the part of wide rows the registers do not hold
        const int j = j0 + sj;
        const bool ok = j <= p_last;
        const size_t r = ok ? (size_t)pages[j / c.page_size] * c.page_size + (j % c.page_size) : 0;
        for (int x = sx + 64 * SA_PF; x < GD; x += 64)
          *reinterpret_cast<uint4*>(ks + sj * KST + x) = ok ? *reinterpret_cast<const uint4*>(kcache + r * GD + x) : uint4{0u, 0u, 0u, 0u};
        for (int g = 8 + (tid & 7); g < G; g += 8) kis[sj * G + g] = ok ? kinv[r * G + g] : 0.f;
      }
    }
    request(jt + 1);
    __syncthreads();
    // scores -> weights (fp32) of this wavefront's heads
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
      sq_v8bf kf[DS];
      int kg_have = -1;
#pragma unroll
      for (int u = 0; u < NHW; u++) {
        const int g = h0 + u;
        if (g < H) {
          const int kg = g / rep;
          if (kg != kg_have) {
#pragma unroll
            for (int ds = 0; ds < DS; ds++)
              kf[ds] = *reinterpret_cast<const sq_v8bf*>(ks + (nt * 16 + l16) * KST + kg * D + ds * 32 + lq * 8);
            kg_have = kg;
          }
          v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ds = 0; ds < DS; ds++) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[u][ds], kf[ds], acc, 0, 0, 0);
          const int jj = nt * 16 + l16, j = j0 + jj;
          const float ki = kis[jj * G + kg];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const int i = lq * 4 + r, pi = p0 + i;
            float w = 0.f;
            if (i < nrows && j <= pi) w = sigmoid_fast(acc[r] * ki - slope[u] * (float)(pi - j) + bias[u]);
            ps[(g * 16 + i) * SA_PST + jj] = w;
          }
        }
      }
    }
    __syncthreads();
    // head mixing (fp32) into registers; when every wavefront has read the fp32 tiles, the bf16 results take their place.
    // A decode step's tile has one row: its wavefronts mix two weights per lane instead of eight.
    {
      float wacc[NHW][8];
#pragma unroll
      for (int u = 0; u < NHW; u++)
#pragma unroll
        for (int x = 0; x < 8; x++) wacc[u][x] = 0.f;
      if (nrows == 1) {
        if (lq == 0) {
          for (int g = 0; g < H; g++) {
            const float pv0 = ps[(g * 16) * SA_PST + l16], pv1 = ps[(g * 16) * SA_PST + 16 + l16];
#pragma unroll
            for (int u = 0; u < NHW; u++) {
              const int h = h0 + u;
              const float tk = h < H ? tks[h * H + g] : 0.f;
              wacc[u][0] = fmaf(tk, pv0, wacc[u][0]);
              wacc[u][4] = fmaf(tk, pv1, wacc[u][4]);
            }
          }
        }
      } else if (lq * 4 < nrows) {
        for (int g = 0; g < H; g++) {
          float pv[8];
#pragma unroll
          for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int r = 0; r < 4; r++) pv[nt * 4 + r] = ps[(g * 16 + lq * 4 + r) * SA_PST + nt * 16 + l16];
#pragma unroll
          for (int u = 0; u < NHW; u++) {
            const int h = h0 + u;
            const float tk = h < H ? tks[h * H + g] : 0.f;
#pragma unroll
            for (int x = 0; x < 8; x++) wacc[u][x] = fmaf(tk, pv[x], wacc[u][x]);
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < NHW; u++) {
        const int h = h0 + u;
        if (h < H) {
#pragma unroll
          for (int nt = 0; nt < 2; nt++)
#pragma unroll
            for (int r = 0; r < 4; r++) wm[(h * 16 + lq * 4 + r) * SA_WST + nt * 16 + l16] = to_bf16_rne(wacc[u][nt * 4 + r]);
        }
      }
    }
    __syncthreads();
    // O_h += W_h V: B operand = V[k = key lq*8 .. +8][n = d]: eight 2-byte reads down a column of the key tile
#pragma unroll
    for (int dn = 0; dn < DS * 2; dn++) {
      sq_v8bf vf;
      int kg_have = -1;
#pragma unroll
      for (int u = 0; u < NHW; u++) {
        const int h = h0 + u;
        if (h < H) {
          const int kg = shared_kv ? h0 / rep : h / rep;
          if (kg != kg_have) {
            const bf16_t* col = ks + (size_t)(lq * 8) * KST + kg * D + dn * 16 + l16;
            uint4 pk;
            pk.x = (uint32_t)col[0] | ((uint32_t)col[KST] << 16);
            pk.y = (uint32_t)col[2 * KST] | ((uint32_t)col[3 * KST] << 16);
            pk.z = (uint32_t)col[4 * KST] | ((uint32_t)col[5 * KST] << 16);
            pk.w = (uint32_t)col[6 * KST] | ((uint32_t)col[7 * KST] << 16);
            vf = __builtin_bit_cast(sq_v8bf, pk);
            kg_have = kg;
          }
          const sq_v8bf wf = *reinterpret_cast<const sq_v8bf*>(wm + (h * 16 + l16) * SA_WST + lq * 8);
          o[u][dn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, vf, o[u][dn], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < NHW; u++) {
    const int h = h0 + u;
    if (h < H) {
#pragma unroll
      for (int dn = 0; dn < DS * 2; dn++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int i = lq * 4 + r;
          if (i < nrows) {
            const size_t e = (size_t)(row0 + i) * HD + h * D + dn * 16 + l16;
            if (nsplit > 1) partial[(size_t)split * T * HD + e] = o[u][dn][r];
            else out[e] = to_bf16_rne(o[u][dn][r]);
          }
        }
    }
  }
}

size_t sigattn_mfma_lds(const ktx_sigattn_config& c) {
  const size_t GD = (size_t)c.kv_heads * c.dim, H = c.heads;
  return SA_KN * (GD + 8) * 2 + H * 16 * SA_PST * 4 + SA_KN * c.kv_heads * 4 + H * H * 4;      // (the bf16 tiles reuse the fp32 ones)
}

// ---------------------------------------------------------------------------------------------------------------------
// fp32 norm glue (see the header); one workgroup per row, the row is re-read instead of staged
template <typename OT>
__global__ void __launch_bounds__(256) rms_combine_kernel(int W, const float* __restrict__ y1, const float* __restrict__ w1,
                                                          const float* __restrict__ y2, const float* __restrict__ w2,
                                                          const float* __restrict__ wn, int one_plus, float eps,
                                                          float* __restrict__ xres, const int32_t* __restrict__ rows,
                                                          OT* __restrict__ out) {
  __shared__ float red[4];
  constexpr int RMAX = 16;                  // rows up to 256 * 16 elements stay in registers; longer ones are re-read
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* a = y1 + (size_t)(rows ? rows[t] : t) * W;
  const float* b = y2 ? y2 + (size_t)t * W : nullptr;
  const bool in_regs = W <= 256 * RMAX;
  float za[RMAX], zb[RMAX];
  float r1 = 1.f, r2 = 1.f;
  if (in_regs) {
#pragma unroll
    for (int i = 0; i < RMAX; i++) {
      const int e = tid + i * 256;
      za[i] = e < W ? a[e] : 0.f;
      zb[i] = (b && e < W) ? b[e] : 0.f;
    }
  }
  if (b) {
    float s1 = 0.f, s2 = 0.f;
    if (in_regs) {
#pragma unroll
      for (int i = 0; i < RMAX; i++) {
        s1 += za[i] * za[i];
        s2 += zb[i] * zb[i];
      }
    } else {
      for (int e = tid; e < W; e += 256) {
        s1 += a[e] * a[e];
        s2 += b[e] * b[e];
      }
    }
    s1 = block_sum256(s1, red);
    s2 = block_sum256(s2, red);
    r1 = 1.0f / sqrtf(s1 / (float)W + eps);
    r2 = 1.0f / sqrtf(s2 / (float)W + eps);
    if (in_regs) {
#pragma unroll
      for (int i = 0; i < RMAX; i++) {
        const int e = tid + i * 256;
        if (e < W) za[i] = 0.5f * (za[i] * r1 * w1[e] + zb[i] * r2 * w2[e]);
      }
    }
  }
  float rz = 1.f;
  if (wn) {
    float sz = 0.f;
    if (in_regs) {
#pragma unroll
      for (int i = 0; i < RMAX; i++) sz += za[i] * za[i];
    } else {
      for (int e = tid; e < W; e += 256) {
        const float z = b ? 0.5f * (a[e] * r1 * w1[e] + b[e] * r2 * w2[e]) : a[e];
        sz += z * z;
      }
    }
    sz = block_sum256(sz, red);
    rz = 1.0f / sqrtf(sz / (float)W + eps);
  }
  if (in_regs) {
#pragma unroll
    for (int i = 0; i < RMAX; i++) {
      const int e = tid + i * 256;
      if (e < W) {
        const float r = wn ? za[i] * rz * (one_plus ? 1.0f + wn[e] : wn[e]) : za[i];
        if (xres) xres[(size_t)t * W + e] += r;
        else st_elem(out, (size_t)t * W + e, r);
      }
    }
    return;
  }
  for (int e = tid; e < W; e += 256) {
    const float z = b ? 0.5f * (a[e] * r1 * w1[e] + b[e] * r2 * w2[e]) : a[e];
    const float r = wn ? z * rz * (one_plus ? 1.0f + wn[e] : wn[e]) : z;
    if (xres) xres[(size_t)t * W + e] += r;
    else st_elem(out, (size_t)t * W + e, r);
  }
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

template <typename KT, typename OT>
int sigattn_fwd_launch(const ktx_sigattn_config& c, int T, int KC, size_t lds, int nsplit, const float* q, const void* kc,
                              const float* kinv, const int32_t* tr, const int32_t* pos, const int32_t* pip, const int32_t* pix,
                              const float* pb, const float* talk, float* partial, void* out, hipStream_t st) {
  const int HD = c.heads * c.dim;
  const int no = (HD + 255) / 256;
  const dim3 grid(T, nsplit);
#define KTX_SA_GO(NO)                                                                                                      \
  do {                                                                                                                     \
    KTX_HIP(ktx_set_max_lds((const void*)sigattn_fwd_kernel<KT, OT, NO>, 160 * 1024));                                     \
    sigattn_fwd_kernel<KT, OT, NO><<<grid, 256, lds, st>>>(c, T, KC, q, (const KT*)kc, kinv, tr, pos, pip, pix, pb, talk, partial, \
                                                           (OT*)out);                                                      \
  } while (0)
  if (no <= 1) KTX_SA_GO(1);
  else if (no <= 2) KTX_SA_GO(2);
  else if (no <= 4) KTX_SA_GO(4);
  else if (no <= 8) KTX_SA_GO(8);
  else if (no <= 16) KTX_SA_GO(16);
  else if (no <= 32) KTX_SA_GO(32);
  else return ktx_fail("ktx_sigattn_forward: heads * dim must be <= 8192");
#undef KTX_SA_GO
  KTX_HIP(hipGetLastError());
  return 0;
}


}  // namespace

// =====================================================================================================================
extern "C" {

int ktx_embed_sinpos(int T, int width, int vocab, const int32_t* d_tokens, const int32_t* d_pos, const void* d_embed,
                     int embed_dtype, const double* d_inv_freq, float* d_x, ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && width > 0 && vocab > 0, "ktx_embed_sinpos: T >= 0, width, vocab > 0");
  KTX_REQUIRE(d_tokens && d_embed && d_x && (d_pos || !d_inv_freq), "ktx_embed_sinpos: null pointer");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (embed_dtype == KTX_SEQ_BF16)
    embed_sinpos_kernel<bf16_t><<<T, 256, 0, st>>>(width, vocab, d_tokens, d_pos, (const bf16_t*)d_embed, d_inv_freq, d_x);
  else if (embed_dtype == KTX_SEQ_F32)
    embed_sinpos_kernel<float><<<T, 256, 0, st>>>(width, vocab, d_tokens, d_pos, (const float*)d_embed, d_inv_freq, d_x);
  else
    return ktx_fail("ktx_embed_sinpos: unknown element type");
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_dense_gemv_glu(int M, int F, int K, const void* d_A, int a_dtype, int64_t lda, const void* d_W, void* d_Y, int y_dtype, int64_t ldy,
                       float limit, float slope, float up_shift, ktx_stream_t stream) {
  KTX_REQUIRE(M >= 0 && M <= 16 && F > 0 && K > 0 && K % 32 == 0 && d_A && d_W && d_Y && lda >= K && ldy >= F && limit > 0.f,
              "ktx_dense_gemv_glu: at most 16 rows, K a multiple of 32");
  KTX_REQUIRE((a_dtype == KTX_SEQ_F32 || a_dtype == KTX_SEQ_BF16) && (y_dtype == KTX_SEQ_F32 || y_dtype == KTX_SEQ_BF16),
              "ktx_dense_gemv_glu: unknown element type");
  KTX_REQUIRE(aligned16(d_W) && aligned16(d_A) && (lda * (a_dtype == KTX_SEQ_F32 ? 4 : 2)) % 16 == 0, "ktx_dense_gemv_glu: 16-byte aligned rows");
  if (M == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const int N = 2 * F;
  const unsigned blocks = (unsigned)((N + 15) / 16);
#define KTX_GLU_GO(AT, YT)                                                                                                         \
  dense_gemv_mfma_kernel<AT, YT, true><<<blocks, 256, 0, st>>>(M, N, K, (const AT*)d_A, lda, (const bf16_t*)d_W, (YT*)d_Y, ldy, 0, limit, \
                                                               slope, up_shift)
  if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32) KTX_GLU_GO(float, float);
  else if (a_dtype == KTX_SEQ_F32) KTX_GLU_GO(float, bf16_t);
  else if (y_dtype == KTX_SEQ_F32) KTX_GLU_GO(bf16_t, float);
  else KTX_GLU_GO(bf16_t, bf16_t);
#undef KTX_GLU_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_dense_gemm(int M, int N, int K, const void* d_A, int a_dtype, int64_t lda, const void* d_W, int w_dtype, void* d_Y,
                   int y_dtype, int64_t ldy, int act, int ksplit, ktx_stream_t stream) {
  KTX_REQUIRE(M >= 0 && N > 0 && K > 0, "ktx_dense_gemm: M >= 0, N, K > 0");
  KTX_REQUIRE(d_A && d_W && d_Y, "ktx_dense_gemm: null pointer");
  KTX_REQUIRE(lda >= K && ldy >= N, "ktx_dense_gemm: lda >= K and ldy >= N");
  KTX_REQUIRE(act == KTX_ACT_NONE || act == KTX_ACT_GELU_TANH, "ktx_dense_gemm: unknown activation");
  KTX_REQUIRE(ksplit >= 1 && (ksplit == 1 || (y_dtype == KTX_SEQ_F32 && act == KTX_ACT_NONE)),
              "ktx_dense_gemm: split-K adds into a zeroed fp32 output and takes no activation");
  KTX_REQUIRE(!(w_dtype == KTX_SEQ_F32 && a_dtype != KTX_SEQ_F32), "ktx_dense_gemm: an fp32 product needs fp32 activations");
  if (M == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (M <= 16 && ksplit == 1 && w_dtype == KTX_SEQ_BF16 && K % 32 == 0 && aligned16(d_W) && aligned16(d_A) &&
      (lda * (a_dtype == KTX_SEQ_F32 ? 4 : 2)) % 16 == 0) {
    const unsigned blocks = (unsigned)((N + 15) / 16);
    if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32)
      dense_gemv_mfma_kernel<float, float, false><<<blocks, 256, 0, st>>>(M, N, K, (const float*)d_A, lda, (const bf16_t*)d_W, (float*)d_Y, ldy, act, 0.f, 0.f, 0.f);
    else if (a_dtype == KTX_SEQ_F32)
      dense_gemv_mfma_kernel<float, bf16_t, false><<<blocks, 256, 0, st>>>(M, N, K, (const float*)d_A, lda, (const bf16_t*)d_W, (bf16_t*)d_Y, ldy, act, 0.f, 0.f, 0.f);
    else if (y_dtype == KTX_SEQ_F32)
      dense_gemv_mfma_kernel<bf16_t, float, false><<<blocks, 256, 0, st>>>(M, N, K, (const bf16_t*)d_A, lda, (const bf16_t*)d_W, (float*)d_Y, ldy, act, 0.f, 0.f, 0.f);
    else
      dense_gemv_mfma_kernel<bf16_t, bf16_t, false><<<blocks, 256, 0, st>>>(M, N, K, (const bf16_t*)d_A, lda, (const bf16_t*)d_W, (bf16_t*)d_Y, ldy, act, 0.f, 0.f, 0.f);
    KTX_HIP(hipGetLastError());
    return 0;
  }
  {
    // decode-sized calls of any other shape or type: the streaming kernel, when the activation rows fit the LDS
    const size_t wsz0 = w_dtype == KTX_SEQ_F32 ? 4 : 2;
    const int mm = M <= 2 ? 2 : 8;
    const size_t lds = (size_t)mm * ((K + 7) & ~7) * wsz0;
    if (M <= 8 && ksplit == 1 && lds <= 128 * 1024 && (w_dtype == KTX_SEQ_BF16 || y_dtype == KTX_SEQ_F32)) {
      const bool vec = aligned16(d_W) && ((size_t)K * wsz0) % 16 == 0;
      const unsigned blocks = (unsigned)((N + 7) / 8);
#define KTX_GEMV_GO(AT, CT, YT, MM)                                                                                     \
  do {                                                                                                                  \
    KTX_HIP(ktx_set_max_lds((const void*)dense_gemv_kernel<AT, CT, YT, MM>, 128 * 1024));                               \
    dense_gemv_kernel<AT, CT, YT, MM><<<blocks, 256, lds, st>>>(M, N, K, (const AT*)d_A, lda, (const CT*)d_W, (YT*)d_Y, ldy, act, vec); \
  } while (0)
#define KTX_GEMV_MM(AT, CT, YT)            \
  do {                                     \
    if (mm == 2) KTX_GEMV_GO(AT, CT, YT, 2); \
    else KTX_GEMV_GO(AT, CT, YT, 8);       \
  } while (0)
      if (w_dtype == KTX_SEQ_F32) KTX_GEMV_MM(float, float, float);
      else if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32) KTX_GEMV_MM(float, bf16_t, float);
      else if (a_dtype == KTX_SEQ_F32) KTX_GEMV_MM(float, bf16_t, bf16_t);
      else if (y_dtype == KTX_SEQ_F32) KTX_GEMV_MM(bf16_t, bf16_t, float);
      else KTX_GEMV_MM(bf16_t, bf16_t, bf16_t);
#undef KTX_GEMV_MM
#undef KTX_GEMV_GO
      KTX_HIP(hipGetLastError());
      return 0;
    }
  }
  const dim3 grid((N + 63) / 64, (M + 63) / 64, ksplit);
  KTX_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "ktx_dense_gemm: too many row tiles / splits");
  const size_t asz = a_dtype == KTX_SEQ_F32 ? 4 : 2, wsz = w_dtype == KTX_SEQ_F32 ? 4 : 2;
  const bool vec_a = aligned16(d_A) && (lda * asz) % 16 == 0 && K % 8 == 0;
  const bool vec_w = aligned16(d_W) && ((size_t)K * wsz) % 16 == 0 && K % 8 == 0;
#define KTX_GEMM_GO(AT, CT, YT)                                                                                          \
  dense_gemm_kernel<AT, CT, YT><<<grid, 256, 0, st>>>(M, N, K, (const AT*)d_A, lda, (const CT*)d_W, (YT*)d_Y, ldy, act, ksplit, \
                                                      vec_a, vec_w)
  if (w_dtype == KTX_SEQ_BF16) {
    if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_F32) KTX_GEMM_GO(float, bf16_t, float);
    else if (a_dtype == KTX_SEQ_F32 && y_dtype == KTX_SEQ_BF16) KTX_GEMM_GO(float, bf16_t, bf16_t);
    else if (a_dtype == KTX_SEQ_BF16 && y_dtype == KTX_SEQ_F32) KTX_GEMM_GO(bf16_t, bf16_t, float);
    else if (a_dtype == KTX_SEQ_BF16 && y_dtype == KTX_SEQ_BF16) KTX_GEMM_GO(bf16_t, bf16_t, bf16_t);
    else return ktx_fail("ktx_dense_gemm: unknown element type");
  } else if (w_dtype == KTX_SEQ_F32) {
    if (y_dtype == KTX_SEQ_F32) KTX_GEMM_GO(float, float, float);
    else return ktx_fail("ktx_dense_gemm: an fp32 product writes fp32");
  } else {
    return ktx_fail("ktx_dense_gemm: unknown element type");
  }
#undef KTX_GEMM_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

static int sigattn_check(const ktx_sigattn_config* c, const char* who) {
  if (!c || c->heads <= 0 || c->kv_heads <= 0 || c->dim <= 0 || c->heads % c->kv_heads != 0 || c->page_size <= 0 ||
      (c->cache_dtype != KTX_SEQ_F32 && c->cache_dtype != KTX_SEQ_BF16))
    return ktx_fail(std::string(who) + ": heads, kv_heads (dividing heads), dim, page_size must be positive and cache_dtype known");
  return 0;
}

int ktx_sigattn_prep(const ktx_sigattn_config* cfg, int T, const float* d_proj, int64_t ldp, int q_off, int k_off,
                     const float* d_wq, const float* d_wk, float eps, const int32_t* d_pos, const int32_t* d_cache_loc,
                     void* d_kcache, float* d_kinv, float* d_q_out, ktx_stream_t stream) {
  if (int rc = sigattn_check(cfg, "ktx_sigattn_prep")) return rc;
  KTX_REQUIRE(T >= 0 && d_proj && d_wq && d_wk && d_pos && d_cache_loc && d_kcache && d_kinv && d_q_out, "ktx_sigattn_prep: null pointer");
  KTX_REQUIRE(q_off >= 0 && k_off >= 0 && ldp >= (int64_t)q_off + cfg->heads * cfg->dim && ldp >= (int64_t)k_off + cfg->kv_heads * cfg->dim,
              "ktx_sigattn_prep: q / k columns lie outside a row of proj");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (cfg->cache_dtype == KTX_SEQ_BF16)
    sigattn_prep_kernel<bf16_t><<<T, 256, 0, st>>>(*cfg, d_proj, ldp, q_off, k_off, d_wq, d_wk, eps, d_pos, d_cache_loc,
                                                   (bf16_t*)d_kcache, d_kinv, d_q_out);
  else
    sigattn_prep_kernel<float><<<T, 256, 0, st>>>(*cfg, d_proj, ldp, q_off, k_off, d_wq, d_wk, eps, d_pos, d_cache_loc,
                                                  (float*)d_kcache, d_kinv, d_q_out);
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_sigattn_forward(const ktx_sigattn_config* cfg, int T, const float* d_q, const void* d_kcache, const float* d_kinv,
                        const int32_t* d_tok_req, const int32_t* d_pos, const int32_t* d_page_indptr,
                        const int32_t* d_page_indices, const float* d_pb, const float* d_talk, int nsplit, float* d_partial,
                        void* d_out, int out_dtype, ktx_stream_t stream) {
  if (int rc = sigattn_check(cfg, "ktx_sigattn_forward")) return rc;
  KTX_REQUIRE(T >= 0 && d_q && d_kcache && d_kinv && d_tok_req && d_pos && d_page_indptr && d_page_indices && d_pb && d_talk && d_out,
              "ktx_sigattn_forward: null pointer");
  KTX_REQUIRE(nsplit >= 1 && nsplit <= 65535 && (nsplit == 1 || d_partial), "ktx_sigattn_forward: nsplit >= 1, with scratch when > 1");
  KTX_REQUIRE(out_dtype == KTX_SEQ_F32 || out_dtype == KTX_SEQ_BF16, "ktx_sigattn_forward: unknown output type");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const ktx_sigattn_config& c = *cfg;
  const size_t HD = (size_t)c.heads * c.dim, kst = ((size_t)c.kv_heads * c.dim) | 1;
  // keys per staged chunk: the largest power of two (<= 64) whose rows fit 96 KiB of LDS beside q and the weight tiles
  int KC = 64;
  auto lds_of = [&](int kc) { return (HD + (size_t)kc * kst + 2 * (size_t)c.heads * kc + kc) * sizeof(float); };
  while (KC > 1 && lds_of(KC) > 96 * 1024) KC >>= 1;
  KTX_REQUIRE(lds_of(KC) <= 150 * 1024, "ktx_sigattn_forward: one key row of all heads does not fit the LDS");
  const size_t lds = lds_of(KC);
  int rc;
  const bool direct = nsplit == 1;
  if (c.cache_dtype == KTX_SEQ_BF16) {
    if (direct && out_dtype == KTX_SEQ_BF16)
      rc = sigattn_fwd_launch<bf16_t, bf16_t>(c, T, KC, lds, nsplit, d_q, d_kcache, d_kinv, d_tok_req, d_pos, d_page_indptr, d_page_indices, d_pb, d_talk, d_partial, d_out, st);
    else
      rc = sigattn_fwd_launch<bf16_t, float>(c, T, KC, lds, nsplit, d_q, d_kcache, d_kinv, d_tok_req, d_pos, d_page_indptr, d_page_indices, d_pb, d_talk, d_partial, d_out, st);
  } else {
    if (direct && out_dtype == KTX_SEQ_BF16)
      rc = sigattn_fwd_launch<float, bf16_t>(c, T, KC, lds, nsplit, d_q, d_kcache, d_kinv, d_tok_req, d_pos, d_page_indptr, d_page_indices, d_pb, d_talk, d_partial, d_out, st);
    else
      rc = sigattn_fwd_launch<float, float>(c, T, KC, lds, nsplit, d_q, d_kcache, d_kinv, d_tok_req, d_pos, d_page_indptr, d_page_indices, d_pb, d_talk, d_partial, d_out, st);
  }
  if (rc) return rc;
  if (!direct) {
    const size_t n = (size_t)T * HD;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (out_dtype == KTX_SEQ_BF16) sigattn_reduce_kernel<bf16_t><<<blocks, 256, 0, st>>>(nsplit, n, d_partial, (bf16_t*)d_out);
    else sigattn_reduce_kernel<float><<<blocks, 256, 0, st>>>(nsplit, n, d_partial, (float*)d_out);
    KTX_HIP(hipGetLastError());
  }
  return 0;
}

int ktx_sigattn_prefill_eligible(const ktx_sigattn_config* c) {
  if (!c || sigattn_check(c, "ktx_sigattn_prefill_eligible")) return 0;
  return c->cache_dtype == KTX_SEQ_BF16 && c->dim % 32 == 0 && c->dim <= 128 && c->heads <= 16 && sigattn_mfma_lds(*c) <= 150 * 1024;
}

int ktx_sigattn_prefill(const ktx_sigattn_config* cfg, int B, int T, int max_q_len, const float* d_q, const void* d_kcache,
                        const float* d_kinv, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_page_indptr,
                        const int32_t* d_page_indices, const float* d_pb, const float* d_talk, int nsplit, float* d_partial,
                        void* d_out, ktx_stream_t stream) {
  KTX_REQUIRE(ktx_sigattn_prefill_eligible(cfg), "ktx_sigattn_prefill: needs a bf16 cache, dim % 32 == 0, dim <= 128, heads <= 16");
  KTX_REQUIRE(B >= 0 && T >= 0 && max_q_len >= 0 && d_q && d_kcache && d_kinv && d_q_indptr && d_pos0 && d_page_indptr && d_page_indices &&
                  d_pb && d_talk && d_out, "ktx_sigattn_prefill: null pointer");
  KTX_REQUIRE(B <= 65535 && nsplit >= 1 && nsplit <= 65535 && (nsplit == 1 || d_partial),
              "ktx_sigattn_prefill: at most 65535 requests and key ranges a call; scratch when nsplit > 1");
  if (B == 0 || max_q_len == 0 || T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const ktx_sigattn_config& c = *cfg;
  const dim3 grid((max_q_len + 15) / 16, B, nsplit);
  const size_t lds = sigattn_mfma_lds(c);
  const int nhw = (c.heads + 3) / 4, ds = c.dim / 32;
#define KTX_SP_GO(NHW, DS)                                                                                                   \
  do {                                                                                                                       \
    KTX_HIP(ktx_set_max_lds((const void*)sigattn_mfma_kernel<NHW, DS>, 160 * 1024));                                         \
    sigattn_mfma_kernel<NHW, DS><<<grid, 256, lds, st>>>(c, T, d_q, (const bf16_t*)d_kcache, d_kinv, d_q_indptr, d_pos0,     \
                                                         d_page_indptr, d_page_indices, d_pb, d_talk, d_partial, (bf16_t*)d_out); \
  } while (0)
#define KTX_SP_DS(NHW)                                                          \
  do {                                                                          \
    if (ds == 1) KTX_SP_GO(NHW, 1);                                             \
    else if (ds == 2) KTX_SP_GO(NHW, 2);                                        \
    else if (ds == 3) KTX_SP_GO(NHW, 3);                                        \
    else KTX_SP_GO(NHW, 4);                                                     \
  } while (0)
  if (nhw <= 1) KTX_SP_DS(1);
  else if (nhw <= 2) KTX_SP_DS(2);
  else if (nhw <= 3) KTX_SP_DS(3);
  else KTX_SP_DS(4);
#undef KTX_SP_DS
#undef KTX_SP_GO
  KTX_HIP(hipGetLastError());
  if (nsplit > 1) {
    const size_t n = (size_t)T * c.heads * c.dim;
    sigattn_reduce_kernel<bf16_t><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(nsplit, n, d_partial, (bf16_t*)d_out);
    KTX_HIP(hipGetLastError());
  }
  return 0;
}

int ktx_gelu_tanh(size_t n, void* d_y, int dtype, ktx_stream_t stream) {
  KTX_REQUIRE(d_y || n == 0, "ktx_gelu_tanh: null pointer");
  if (n == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (dtype == KTX_SEQ_BF16) gelu_tanh_kernel<bf16_t><<<blocks, 256, 0, st>>>(n, (bf16_t*)d_y);
  else if (dtype == KTX_SEQ_F32) gelu_tanh_kernel<float><<<blocks, 256, 0, st>>>(n, (float*)d_y);
  else return ktx_fail("ktx_gelu_tanh: unknown element type");
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_mlstm_forward(const ktx_mlstm_config* cfg, int B, const int32_t* d_q_indptr, const int32_t* d_pos0, const int32_t* d_slot,
                      const float* d_proj, int64_t ldp, int q_off, int k_off, int v_off, int i_off, int f_off, const float* d_ib,
                      const float* d_fb, float* d_S, float* d_n, float* d_m, float* d_gates, float* d_o_raw, int max_q_len,
                      ktx_stream_t stream) {
  KTX_REQUIRE(cfg && cfg->heads > 0 && cfg->dim > 0 && cfg->vdim > 0, "ktx_mlstm_forward: heads, dim, vdim must be positive");
  KTX_REQUIRE(cfg->dim <= 256, "ktx_mlstm_forward: dim must be <= 256 (a wavefront keeps dim / 4 state rows in registers)");
  KTX_REQUIRE(B >= 0 && d_q_indptr && d_pos0 && d_slot && d_proj && d_ib && d_fb && d_S && d_n && d_m && d_gates && d_o_raw,
              "ktx_mlstm_forward: null pointer");
  const int64_t need = std::max(std::max((int64_t)q_off + cfg->heads * cfg->dim, (int64_t)k_off + cfg->heads * cfg->dim),
                                std::max((int64_t)v_off + cfg->heads * cfg->vdim, (int64_t)std::max(i_off, f_off) + cfg->heads));
  KTX_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && i_off >= 0 && f_off >= 0 && ldp >= need,
              "ktx_mlstm_forward: q / k / v / gate columns lie outside a row of proj");
  if (B == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(B, cfg->heads, (cfg->vdim + 63) / 64);
  KTX_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "ktx_mlstm_forward: too many heads / value columns");
  // scratch layout: [T][heads][6] gate records, then [B][heads] starting maxima; T is not known here, so the maxima come FIRST
  float* minit = d_gates;
  float* grec = d_gates + (size_t)B * cfg->heads;
  mlstm_gates_kernel<<<dim3(B, cfg->heads), 256, 0, st>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_proj, ldp, i_off, f_off, d_ib, d_fb, d_m,
                                                          grec, minit);
  if (max_q_len >= ML_CL && mlstm_chunk_lds(cfg->dim) <= 150 * 1024) {
    KTX_HIP(ktx_set_max_lds((const void*)mlstm_chunk_kernel, 160 * 1024));
    mlstm_chunk_kernel<<<grid, 256, mlstm_chunk_lds(cfg->dim), st>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_proj, ldp, q_off, k_off, v_off,
                                                                     grec, minit, d_S, d_n, d_o_raw);
    KTX_HIP(hipGetLastError());
    return 0;
  }
  d_gates = grec;
  const int dpg = (cfg->dim + 3) / 4;
#define KTX_ML_GO(DPG)                                                                                                       \
  mlstm_fwd_kernel<DPG><<<grid, 256, 0, st>>>(*cfg, d_q_indptr, d_pos0, d_slot, d_proj, ldp, q_off, k_off, v_off, d_gates, d_S, \
                                              d_n, d_o_raw)
  if (dpg <= 4) KTX_ML_GO(4);
  else if (dpg <= 8) KTX_ML_GO(8);
  else if (dpg <= 16) KTX_ML_GO(16);
  else if (dpg <= 32) KTX_ML_GO(32);
  else KTX_ML_GO(64);
#undef KTX_ML_GO
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_mlstm_gate_norm(const ktx_mlstm_config* cfg, int T, const float* d_o_raw, const float* d_proj, int64_t ldp, int g_off,
                        const float* d_w, void* d_out, int out_dtype, ktx_stream_t stream) {
  KTX_REQUIRE(cfg && cfg->heads > 0 && cfg->vdim > 0, "ktx_mlstm_gate_norm: heads, vdim must be positive");
  KTX_REQUIRE(T >= 0 && d_o_raw && d_proj && d_w && d_out, "ktx_mlstm_gate_norm: null pointer");
  KTX_REQUIRE(g_off >= 0 && ldp >= (int64_t)g_off + cfg->heads * cfg->vdim, "ktx_mlstm_gate_norm: gate columns lie outside a row of proj");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  const unsigned blocks = (unsigned)(((size_t)T * cfg->heads + 3) / 4);
  if (out_dtype == KTX_SEQ_BF16) mlstm_gate_norm_kernel<bf16_t><<<blocks, 256, 0, st>>>(*cfg, T, d_o_raw, d_proj, ldp, g_off, d_w, (bf16_t*)d_out);
  else if (out_dtype == KTX_SEQ_F32) mlstm_gate_norm_kernel<float><<<blocks, 256, 0, st>>>(*cfg, T, d_o_raw, d_proj, ldp, g_off, d_w, (float*)d_out);
  else return ktx_fail("ktx_mlstm_gate_norm: unknown output type");
  KTX_HIP(hipGetLastError());
  return 0;
}

int ktx_rms_combine(int T, int W, const float* d_y1, const float* d_w1, const float* d_y2, const float* d_w2, const float* d_wn,
                    int one_plus, float eps, float* d_x_residual, const int32_t* d_rows, void* d_out, int out_dtype,
                    ktx_stream_t stream) {
  KTX_REQUIRE(T >= 0 && W > 0 && d_y1, "ktx_rms_combine: T >= 0, W > 0, y1 non-null");
  KTX_REQUIRE(!d_y2 || (d_w1 && d_w2), "ktx_rms_combine: two inputs need their two weights");
  KTX_REQUIRE(!d_y2 || !d_rows, "ktx_rms_combine: the row gather is for the single-input form");
  KTX_REQUIRE((d_x_residual != nullptr) != (d_out != nullptr), "ktx_rms_combine: exactly one of x_residual / out");
  if (T == 0) return 0;
  hipStream_t st = (hipStream_t)stream;
  if (d_x_residual || out_dtype == KTX_SEQ_F32)
    rms_combine_kernel<float><<<T, 256, 0, st>>>(W, d_y1, d_w1, d_y2, d_w2, d_wn, one_plus, eps, d_x_residual, d_rows, (float*)d_out);
  else if (out_dtype == KTX_SEQ_BF16)
    rms_combine_kernel<bf16_t><<<T, 256, 0, st>>>(W, d_y1, d_w1, d_y2, d_w2, d_wn, one_plus, eps, d_x_residual, d_rows, (bf16_t*)d_out);
  else
    return ktx_fail("ktx_rms_combine: unknown output type");
  KTX_HIP(hipGetLastError());
  return 0;
}

}  // extern "C"
