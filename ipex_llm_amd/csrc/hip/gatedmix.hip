// Kernels of the gated recurrent mixers and the two-norm parallel blocks
// (gfx950, wave64).
//
//   norm pair + shift  one workgroup per token: LayerNorm statistics of the
//                      token's row and of the row before it (the previous
//                      token of the same portion; at a portion's start the
//                      sequence's state slot, at position 0 zeros), both
//                      norms' results, the first one shifted towards the
//                      previous token's.  The last token of every sequence
//                      leaves its unshifted first norm for the slot: written
//                      by the same launch when every sequence brings one
//                      token, otherwise through a scratch row and a copy
//                      launch (another workgroup may still read the slot)
//   minGRU scan        S' = (1 - z) S + z c is a linear recurrence per
//                      channel: a workgroup holds 64 channels x NC pieces of
//                      a portion; every thread folds its piece into (product
//                      of the factors, result from zero), the pieces' carries
//                      are chained through LDS in order, then every thread
//                      runs its piece again from its carry and writes
//                      S silu(g).  NC = 1 for decoded tokens
//   gated linear attention scan
//                      S' = diag(alpha) S + k v^T, o = S'^T q.  One workgroup:
//                      64 value columns of one (sequence, head); wave w keeps
//                      the state rows [w NS, (w + 1) NS) of those columns in
//                      registers; tokens go through LDS in chunks (decays
//                      exp(log_sigmoid(a) / tau), keys and scaled queries as
//                      f32, zero padded to the waves' rows); the waves'
//                      partial o are summed in wave order
//   head norm + gate   per-head RMS norm with a weight shared by the heads,
//                      times silu(gate)
//   pair mean          (rms_norm(a) wa + rms_norm(b) wb) / 2
//   softcap            cap tanh(x / cap)
//
// Activations are bf16 or f32 (template E); accumulation is always f32.
#include "gatedmix.h"

#include <math.h>

namespace illm {
namespace gm {
namespace {

template <typename E> __device__ __forceinline__ float ldf(const E* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<__bf16>(const __bf16* p) { return (float)*p; }
template <typename E> __device__ __forceinline__ void stf(E* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<__bf16>(__bf16* p, float v) { *p = (__bf16)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int w = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[w] = v;
  __syncthreads();
  float s = 0.f;
  for (int i = 0; i < nw; i++) s += red[i];
  return s;
}
__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu(float z) { return z / (1.0f + expf(-z)); }

// mean and 1 / sqrt(variance + eps) of a row (variance = mean squared deviation), every thread gets both
__device__ __forceinline__ void row_stats(const float* __restrict__ x, int W, float eps, float* red, float* mean,
                                          float* rstd) {
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += x[c];
  const float mu = block_sum(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float dlt = x[c] - mu;
    q += dlt * dlt;
  }
  *mean = mu;
  *rstd = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
}

// ------------------------------------------------------------------ norm pair + shift
template <typename E>
__global__ void __launch_bounds__(256) ln_pair_shift_k(const float* __restrict__ x, const E* __restrict__ w1,
                                                      const E* __restrict__ w2, const float* __restrict__ mu,
                                                      float eps, float* __restrict__ state,
                                                      const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_of,
                                                      const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                      E* __restrict__ h1, E* __restrict__ h2, float* __restrict__ last,
                                                      int W, bool single) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * W;
  float mean, rstd;
  row_stats(xr, W, eps, red, &mean, &rstd);
  if (!mu) {                                                        // no shift: two plain norms
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      const float xn = (xr[c] - mean) * rstd;
      stf(h1 + t * W + c, xn * ldf(w1 + c));
      if (w2) stf(h2 + t * W + c, xn * ldf(w2 + c));
    }
    return;
  }
  const int b = seq_of[t];
  const int i = (int)t - cu[b];
  const bool is_last = (int)t == cu[b + 1] - 1;
  float pm = 0.f, pr = 0.f;
  if (i > 0) row_stats(xr - W, W, eps, red, &pm, &pr);              // the previous token is in this portion
  float* st = state + (int64_t)slots[b] * W;
  const bool from_slot = i == 0 && pos[t] > 0;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float wv = ldf(w1 + c);
    const float xn = (xr[c] - mean) * rstd;
    const float n1 = xn * wv;
    float prev = 0.f;
    if (i > 0) prev = (xr[c - W] - pm) * pr * wv;
    else if (from_slot) prev = st[c];
    stf(h1 + t * W + c, n1 + (prev - n1) * mu[c]);
    if (w2) stf(h2 + t * W + c, xn * ldf(w2 + c));
    if (is_last) {
      if (single) st[c] = n1;                                       // this workgroup is the slot's only reader
      else last[(int64_t)b * W + c] = n1;
    }
  }
}

__global__ void __launch_bounds__(256) rows_to_slots_k(const float* __restrict__ last, float* __restrict__ state,
                                                      const int32_t* __restrict__ cu, const int32_t* __restrict__ slots,
                                                      int W) {
  const int b = blockIdx.x;
  if (cu[b + 1] <= cu[b]) return;
  for (int c = threadIdx.x; c < W; c += blockDim.x) state[(int64_t)slots[b] * W + c] = last[(int64_t)b * W + c];
}

// ------------------------------------------------------------------ minGRU
// thread (lane = channel, wave = piece); LDS: factors [NC][64], results [NC][64]
template <typename E>
__global__ void __launch_bounds__(1024) mingru_scan_k(const E* __restrict__ y, int64_t y_ld, int width,
                                                     float* __restrict__ state, const int32_t* __restrict__ cu,
                                                     const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                     E* __restrict__ out) {
  __shared__ float fa[16][64];
  __shared__ float fb[16][64];
  const int b = blockIdx.y;
  const int lane = threadIdx.x & 63, j = threadIdx.x >> 6, NC = blockDim.x >> 6;
  const int c = blockIdx.x * 64 + lane;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  if (n <= 0) return;
  const bool ok = c < width;
  const int per = (n + NC - 1) / NC;
  const int lo = min(n, j * per), hi = min(n, lo + per);
  const E* yz = y + (int64_t)t0 * y_ld + (ok ? c : 0);
  // the piece folded: S_out = A S_in + B
  float A = 1.f, Bv = 0.f;
  constexpr int UN = 8;                                             // tokens whose inputs are requested together
  if (NC > 1) {
    if (ok)
      for (int tb = lo; tb < hi; tb += UN) {
        float zr[UN], ur[UN];
#pragma unroll
        for (int i = 0; i < UN; i++) {
          const int t = min(tb + i, hi - 1);
          zr[i] = ldf(yz + (int64_t)t * y_ld);
          ur[i] = ldf(yz + (int64_t)t * y_ld + width);
        }
#pragma unroll
        for (int i = 0; i < UN; i++) {
          if (tb + i >= hi) break;
          const float z = sigmoidf(zr[i]);
          const float cand = ur[i] >= 0.f ? ur[i] + 0.5f : sigmoidf(ur[i]);
          A *= 1.0f - z;
          Bv = fmaf(1.0f - z, Bv, z * cand);
        }
      }
    fa[j][lane] = A;
    fb[j][lane] = Bv;
    __syncthreads();
  }
  float* st = state + (int64_t)slots[b] * width + (ok ? c : 0);
  float S = (ok && pos[t0] != 0) ? *st : 0.f;
  for (int jj = 0; jj < j; jj++) S = fmaf(fa[jj][lane], S, fb[jj][lane]);    // the carries in order
  __syncthreads();                                                  // every piece has read the slot
  if (!ok) return;
  E* o = out + (int64_t)t0 * width + c;
  for (int tb = lo; tb < hi; tb += UN) {
    float zr[UN], ur[UN], gr[UN];
#pragma unroll
    for (int i = 0; i < UN; i++) {
      const int t = min(tb + i, hi - 1);
      zr[i] = ldf(yz + (int64_t)t * y_ld);
      ur[i] = ldf(yz + (int64_t)t * y_ld + width);
      gr[i] = ldf(yz + (int64_t)t * y_ld + 2 * width);
    }
#pragma unroll
    for (int i = 0; i < UN; i++) {
      if (tb + i >= hi) break;
      const float z = sigmoidf(zr[i]);
      const float cand = ur[i] >= 0.f ? ur[i] + 0.5f : sigmoidf(ur[i]);
      S = fmaf(1.0f - z, S, z * cand);
      stf(o + (int64_t)(tb + i) * width, S * silu(gr[i]));
    }
  }
  if (hi == n && lo < n) *st = S;                                   // the piece that holds the last token
}

// ------------------------------------------------------------------ gated linear attention
// MAXT: the most threads a launch brings (256, 512 or 1024: the register budget follows it)
template <typename E, int NS, int MAXT>
__global__ void __launch_bounds__(MAXT) gla_scan_k(const E* __restrict__ q, int64_t q_ld, const E* __restrict__ k,
                                                  int64_t k_ld, const E* __restrict__ v, int64_t v_ld,
                                                  const E* __restrict__ a, int64_t a_ld, float inv_tau, float q_scale,
                                                  float* __restrict__ S, const int32_t* __restrict__ cu,
                                                  const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                  float* __restrict__ out, int H, int d, int dv, int TC) {
  extern __shared__ __align__(16) float sm[];
  const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * 64;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  const int NP = NW * NS;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  if (n <= 0) return;
  const int pc = p0 + lane;
  float* As = sm;                                                   // [TC][NP] decays
  float* Ks = As + (size_t)TC * NP;                                 // [TC][NP]
  float* Qs = Ks + (size_t)TC * NP;                                 // [TC][NP]
  float* vs = Qs + (size_t)TC * NP;                                 // [TC][64]
  float* pt = vs + (size_t)TC * 64;                                 // [NW][TC][64]
  float st[NS];
  float* Sg = S + (((int64_t)slots[b] * H + h) * d) * dv;           // [d][dv]
  const bool fresh = pos[t0] == 0;
#pragma unroll
  for (int i = 0; i < NS; i++) {
    const int r = wv * NS + i;
    st[i] = (!fresh && r < d && pc < dv) ? Sg[(int64_t)r * dv + pc] : 0.f;
  }
  for (int c0 = 0; c0 < n; c0 += TC) {
    const int nc = min(TC, n - c0);
    __syncthreads();
    for (int i = threadIdx.x; i < nc * NP; i += blockDim.x) {
      const int tt = i / NP, r = i - tt * NP;
      const int64_t t = t0 + c0 + tt;
      float al = 1.f, kk = 0.f, qq = 0.f;
      if (r < d) {
        const float z = ldf(a + t * a_ld + h * d + r);
        // log sigmoid(z) = min(z, 0) - log1p(exp(-|z|))
        al = expf((fminf(z, 0.f) - log1pf(expf(-fabsf(z)))) * inv_tau);
        kk = ldf(k + t * k_ld + h * d + r);
        qq = ldf(q + t * q_ld + h * d + r) * q_scale;
      }
      As[i] = al;
      Ks[i] = kk;
      Qs[i] = qq;
    }
    for (int i = threadIdx.x; i < nc * 64; i += blockDim.x) {
      const int tt = i >> 6, cc = p0 + (i & 63);
      vs[i] = cc < dv ? ldf(v + (int64_t)(t0 + c0 + tt) * v_ld + h * dv + cc) : 0.f;
    }
    __syncthreads();
    for (int tt = 0; tt < nc; tt++) {
      const float vv = vs[tt * 64 + lane];
      const float4* a4 = (const float4*)(As + (size_t)tt * NP + wv * NS);
      const float4* k4 = (const float4*)(Ks + (size_t)tt * NP + wv * NS);
      const float4* q4 = (const float4*)(Qs + (size_t)tt * NP + wv * NS);
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NS / 4; i++) {
        const float4 av = a4[i], kv = k4[i], qv = q4[i];
        st[4 * i] = fmaf(av.x, st[4 * i], kv.x * vv);
        st[4 * i + 1] = fmaf(av.y, st[4 * i + 1], kv.y * vv);
        st[4 * i + 2] = fmaf(av.z, st[4 * i + 2], kv.z * vv);
        st[4 * i + 3] = fmaf(av.w, st[4 * i + 3], kv.w * vv);
        acc = fmaf(st[4 * i], qv.x, acc);
        acc = fmaf(st[4 * i + 1], qv.y, acc);
        acc = fmaf(st[4 * i + 2], qv.z, acc);
        acc = fmaf(st[4 * i + 3], qv.w, acc);
      }
      pt[((size_t)wv * TC + tt) * 64 + lane] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nc * 64; i += blockDim.x) {
      const int tt = i >> 6, cc = p0 + (i & 63);
      if (cc >= dv) continue;
      float o = 0.f;
      for (int w = 0; w < NW; w++) o += pt[((size_t)w * TC + tt) * 64 + (i & 63)];
      out[((int64_t)(t0 + c0 + tt) * H + h) * dv + cc] = o;
    }
  }
#pragma unroll
  for (int i = 0; i < NS; i++) {
    const int r = wv * NS + i;
    if (r < d && pc < dv) Sg[(int64_t)r * dv + pc] = st[i];
  }
}

// the product of a piece's decays per (head, key channel): P = exp(sum_t log_sigmoid(a_t) / tau), summed in f64.
// One workgroup per (piece, head): 64 channels x 4 token groups
template <typename E>
__global__ void __launch_bounds__(256) gla_piece_decay_k(const E* __restrict__ a, int64_t a_ld,
                                                        const int32_t* __restrict__ cu, float inv_tau,
                                                        float* __restrict__ P, int H, int d) {
  __shared__ double part[4][64];
  const int piece = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, tg = threadIdx.x >> 6;
  const int t0 = cu[piece], t1 = cu[piece + 1];
  for (int r0 = 0; r0 < d; r0 += 64) {
    const int r = r0 + lane;
    double sum = 0.0;
    if (r < d)
      for (int t = t0 + tg; t < t1; t += 4) {
        const float z = ldf(a + (int64_t)t * a_ld + h * d + r);
        sum += (double)(fminf(z, 0.f) - log1pf(expf(-fabsf(z))));
      }
    __syncthreads();
    part[tg][lane] = sum;
    __syncthreads();
    if (tg == 0 && r < d)
      P[((int64_t)piece * H + h) * d + r] =
          expf((float)((part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane]) * (double)inv_tau));
  }
}

// start states of the pieces of a sequence, piece after piece: the first piece's end state Z[f] starts the second;
// then S <- diag(P) S + Z.  seqs int32 [n][2]: first piece, number of pieces
__global__ void __launch_bounds__(256) gla_chain_k(const float* __restrict__ Z, float* __restrict__ Sin,
                                                  const float* __restrict__ P, const int32_t* __restrict__ seqs, int HD,
                                                  int dv) {
  const int f = seqs[2 * blockIdx.x], m = seqs[2 * blockIdx.x + 1];
  if (m < 2) return;
  const int64_t n = (int64_t)HD * dv;
  for (int64_t e = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.y * blockDim.x) {
    const int64_t hr = e / dv;
    float S = Z[f * n + e];
    Sin[(f + 1) * n + e] = S;
    for (int j = 2; j < m; j++) {
      S = fmaf(P[(int64_t)(f + j - 1) * HD + hr], S, Z[(f + j - 1) * n + e]);
      Sin[(f + j) * n + e] = S;
    }
  }
}

// ------------------------------------------------------------------ element-wise steps
template <typename E>
__global__ void __launch_bounds__(64) head_rms_silu_k(const float* __restrict__ o, const E* __restrict__ nw,
                                                     const E* __restrict__ gate, int64_t g_ld, E* __restrict__ out, int H,
                                                     int dv, float eps) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* in = o + (t * H + h) * dv;
  float q = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) q += in[c] * in[c];
  const float rs = 1.0f / sqrtf(wave_sum(q) / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += 64)
    stf(out + (t * H + h) * dv + c, in[c] * rs * ldf(nw + c) * silu(ldf(gate + t * g_ld + h * dv + c)));
}

template <typename E>
__global__ void __launch_bounds__(256) rms_pair_mean_k(const E* __restrict__ a, const E* __restrict__ b,
                                                      const E* __restrict__ wa, const E* __restrict__ wb,
                                                      E* __restrict__ out, int W, float eps) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  float qa = 0.f, qb = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float x = ldf(a + t * W + c), y = ldf(b + t * W + c);
    qa += x * x;
    qb += y * y;
  }
  const float ra = 1.0f / sqrtf(block_sum(qa, red) / (float)W + eps);
  const float rb = 1.0f / sqrtf(block_sum(qb, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    stf(out + t * W + c, 0.5f * (ldf(a + t * W + c) * ra * ldf(wa + c) + ldf(b + t * W + c) * rb * ldf(wb + c)));
}

__global__ void __launch_bounds__(256) softcap_k(float* __restrict__ x, int64_t n, float cap) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] / cap);
}

}  // namespace

void layer_norm_pair_shift(bool bf16, const float* x, const void* w1, const void* w2, const float* mu, float eps,
                           float* state, const int32_t* cu, const int32_t* seq_of, const int32_t* slots,
                           const int64_t* pos, void* h1, void* h2, float* last, int T, int B, int W, bool single,
                           hipStream_t st) {
  if (T <= 0) return;
  if (bf16)
    ln_pair_shift_k<__bf16><<<T, 256, 0, st>>>(x, (const __bf16*)w1, (const __bf16*)w2, mu, eps, state, cu, seq_of, slots,
                                               pos, (__bf16*)h1, (__bf16*)h2, last, W, single);
  else
    ln_pair_shift_k<float><<<T, 256, 0, st>>>(x, (const float*)w1, (const float*)w2, mu, eps, state, cu, seq_of, slots,
                                              pos, (float*)h1, (float*)h2, last, W, single);
  if (mu && !single) rows_to_slots_k<<<B, 256, 0, st>>>(last, state, cu, slots, W);
}

void mingru_scan(bool bf16, const void* y, int64_t y_ld, int width, float* state, const int32_t* cu,
                 const int32_t* slots, const int64_t* pos, void* out, int B, int max_n, hipStream_t st) {
  if (B <= 0 || width <= 0) return;
  // pieces per portion: at least 16 tokens a piece, as many as fill the chip, at most 16
  const int64_t groups = (int64_t)B * ((width + 63) / 64);
  int nc = 1;
  while (nc < 16 && max_n >= 32 * nc && groups * nc < 1024) nc *= 2;
  const dim3 grid((width + 63) / 64, B), block(64 * nc);
  if (bf16)
    mingru_scan_k<__bf16><<<grid, block, 0, st>>>((const __bf16*)y, y_ld, width, state, cu, slots, pos, (__bf16*)out);
  else
    mingru_scan_k<float><<<grid, block, 0, st>>>((const float*)y, y_ld, width, state, cu, slots, pos, (float*)out);
}

void gla_scan(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
              const void* a, int64_t a_ld, float tau, float q_scale, float* S, const int32_t* cu, const int32_t* slots,
              const int64_t* pos, float* out, int B, int H, int d, int dv, hipStream_t st) {
  if (B <= 0 || d > kGlaMaxDim) return;                             // (sizes are refused by the caller beforehand)
  // state rows per wave: as few as fill the chip (the scan is sequential in time), at most 16 waves a workgroup
  const int64_t cols = (int64_t)B * H * ((dv + 63) / 64);
  int NS = 64;
  for (int ns = 8; ns <= 64; ns *= 2) {
    const int nw = (d + ns - 1) / ns;
    if (nw <= 16 && (ns == 64 || cols * ((d + 2 * ns - 1) / (2 * ns)) < 1024)) {
      NS = ns;
      break;
    }
  }
  const int NW = (d + NS - 1) / NS, NP = NW * NS;
  const size_t per_tok = ((size_t)3 * NP + 64 + (size_t)NW * 64) * sizeof(float);
  int TC = (int)((48 * 1024) / per_tok);
  TC = TC > 32 ? 32 : (TC < 1 ? 1 : TC);
  const size_t lds = per_tok * TC;
  const dim3 grid(B, H, (dv + 63) / 64), block(64 * NW);
#define GM_GLA_T(E, NSV, MT)                                                                                        \
  gla_scan_k<E, NSV, MT><<<grid, block, lds, st>>>((const E*)q, q_ld, (const E*)k, k_ld, (const E*)v, v_ld,          \
                                                   (const E*)a, a_ld, 1.0f / tau, q_scale, S, cu, slots, pos, out, H, \
                                                   d, dv, TC)
#define GM_GLA(E, NSV)                          \
  if (NW <= 4) GM_GLA_T(E, NSV, 256);           \
  else if (NW <= 8) GM_GLA_T(E, NSV, 512);      \
  else GM_GLA_T(E, NSV, 1024)
#define GM_GLA_NS(E)                     \
  if (NS == 8) { GM_GLA(E, 8); }         \
  else if (NS == 16) { GM_GLA(E, 16); }  \
  else if (NS == 32) { GM_GLA(E, 32); }  \
  else { GM_GLA(E, 64); }
  if (bf16) { GM_GLA_NS(__bf16); } else { GM_GLA_NS(float); }
#undef GM_GLA_NS
#undef GM_GLA
#undef GM_GLA_T
}

void gla_piece_decay(bool bf16, const void* a, int64_t a_ld, const int32_t* cu, float tau, float* P, int NP, int H, int d,
                     hipStream_t st) {
  if (NP <= 0) return;
  if (bf16) gla_piece_decay_k<__bf16><<<dim3(NP, H), 256, 0, st>>>((const __bf16*)a, a_ld, cu, 1.0f / tau, P, H, d);
  else gla_piece_decay_k<float><<<dim3(NP, H), 256, 0, st>>>((const float*)a, a_ld, cu, 1.0f / tau, P, H, d);
}

void gla_chain(const float* Z, float* Sin, const float* P, const int32_t* seqs, int nseq, int H, int d, int dv,
               hipStream_t st) {
  if (nseq <= 0) return;
  const int64_t n = (int64_t)H * d * dv;
  const int by = (int)((n + 255) / 256 > 1024 ? 1024 : (n + 255) / 256);
  gla_chain_k<<<dim3(nseq, by), 256, 0, st>>>(Z, Sin, P, seqs, H * d, dv);
}

void head_rms_silu(bool bf16, const float* o, const void* w, const void* gate, int64_t g_ld, void* out, int T, int H,
                   int dv, float eps, hipStream_t st) {
  if (T <= 0) return;
  if (bf16)
    head_rms_silu_k<__bf16><<<dim3(T, H), 64, 0, st>>>(o, (const __bf16*)w, (const __bf16*)gate, g_ld, (__bf16*)out, H, dv, eps);
  else
    head_rms_silu_k<float><<<dim3(T, H), 64, 0, st>>>(o, (const float*)w, (const float*)gate, g_ld, (float*)out, H, dv, eps);
}

void rms_pair_mean(bool bf16, const void* a, const void* b, const void* wa, const void* wb, void* out, int T, int W,
                   float eps, hipStream_t st) {
  if (T <= 0) return;
  if (bf16)
    rms_pair_mean_k<__bf16><<<T, 256, 0, st>>>((const __bf16*)a, (const __bf16*)b, (const __bf16*)wa, (const __bf16*)wb,
                                               (__bf16*)out, W, eps);
  else
    rms_pair_mean_k<float><<<T, 256, 0, st>>>((const float*)a, (const float*)b, (const float*)wa, (const float*)wb,
                                              (float*)out, W, eps);
}

void softcap(float* x, int64_t n, float cap, hipStream_t st) {
  if (n <= 0) return;
  const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
  softcap_k<<<blocks, 256, 0, st>>>(x, n, cap);
}

}  // namespace gm
}  // namespace illm
