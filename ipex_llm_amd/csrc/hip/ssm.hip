// Kernels of the state-space mixer (gfx950, wave64).
//
//   conv + SiLU        a thread per (token, channel); tokens before a portion's
//                      start come from the sequence's state slot, positions
//                      before 0 are zero; a second launch (or the same one at
//                      decode) leaves the portion's last inputs in the slot
//   selective scan     S' = a S + dt B x^T, y = S'^T C + D x.  One workgroup:
//                      64 value columns of one (sequence, head).  Wave w keeps
//                      the state rows [w NS, (w + 1) NS) of those columns in
//                      registers; tokens go through LDS in chunks (B and C
//                      rows zero padded to the waves' rows, the step sizes with
//                      their softplus and the decays computed once per chunk);
//                      every wave leaves a partial y per token and the partials
//                      are summed in a fixed order, so a result never depends
//                      on how the tokens were cut into steps.  The rows per
//                      wave (8 .. 64) are chosen so that the launch fills the
//                      chip: few sequences and heads -> more, thinner waves
//   gated group norm   y silu(z), every group divided by its root mean square
//
// Activations are bf16 or f32 (template E); accumulation is always f32.
#include "ssm.h"

#include <math.h>

namespace illm {
namespace ssm {
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
__device__ __forceinline__ float silu(float z) { return z / (1.0f + expf(-z)); }

constexpr int kMaxTaps = 16;

// ------------------------------------------------------------------ convolution
// V consecutive channels per thread (V = 4: 4-element accesses; the launcher checks sizes and alignment)
template <typename E, int V> struct LdV;
template <typename E> struct LdV<E, 1> {
  static __device__ __forceinline__ void ld(const E* p, float* v) { v[0] = ldf(p); }
};
template <> struct LdV<float, 4> {
  static __device__ __forceinline__ void ld(const float* p, float* v) {
    const float4 a = *(const float4*)p;
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
  }
};
template <> struct LdV<__bf16, 4> {
  typedef __bf16 B4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ void ld(const __bf16* p, float* v) {
    const B4 a = *(const B4*)p;
    v[0] = (float)a[0], v[1] = (float)a[1], v[2] = (float)a[2], v[3] = (float)a[3];
  }
};
template <int V> __device__ __forceinline__ void stv(float* p, const float* v);
template <> __device__ __forceinline__ void stv<1>(float* p, const float* v) { p[0] = v[0]; }
template <> __device__ __forceinline__ void stv<4>(float* p, const float* v) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
}

// bias may be null; ACT: SiLU on the result
template <typename E, int V, bool ACT>
__global__ void __launch_bounds__(256) conv_silu_k(const E* __restrict__ u, int64_t u_ld, const float* __restrict__ w,
                                                  const float* __restrict__ bias, int taps, float* __restrict__ state,
                                                  const int32_t* __restrict__ cu, const int32_t* __restrict__ seq_of,
                                                  const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                  float* __restrict__ out, int C, bool single) {
  const int t = blockIdx.x;
  const int c = V * (blockIdx.y * blockDim.x + threadIdx.x);
  if (c >= C) return;
  const int b = seq_of[t];
  const int i = t - cu[b];                                          // index inside the portion
  const int64_t p = pos[t];
  float* st = state + (int64_t)slots[b] * (taps - 1) * C + c;       // [taps - 1][C], oldest first
  float acc[V];
#pragma unroll
  for (int q = 0; q < V; q++) acc[q] = 0.f;
  if (bias) LdV<float, V>::ld(bias + c, acc);
  for (int j = 0; j < taps; j++) {
    const int back = taps - 1 - j;                                  // the input of position p - back
    float v[V];
#pragma unroll
    for (int q = 0; q < V; q++) v[q] = 0.f;
    if (back <= i) LdV<E, V>::ld(u + (int64_t)(t - back) * u_ld + c, v);
    else if (p - back >= 0) LdV<float, V>::ld(st + (int64_t)(taps - 1 + i - back) * C, v);
#pragma unroll
    for (int q = 0; q < V; q++) acc[q] = fmaf(w[(int64_t)(c + q) * taps + j], v[q], acc[q]);
  }
  if (ACT) {
#pragma unroll
    for (int q = 0; q < V; q++) acc[q] = silu(acc[q]);
  }
  stv<V>(out + (int64_t)t * C + c, acc);
  if (single && taps > 1) {
    // the only token of its sequence (i == 0): the slot moves up by one position; row j held position
    // p - (taps - 1 - j), positions before 0 are zero whatever the slot held
    for (int j = 1; j < taps - 1; j++) {
      float v[V];
#pragma unroll
      for (int q = 0; q < V; q++) v[q] = 0.f;
      if (p - (taps - 1 - j) >= 0) LdV<float, V>::ld(st + (int64_t)j * C, v);
      stv<V>(st + (int64_t)(j - 1) * C, v);
    }
    float v[V];
    LdV<E, V>::ld(u + (int64_t)t * u_ld + c, v);
    stv<V>(st + (int64_t)(taps - 2) * C, v);
  }
}

// after a portion of n tokens that started at position p0: the slot holds the inputs of positions p0 + n - taps + 1 ..
// p0 + n - 1 (zeros for positions before 0)
template <typename E>
__global__ void __launch_bounds__(256) conv_state_k(const E* __restrict__ u, int64_t u_ld, int taps,
                                                   float* __restrict__ state, const int32_t* __restrict__ cu,
                                                   const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                   int C) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  if (n <= 0) return;
  const int64_t p0 = pos[t0];
  float* st = state + (int64_t)slots[b] * (taps - 1) * C + c;
  float nv[kMaxTaps];
  for (int k = 0; k < taps - 1; k++) {
    const int64_t i = (int64_t)n - (taps - 1) + k;                  // index inside the portion of that position
    float v = 0.f;
    if (i >= 0) v = ldf(u + (int64_t)(t0 + i) * u_ld + c);
    else if (p0 + i >= 0) v = st[(int64_t)(k + n) * C];
    nv[k] = v;
  }
  for (int k = 0; k < taps - 1; k++) st[(int64_t)k * C] = nv[k];
}

// ------------------------------------------------------------------ scan
template <typename E, int NS>
__global__ void __launch_bounds__(1024) scan_k(
    const float* __restrict__ x, int64_t x_ld, const float* __restrict__ Bm, int64_t b_ld, const float* __restrict__ Cm,
    int64_t c_ld, const E* __restrict__ dtp, int64_t dt_ld, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip, float* __restrict__ S,
    const int32_t* __restrict__ cu, const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
    float* __restrict__ out, int H, int P, int G, int N, int TC) {
  extern __shared__ __align__(16) float sm[];
  const int b = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * 64;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  const int NP = NW * NS;
  const int t0 = cu[b], n = cu[b + 1] - t0;
  if (n <= 0) return;
  const int g = h / (H / G);
  const int pc = p0 + lane;
  float* Bs = sm;                                                   // [TC][NP]
  float* Cs = Bs + (size_t)TC * NP;                                 // [TC][NP]
  float* xs = Cs + (size_t)TC * NP;                                 // [TC][64]
  float* pt = xs + (size_t)TC * 64;                                 // [NW][TC][64]
  float* ds = pt + (size_t)NW * TC * 64;                            // [TC] step sizes, [TC] decays
  float st[NS];
  float* Sg = S + (((int64_t)slots[b] * H + h) * N) * P;            // [N][P]
  const bool fresh = pos[t0] == 0;
#pragma unroll
  for (int i = 0; i < NS; i++) {
    const int nn = wv * NS + i;
    st[i] = (!fresh && nn < N && pc < P) ? Sg[(int64_t)nn * P + pc] : 0.f;
  }
  const float rate = expf(a_log[h]), bias = dt_bias[h], dsk = d_skip[h];
  // a chunk's B / C / x / dt elements travel global -> registers -> LDS; the registers of the NEXT chunk are
  // requested before the current chunk's arithmetic, so their latency hides behind it (the host sizes TC so that
  // PE elements per thread and array cover a chunk)
  constexpr int PE = 4;
  float rb[PE], rc[PE], rx[PE], rdt = 0.f;
  auto fetch = [&](int c0) {
    const int nt = min(TC, n - c0);
#pragma unroll
    for (int k = 0; k < PE; k++) {
      const int i = threadIdx.x + k * blockDim.x;
      rb[k] = rc[k] = 0.f;
      if (i < nt * NP) {
        const int tk = i / NP, nn = i - tk * NP;
        const int64_t t = t0 + c0 + tk;
        if (nn < N) {
          rb[k] = Bm[t * b_ld + (int64_t)g * N + nn];
          rc[k] = Cm[t * c_ld + (int64_t)g * N + nn];
        }
      }
    }
#pragma unroll
    for (int k = 0; k < PE; k++) {
      const int i = threadIdx.x + k * blockDim.x;                   // (token i / 64, this lane's column)
      rx[k] = (i < nt * 64 && pc < P) ? x[(int64_t)(t0 + c0 + (i >> 6)) * x_ld + (int64_t)h * P + pc] : 0.f;
    }
    if (threadIdx.x < nt) rdt = ldf(dtp + (int64_t)(t0 + c0 + threadIdx.x) * dt_ld + h);
  };
  fetch(0);
  for (int c0 = 0; c0 < n; c0 += TC) {
    const int nt = min(TC, n - c0);
    __syncthreads();                                                // the last chunk's reads are done
#pragma unroll
    for (int k = 0; k < PE; k++) {
      const int i = threadIdx.x + k * blockDim.x;
      if (i < nt * NP) {
        Bs[i] = rb[k];
        Cs[i] = rc[k];
      }
    }
#pragma unroll
    for (int k = 0; k < PE; k++) {
      const int i = threadIdx.x + k * blockDim.x;
      if (i < nt * 64) xs[i] = rx[k];
    }
    if (threadIdx.x < nt) {
      const float z = rdt + bias;
      const float dt = z > 20.f ? z : log1pf(expf(z));              // softplus
      ds[threadIdx.x] = dt;
      ds[TC + threadIdx.x] = expf(-rate * dt);
    }
    __syncthreads();
    if (c0 + TC < n) fetch(c0 + TC);
    for (int tk = 0; tk < nt; tk++) {
      const float da = ds[TC + tk];
      const float dx = ds[tk] * xs[tk * 64 + lane];
      const float4* b4 = (const float4*)(Bs + (size_t)tk * NP + wv * NS);
      const float4* c4 = (const float4*)(Cs + (size_t)tk * NP + wv * NS);
      // y's sum over the state rows has one fixed shape, whatever NS is: units of 8 rows (four chains of two),
      // then a balanced pairwise tree over the units -- here over the wave's units, below over the waves
      float un[NS / 8];
#pragma unroll
      for (int u = 0; u < NS / 8; u++) {
        const float4 b0 = b4[2 * u], b1 = b4[2 * u + 1], c0v = c4[2 * u], c1v = c4[2 * u + 1];
        float* r = st + 8 * u;
        r[0] = fmaf(da, r[0], dx * b0.x);
        r[1] = fmaf(da, r[1], dx * b0.y);
        r[2] = fmaf(da, r[2], dx * b0.z);
        r[3] = fmaf(da, r[3], dx * b0.w);
        r[4] = fmaf(da, r[4], dx * b1.x);
        r[5] = fmaf(da, r[5], dx * b1.y);
        r[6] = fmaf(da, r[6], dx * b1.z);
        r[7] = fmaf(da, r[7], dx * b1.w);
        const float a0 = fmaf(r[4], c1v.x, r[0] * c0v.x), a1 = fmaf(r[5], c1v.y, r[1] * c0v.y);
        const float a2 = fmaf(r[6], c1v.z, r[2] * c0v.z), a3 = fmaf(r[7], c1v.w, r[3] * c0v.w);
        un[u] = (a0 + a1) + (a2 + a3);
      }
#pragma unroll
      for (int sft = 1; sft < NS / 8; sft *= 2)
#pragma unroll
        for (int u = 0; u + sft < NS / 8; u += 2 * sft) un[u] += un[u + sft];
      pt[((size_t)wv * TC + tk) * 64 + lane] = un[0];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nt * 64; i += blockDim.x) {
      const int tk = i >> 6, l = i & 63;
      if (p0 + l >= P) continue;
      float v[16];                                                  // the waves' partials, zeros past NW
#pragma unroll
      for (int w = 0; w < 16; w++) v[w] = w < NW ? pt[((size_t)w * TC + tk) * 64 + l] : 0.f;
#pragma unroll
      for (int sft = 1; sft < 16; sft *= 2)
#pragma unroll
        for (int w = 0; w + sft < 16; w += 2 * sft) v[w] += v[w + sft];
      out[((int64_t)(t0 + c0 + tk) * H + h) * P + p0 + l] = fmaf(dsk, xs[i], v[0]);
    }
  }
#pragma unroll
  for (int i = 0; i < NS; i++) {
    const int nn = wv * NS + i;
    if (nn < N && pc < P) Sg[(int64_t)nn * P + pc] = st[i];
  }
}

// ------------------------------------------------------------------ gate + group norm
template <typename E>
__global__ void __launch_bounds__(256) gated_group_norm_k(const float* __restrict__ y, const E* __restrict__ z, int64_t z_ld,
                                                         const E* __restrict__ w, E* __restrict__ out, int C, int gs,
                                                         float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  float q = 0.f;
  for (int c = threadIdx.x; c < gs; c += blockDim.x) {
    const float v = y[t * C + c0 + c] * silu(ldf(z + t * z_ld + c0 + c));
    q += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += blockDim.x) {
    const float v = y[t * C + c0 + c] * silu(ldf(z + t * z_ld + c0 + c));
    stf(out + t * C + c0 + c, v * rs * ldf(w + c0 + c));
  }
}

}  // namespace

void conv_silu(bool bf16, const void* u, int64_t u_ld, const float* w, const float* b, int taps, float* state,
               const int32_t* cu, const int32_t* seq_of, const int32_t* slots, const int64_t* pos, float* out, int T,
               int B, int C, bool single, bool act, hipStream_t st) {
  if (T <= 0 || C <= 0) return;
  const size_t eb = bf16 ? 2 : 4;
  const bool v4 = (C & 3) == 0 && (u_ld & 3) == 0 && ((uintptr_t)u % (4 * eb)) == 0;
  const int cw = v4 ? C / 4 : C;
  dim3 grid(T, (cw + 255) / 256), gs(B, (C + 255) / 256);
#define SSM_CONV(E, V)                                                                                               \
  if (act)                                                                                                           \
    conv_silu_k<E, V, true><<<grid, 256, 0, st>>>((const E*)u, u_ld, w, b, taps, state, cu, seq_of, slots, pos, out, \
                                                  C, single);                                                        \
  else                                                                                                               \
    conv_silu_k<E, V, false><<<grid, 256, 0, st>>>((const E*)u, u_ld, w, b, taps, state, cu, seq_of, slots, pos, out, \
                                                   C, single)
  if (bf16) {
    if (v4) { SSM_CONV(__bf16, 4); }
    else { SSM_CONV(__bf16, 1); }
    if (!single && taps > 1) conv_state_k<__bf16><<<gs, 256, 0, st>>>((const __bf16*)u, u_ld, taps, state, cu, slots, pos, C);
  } else {
    if (v4) { SSM_CONV(float, 4); }
    else { SSM_CONV(float, 1); }
    if (!single && taps > 1) conv_state_k<float><<<gs, 256, 0, st>>>((const float*)u, u_ld, taps, state, cu, slots, pos, C);
  }
#undef SSM_CONV
}

void selective_scan(bool bf16, const float* x, int64_t x_ld, const float* Bm, int64_t b_ld, const float* Cm,
                    int64_t c_ld, const void* dt, int64_t dt_ld, const float* dt_bias, const float* a_log,
                    const float* d_skip, float* S, const int32_t* cu, const int32_t* slots, const int64_t* pos,
                    float* out, int B, int H, int P, int G, int N, hipStream_t st) {
  if (B <= 0 || N > kScanMaxState) return;                          // (sizes are refused by the caller beforehand)
  // state rows per wave: as few as fill the chip -- the scan is sequential in time, so its only parallelism is
  // (sequence, head, 64 columns, wave); at most 16 waves a workgroup
  const int64_t cols = (int64_t)B * H * ((P + 63) / 64);
  int NS = 64;
  for (int ns = 8; ns <= 64; ns *= 2) {
    const int nw = (N + ns - 1) / ns;
    if (nw <= 16 && (ns == 64 || cols * ((N + 2 * ns - 1) / (2 * ns)) < 2048)) {
      NS = ns;
      break;
    }
  }
  const int NW = (N + NS - 1) / NS;
  const int NP = NW * NS;
  // tokens per chunk: B and C rows, x, the waves' partials and the step sizes within 48 KB; a thread stages at most
  // four elements of B, of C and of x per chunk (4 * 64 NW >= TC * NP and >= 64 TC)
  int TC = (48 * 1024 / 4) / (2 * NP + 64 + NW * 64 + 2);
  TC = TC > 16 ? 16 : TC;
  TC = TC > 256 / NS ? 256 / NS : TC;
  TC = TC > 4 * NW ? 4 * NW : TC;
  TC = TC < 1 ? 1 : TC;
  const size_t lds = ((size_t)TC * (2 * NP + 64 + NW * 64) + 2 * TC) * sizeof(float);
  dim3 grid(B, H, (P + 63) / 64), block(64 * NW);
#define SSM_SCAN(E, NSV)                                                                                              \
  scan_k<E, NSV><<<grid, block, lds, st>>>(x, x_ld, Bm, b_ld, Cm, c_ld, (const E*)dt, dt_ld, dt_bias, a_log, d_skip, S, \
                                           cu, slots, pos, out, H, P, G, N, TC)
  if (bf16) {
    if (NS == 8) SSM_SCAN(__bf16, 8);
    else if (NS == 16) SSM_SCAN(__bf16, 16);
    else if (NS == 32) SSM_SCAN(__bf16, 32);
    else SSM_SCAN(__bf16, 64);
  } else {
    if (NS == 8) SSM_SCAN(float, 8);
    else if (NS == 16) SSM_SCAN(float, 16);
    else if (NS == 32) SSM_SCAN(float, 32);
    else SSM_SCAN(float, 64);
  }
#undef SSM_SCAN
}

void gated_group_norm(bool bf16, const float* y, const void* z, int64_t z_ld, const void* w, void* out, int T, int C,
                      int groups, float eps, hipStream_t st) {
  if (T <= 0) return;
  dim3 grid(T, groups);
  if (bf16)
    gated_group_norm_k<__bf16><<<grid, 256, 0, st>>>(y, (const __bf16*)z, z_ld, (const __bf16*)w, (__bf16*)out, C,
                                                     C / groups, eps);
  else
    gated_group_norm_k<float><<<grid, 256, 0, st>>>(y, (const float*)z, z_ld, (const float*)w, (float*)out, C, C / groups,
                                                    eps);
}

}  // namespace ssm
}  // namespace illm
