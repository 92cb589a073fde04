// Experts behind a sigmoid router (gfx950, wave64).
//
//   moe_route_k    sigmoid scores, the `top` largest per token (lowest index
//                  first among equals) and those scores as weights; or the
//                  `top` largest logits and the softmax over them
//   moe_align_k    pair ids (token * top + k) grouped by expert + offsets,
//                  one workgroup, LDS counters: no host round trip, so a
//                  step with experts can be captured in a hipGraph
//   moe_gemm_k     grouped product over the sorted pairs: blockIdx.x walks
//                  (expert, row block), rows gathered through the pair list.
//                  GLU form: x = w_pair * h[token] (rounded to the activation
//                  type), y = g sigmoid(alpha g) (u + 1) with the clamps;
//                  DOWN form: f32 rows scattered back by pair id.
//                  bf16: 16x16x32 MFMA tiles with f32 accumulation
//                  (moe_gemm_mfma_k); f32, and sizes that are no multiple of
//                  8: vector FMAs.  A row's sum runs over k in one fixed order,
//                  so a token's result does not depend on its batch.
#include "blockmix.h"

#include <math.h>

namespace illm {
namespace bm {
namespace {

template <typename E> __device__ __forceinline__ float ldf(const E* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<__bf16>(const __bf16* p) { return (float)*p; }
template <typename E> __device__ __forceinline__ void stf(E* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<__bf16>(__bf16* p, float v) { *p = (__bf16)v; }
template <typename E> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<__bf16>(float v) { return (float)(__bf16)v; }

constexpr int kMaxPerLane = 8;      // experts <= 512

// SOFTMAX false: scores sigmoid(z), the largest win and are the weights; true: the largest logits win, their weights
// are the softmax over the winners only
template <bool SOFTMAX>
__global__ void __launch_bounds__(64) moe_route_k(const float* __restrict__ z, int E, int top, int32_t* __restrict__ idx,
                                                 float* __restrict__ w) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const float none = SOFTMAX ? -INFINITY : -1.0f;                   // below every score; a taken one goes below that
  float s[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; i++) {
    const int e = lane + i * 64;
    s[i] = e < E ? (SOFTMAX ? fmaxf(z[t * E + e], -3.0e38f) : 1.0f / (1.0f + expf(-z[t * E + e]))) : none;
  }
  float top0 = 0.f, den = 0.f, mine = 0.f;                          // SOFTMAX: lane k keeps winner k's weight (top <= 64)
  for (int k = 0; k < top; k++) {
    float bv = none;
    int be = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; i++) {
      const int e = lane + i * 64;
      if (s[i] > bv) {                               // ascending e within a lane: the first of equals stays
        bv = s[i];
        be = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oe = __shfl_xor(be, o, 64);
      if (ov > bv || (ov == bv && oe < be)) {
        bv = ov;
        be = oe;
      }
    }
    if (SOFTMAX) {                                                  // the first winner is the largest: exp(bv - top0) <= 1
      if (k == 0) top0 = bv;
      bv = expf(bv - top0);
      den += bv;
      if (lane == k) mine = bv;
    }
    if (lane == 0) {
      idx[t * top + k] = be;
      if (!SOFTMAX) w[t * top + k] = bv;
    }
#pragma unroll
    for (int i = 0; i < kMaxPerLane; i++)
      if (lane + i * 64 == be) s[i] = SOFTMAX ? -INFINITY : -2.0f;
  }
  if (SOFTMAX && lane < top) w[t * top + lane] = mine / den;
}

__global__ void __launch_bounds__(1024) moe_align_k(const int32_t* __restrict__ idx, int P, int E, int32_t* __restrict__ off,
                                                   int32_t* __restrict__ sorted) {
  extern __shared__ int cnt[];                       // [E] counters, then [E] cursors
  int* cur = cnt + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    int e = idx[p];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int a = 0;
    for (int e = 0; e < E; e++) {
      off[e] = a;
      cur[e] = a;
      a += cnt[e];
    }
    off[E] = a;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < P; p += blockDim.x) {
    int e = idx[p];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    sorted[atomicAdd(&cur[e], 1)] = p;
  }
}

constexpr int TM = 32, TN = 64, TK = 32;

// which (expert, block of tm rows) this workgroup serves; false: past the last one
__device__ __forceinline__ bool find_block(const int32_t* __restrict__ off, int E, int bx, int tm, int* e_out, int* r0,
                                           int* r1) {
  int acc = 0;
  for (int e = 0; e < E; e++) {
    const int lo = off[e], hi = off[e + 1];
    const int nb = (hi - lo + tm - 1) / tm;
    if (bx < acc + nb) {
      *e_out = e;
      *r0 = lo + (bx - acc) * tm;
      *r1 = hi < *r0 + tm ? hi : *r0 + tm;
      return true;
    }
    acc += nb;
  }
  return false;
}

// x rows: GLU: h[pair / top] * wts[pair]; DOWN: y[sorted position].  w: [E, (GLU ? 2 : 1) N, K].
template <typename E, bool GLU>
__global__ void __launch_bounds__(256) moe_gemm_k(const E* __restrict__ x, const int32_t* __restrict__ off,
                                                 const int32_t* __restrict__ sorted, const float* __restrict__ wts,
                                                 int top, const E* __restrict__ w, E* __restrict__ y,
                                                 float* __restrict__ outp, int nexp, int N, int K, float limit,
                                                 float alpha, float up_shift, bool weigh_out) {
  __shared__ float xs[TM][TK + 1];
  __shared__ float ws[TN][TK + 1];
  __shared__ float ws2[GLU ? TN : 1][TK + 1];
  __shared__ int src_row[TM];
  __shared__ float src_scale[TM];
  __shared__ int dst_row[TM];
  int e, r0, r1;
  if (!find_block(off, nexp, blockIdx.x, TM, &e, &r0, &r1)) return;
  const int tid = threadIdx.x;
  const int n0 = blockIdx.y * TN;
  if (tid < TM) {
    const int sp = r0 + tid;
    if (sp < r1) {
      const int pid = sorted[sp];
      src_row[tid] = GLU ? pid / top : sp;
      src_scale[tid] = (GLU != weigh_out) ? wts[pid] : 1.f;         // GLU: on the input; DOWN (weigh_out): on the result
      dst_row[tid] = GLU ? sp : pid;
    } else {
      src_row[tid] = -1;
      src_scale[tid] = 0.f;
      dst_row[tid] = -1;
    }
  }
  __syncthreads();
  const E* we = w + (int64_t)e * (GLU ? 2 : 1) * N * K;
  const int tx = tid & 15, ty = tid >> 4;          // 4 columns x 2 rows per thread
  float acc[2][4], acc2[2][4];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) acc[i][j] = acc2[i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += TK) {
    for (int i = tid; i < TM * TK; i += 256) {
      const int r = i / TK, c = i - r * TK;
      const int sr = src_row[r];
      float v = 0.f;
      if (sr >= 0 && k0 + c < K) {
        v = ldf(x + (int64_t)sr * K + k0 + c);
        if (GLU && !weigh_out) v = round_to<E>(v * src_scale[r]);
      }
      xs[r][c] = v;
    }
    for (int i = tid; i < TN * TK; i += 256) {
      const int r = i / TK, c = i - r * TK;
      const bool ok = n0 + r < N && k0 + c < K;
      ws[r][c] = ok ? ldf(we + (int64_t)(n0 + r) * K + k0 + c) : 0.f;
      if (GLU) ws2[r][c] = ok ? ldf(we + (int64_t)(N + n0 + r) * K + k0 + c) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int kk = 0; kk < TK; kk++) {
      float a[2], b[4], b2[4];
#pragma unroll
      for (int i = 0; i < 2; i++) a[i] = xs[ty * 2 + i][kk];
#pragma unroll
      for (int j = 0; j < 4; j++) {
        b[j] = ws[tx * 4 + j][kk];
        if (GLU) b2[j] = ws2[tx * 4 + j][kk];
      }
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          acc[i][j] += a[i] * b[j];
          if (GLU) acc2[i][j] += a[i] * b2[j];
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int dr = dst_row[ty * 2 + i];
    if (dr < 0) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      if (GLU) {
        // the products leave the matrix unit in the activation type, as a library product's would
        const float g = fminf(round_to<E>(acc[i][j]), limit);
        const float u = fminf(fmaxf(round_to<E>(acc2[i][j]), -limit), limit);
        stf(y + (int64_t)dr * N + n, g / (1.0f + expf(-alpha * g)) * (u + up_shift));
      } else {
        outp[(int64_t)dr * N + n] = weigh_out ? acc[i][j] * src_scale[ty * 2 + i] : acc[i][j];
      }
    }
  }
}


// ---- bf16 on the matrix cores: 16x16x32 MFMA tiles, f32 accumulation.  A workgroup serves TMM gathered rows x 64
// columns; wave w owns columns 16 w .. 16 w + 15 and reads its weight fragments straight from memory (every weight
// element is used by exactly one wave of the workgroup, for all its row tiles); the gathered, scaled rows go through LDS.
typedef __bf16 bm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float bm_f32x4 __attribute__((ext_vector_type(4)));

template <int TMM, bool GLU>
__global__ void __launch_bounds__(256) moe_gemm_mfma_k(const __bf16* __restrict__ x, const int32_t* __restrict__ off,
                                                      const int32_t* __restrict__ sorted, const float* __restrict__ wts,
                                                      int top, const __bf16* __restrict__ w, __bf16* __restrict__ y,
                                                      float* __restrict__ outp, int nexp, int N, int K, float limit,
                                                      float alpha, float up_shift, bool weigh_out) {
  constexpr int TKK = 64, AP = TKK + 8, MS = TMM / 16;
  __shared__ __attribute__((aligned(16))) __bf16 as[TMM * AP];
  __shared__ int src_row[TMM];
  __shared__ float src_scale[TMM];
  __shared__ int dst_row[TMM];
  int e, r0, r1;
  if (!find_block(off, nexp, blockIdx.x, TMM, &e, &r0, &r1)) return;
  const int tid = threadIdx.x, wv = tid >> 6, lane = tid & 63, r16 = lane & 15, g = lane >> 4;
  if (tid < TMM) {
    const int sp = r0 + tid;
    if (sp < r1) {
      const int pid = sorted[sp];
      src_row[tid] = GLU ? pid / top : sp;
      src_scale[tid] = (GLU != weigh_out) ? wts[pid] : 1.f;         // GLU: on the input; DOWN (weigh_out): on the result
      dst_row[tid] = GLU ? sp : pid;
    } else {
      src_row[tid] = -1;
      src_scale[tid] = 0.f;
      dst_row[tid] = -1;
    }
  }
  __syncthreads();
  const int col = blockIdx.y * 64 + wv * 16 + r16;
  const bool col_ok = col < N;
  const __bf16* we = w + (int64_t)e * (GLU ? 2 : 1) * N * K;
  const __bf16* wg = we + (int64_t)(col_ok ? col : 0) * K;
  const __bf16* wu = we + (int64_t)(N + (col_ok ? col : 0)) * K;
  bm_f32x4 acc[MS], acc2[GLU ? MS : 1];
#pragma unroll
  for (int m = 0; m < MS; m++) {
    acc[m] = bm_f32x4{0.f, 0.f, 0.f, 0.f};
    if (GLU) acc2[m] = bm_f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const bm_bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  // the next k step's operands (gathered row pieces, this wave's weight fragments) are requested before the
  // current step's products and used after them
  constexpr int NA = TMM * 8 / 256;
  bm_bf16x8 pa[NA], pb[2], pb2[2];
  auto request = [&](int k0) {
#pragma unroll
    for (int it = 0; it < NA; it++) {
      const int c = tid + 256 * it;
      const int r = c >> 3, kc = (c & 7) * 8;
      const int sr = src_row[r];
      pa[it] = zero8;
      if (sr >= 0 && k0 + kc < K) pa[it] = *(const bm_bf16x8*)(x + (int64_t)sr * K + k0 + kc);
    }
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      const int kk = k0 + ks * 32 + 8 * g;
      const bool ok = col_ok && kk < K;
      pb[ks] = ok ? *(const bm_bf16x8*)(wg + kk) : zero8;
      pb2[ks] = zero8;
      if (GLU && ok) pb2[ks] = *(const bm_bf16x8*)(wu + kk);
    }
  };
  request(0);
  for (int k0 = 0; k0 < K; k0 += TKK) {
#pragma unroll
    for (int it = 0; it < NA; it++) {
      const int c = tid + 256 * it;
      const int r = c >> 3, kc = (c & 7) * 8;
      bm_bf16x8 v = pa[it];
      if (GLU && !weigh_out) {
        const float sc = src_scale[r];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (__bf16)((float)v[i] * sc);
      }
      *(bm_bf16x8*)(as + r * AP + kc) = v;
    }
    bm_bf16x8 b[2], b2[2];
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
      b[ks] = pb[ks];
      b2[ks] = pb2[ks];
    }
    __syncthreads();
    if (k0 + TKK < K) request(k0 + TKK);
#pragma unroll
    for (int ks = 0; ks < 2; ks++) {
#pragma unroll
      for (int m = 0; m < MS; m++) {
        const bm_bf16x8 a = *(const bm_bf16x8*)(as + (m * 16 + r16) * AP + ks * 32 + 8 * g);
        acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b[ks], acc[m], 0, 0, 0);
        if (GLU) acc2[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b2[ks], acc2[m], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  if (!col_ok) return;
#pragma unroll
  for (int m = 0; m < MS; m++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int dr = dst_row[m * 16 + 4 * g + i];
      if (dr < 0) continue;
      if (GLU) {
        const float gt = fminf((float)(__bf16)acc[m][i], limit);
        const float u = fminf(fmaxf((float)(__bf16)acc2[m][i], -limit), limit);
        y[(int64_t)dr * N + col] = (__bf16)(gt / (1.0f + expf(-alpha * gt)) * (u + up_shift));
      } else {
        outp[(int64_t)dr * N + col] = weigh_out ? acc[m][i] * src_scale[m * 16 + 4 * g + i] : acc[m][i];
      }
    }
  }
}

}  // namespace

void moe_route(const float* z, int T, int E, int top, int32_t* idx, float* w, int mode, hipStream_t st) {
  if (T <= 0) return;
  if (mode == 1) moe_route_k<true><<<T, 64, 0, st>>>(z, E, top, idx, w);
  else moe_route_k<false><<<T, 64, 0, st>>>(z, E, top, idx, w);
}

void moe_align(const int32_t* idx, int P, int E, int32_t* off, int32_t* sorted, hipStream_t st) {
  moe_align_k<<<1, 1024, (size_t)2 * E * sizeof(int), st>>>(idx, P, E, off, sorted);
}

void moe_glu(bool bf16, const void* h, const int32_t* off, const int32_t* sorted, const float* wts, int top,
             const void* w_gu, void* y, int P, int E, int ff, int W, float limit, float alpha, float up_shift,
             bool weigh_out, hipStream_t st) {
  if (P <= 0) return;
  const dim3 grid((P + TM - 1) / TM + E, (ff + TN - 1) / TN);
  if (bf16 && W % 8 == 0) {
    if (P / E >= 64)
      moe_gemm_mfma_k<128, true><<<dim3((P + 127) / 128 + E, (ff + 63) / 64), 256, 0, st>>>(
          (const __bf16*)h, off, sorted, wts, top, (const __bf16*)w_gu, (__bf16*)y, nullptr, E, ff, W, limit, alpha, up_shift,
          weigh_out);
    else
      moe_gemm_mfma_k<32, true><<<dim3((P + 31) / 32 + E, (ff + 63) / 64), 256, 0, st>>>(
          (const __bf16*)h, off, sorted, wts, top, (const __bf16*)w_gu, (__bf16*)y, nullptr, E, ff, W, limit, alpha, up_shift,
          weigh_out);
  } else if (bf16)
    moe_gemm_k<__bf16, true><<<grid, 256, 0, st>>>((const __bf16*)h, off, sorted, wts, top, (const __bf16*)w_gu,
                                                   (__bf16*)y, nullptr, E, ff, W, limit, alpha, up_shift, weigh_out);
  else
    moe_gemm_k<float, true><<<grid, 256, 0, st>>>((const float*)h, off, sorted, wts, top, (const float*)w_gu, (float*)y,
                                                  nullptr, E, ff, W, limit, alpha, up_shift, weigh_out);
}

void moe_down(bool bf16, const void* y, const int32_t* off, const int32_t* sorted, const void* w_down, float* out,
              int P, int E, int ff, int W, const float* wts, hipStream_t st) {
  const bool wo = wts != nullptr;                                   // the routing weight multiplies the result row
  if (P <= 0) return;
  const dim3 grid((P + TM - 1) / TM + E, (W + TN - 1) / TN);
  if (bf16 && ff % 8 == 0) {
    if (P / E >= 64)
      moe_gemm_mfma_k<128, false><<<dim3((P + 127) / 128 + E, (W + 63) / 64), 256, 0, st>>>(
          (const __bf16*)y, off, sorted, wts, 1, (const __bf16*)w_down, nullptr, out, E, W, ff, 0.f, 0.f, 0.f, wo);
    else
      moe_gemm_mfma_k<32, false><<<dim3((P + 31) / 32 + E, (W + 63) / 64), 256, 0, st>>>(
          (const __bf16*)y, off, sorted, wts, 1, (const __bf16*)w_down, nullptr, out, E, W, ff, 0.f, 0.f, 0.f, wo);
  } else if (bf16)
    moe_gemm_k<__bf16, false><<<grid, 256, 0, st>>>((const __bf16*)y, off, sorted, wts, 1, (const __bf16*)w_down,
                                                    nullptr, out, E, W, ff, 0.f, 0.f, 0.f, wo);
  else
    moe_gemm_k<float, false><<<grid, 256, 0, st>>>((const float*)y, off, sorted, wts, 1, (const float*)w_down,
                                                   nullptr, out, E, W, ff, 0.f, 0.f, 0.f, wo);
}

}  // namespace bm
}  // namespace illm
