// Element-wise kernels of the parallel-residual hybrid blocks (gfx950, wave64):
// RMS norm with one number or a vector, RMS-norm-on-output residual add, the
// scaled sum of two sublayers into the f32 residual stream, the short causal
// convolution in front of a mixer with its per-sequence state, squared ReLU,
// the clamped GLU and the token-side gate.
//
// Activations are bf16 or f32 (template E); all arithmetic is f32.
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

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// sum over a block of up to 1024 threads; red: >= 16 floats of LDS
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

template <typename E>
__global__ void __launch_bounds__(1024) rms_norm_rows_k(const float* __restrict__ x, const E* __restrict__ w, int nw,
                                                      float* __restrict__ h, E* __restrict__ ha, int W, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) q += xr[c] * xr[c];
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  const float w0 = ldf(w);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = xr[c] * rs * (nw == 1 ? w0 : ldf(w + c));
    h[t * W + c] = v;
    if (ha) stf(ha + t * W + c, v);
  }
}

template <typename E>
__global__ void __launch_bounds__(1024) add_rms_norm_k(float* __restrict__ x, const E* __restrict__ y,
                                                     const E* __restrict__ w, E* __restrict__ xa, int W, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const E* yr = y + t * W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = ldf(yr + c);
    q += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  float* xr = x + t * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = xr[c] + ldf(yr + c) * rs * ldf(w + c);
    xr[c] = v;
    if (xa) stf(xa + t * W + c, v);
  }
}

// four consecutive values as one access
template <typename E> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void ld(const float* p, float* v) {
    const float4 a = *(const float4*)p;
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
  }
  static __device__ __forceinline__ void st(float* p, const float* v) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
};
template <> struct Vec4<__bf16> {
  typedef __bf16 B4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ void ld(const __bf16* p, float* v) {
    const B4 a = *(const B4*)p;
    v[0] = (float)a[0], v[1] = (float)a[1], v[2] = (float)a[2], v[3] = (float)a[3];
  }
  static __device__ __forceinline__ void st(__bf16* p, const float* v) {
    B4 a;
    a[0] = (__bf16)v[0], a[1] = (__bf16)v[1], a[2] = (__bf16)v[2], a[3] = (__bf16)v[3];
    *(B4*)p = a;
  }
};

// x += y (y may be null), then out = x / sqrt(mean(x^2) + eps) * w: one sublayer's residual sum and the next norm.
// Rows whose length is a multiple of 4 move as 4-value accesses and stay in registers between the two passes
// (up to 16 values a thread; longer rows read the rest back).
template <typename E>
__global__ void __launch_bounds__(1024) add_rms_norm_rows_k(float* __restrict__ x, const E* __restrict__ y,
                                                          const E* __restrict__ w, E* __restrict__ out, int W, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  float* xr = x + t * W;
  float q = 0.f;
  if ((W & 3) == 0) {
    const int W4 = W >> 2, bd = blockDim.x;
    float keep[4][4];
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const int c = 4 * (threadIdx.x + k * bd);
      if (c < W) {
        float v[4], a[4];
        Vec4<float>::ld(xr + c, v);
        if (y) {
          Vec4<E>::ld(y + t * W + c, a);
#pragma unroll
          for (int i = 0; i < 4; i++) v[i] += a[i];
          Vec4<float>::st(xr + c, v);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
          keep[k][i] = v[i];
          q += v[i] * v[i];
        }
      }
    }
    for (int c4 = threadIdx.x + 4 * bd; c4 < W4; c4 += bd) {
      float v[4], a[4];
      Vec4<float>::ld(xr + 4 * c4, v);
      if (y) {
        Vec4<E>::ld(y + t * W + 4 * c4, a);
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] += a[i];
        Vec4<float>::st(xr + 4 * c4, v);
      }
#pragma unroll
      for (int i = 0; i < 4; i++) q += v[i] * v[i];
    }
    const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const int c = 4 * (threadIdx.x + k * bd);
      if (c < W) {
        float g[4], o[4];
        Vec4<E>::ld(w + c, g);
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = keep[k][i] * rs * g[i];
        Vec4<E>::st(out + t * W + c, o);
      }
    }
    for (int c4 = threadIdx.x + 4 * bd; c4 < W4; c4 += bd) {
      float v[4], g[4], o[4];
      Vec4<float>::ld(xr + 4 * c4, v);                              // own writes
      Vec4<E>::ld(w + 4 * c4, g);
#pragma unroll
      for (int i = 0; i < 4; i++) o[i] = v[i] * rs * g[i];
      Vec4<E>::st(out + t * W + 4 * c4, o);
    }
    return;
  }
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = xr[c];
    if (y) {
      v += ldf(y + t * W + c);
      xr[c] = v;
    }
    q += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(out + t * W + c, xr[c] * rs * ldf(w + c));   // own writes
}

template <typename E>
__global__ void __launch_bounds__(256) residual_add_scaled_k(float* __restrict__ x, const E* __restrict__ y1,
                                                            const float* __restrict__ s1, const void* __restrict__ y2,
                                                            bool y2_f32, const E* __restrict__ y3,
                                                            const float* __restrict__ s2, E* __restrict__ xa, int64_t n,
                                                            int W) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % W);
    float d = ldf(y1 + i) * (s1 ? s1[c] : 1.f);
    if (y2 || y3) {
      float f = 0.f;
      if (y2) f = y2_f32 ? ((const float*)y2)[i] : ldf((const E*)y2 + i);
      if (y3) f += ldf(y3 + i);
      d += f * (s2 ? s2[c] : 1.f);
    }
    const float v = x[i] + d;
    x[i] = v;
    if (xa) stf(xa + i, v);
  }
}

// one block per token: out_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j); inputs before the portion come from the
// sequence's state rows (positions p0 - taps + 1 .. p0 - 1, oldest first), inputs before position 0 are zero
template <typename E>
__global__ void __launch_bounds__(256) canon_conv_k(const float* __restrict__ h, const float* __restrict__ w, int taps,
                                                   const float* __restrict__ state, const int32_t* __restrict__ cu,
                                                   const int32_t* __restrict__ seq_of, const int32_t* __restrict__ slots,
                                                   const int64_t* __restrict__ pos, E* __restrict__ out, int W) {
  const int64_t t = blockIdx.x;
  const int b = seq_of[t];
  const int64_t t_start = cu[b];
  const int64_t p = pos[t], p0 = p - (t - t_start);
  const float* st = state + (int64_t)slots[b] * (taps - 1) * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float acc = h[t * W + c];
    for (int j = 0; j < taps; j++) {
      const int64_t sp = p - (taps - 1) + j;
      float v = 0.f;
      if (sp >= p0) v = h[(t - (p - sp)) * W + c];
      else if (sp >= 0) v = st[(sp - (p0 - (taps - 1))) * W + c];
      acc += w[c * taps + j] * v;
    }
    stf(out + t * W + c, acc);
  }
}

// one block per sequence, after canon_conv_k: the state becomes the inputs of the sequence's last taps - 1 positions
constexpr int kMaxHist = 15;
__global__ void __launch_bounds__(256) canon_state_k(const float* __restrict__ h, int taps, float* __restrict__ state,
                                                    const int32_t* __restrict__ cu, const int32_t* __restrict__ slots,
                                                    const int64_t* __restrict__ pos, int W) {
  const int b = blockIdx.x;
  const int64_t t0 = cu[b], n = cu[b + 1] - t0;
  if (n <= 0) return;
  const int64_t p0 = pos[t0];
  const int nh = taps - 1;
  float* st = state + (int64_t)slots[b] * nh * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float keep[kMaxHist];
#pragma unroll
    for (int i = 0; i < kMaxHist; i++) {
      if (i < nh) {
        const int64_t idx = n + i;                 // index into [old state | new inputs]
        if (idx >= nh) keep[i] = h[(t0 + idx - nh) * W + c];
        else keep[i] = (p0 - nh + idx >= 0) ? st[idx * W + c] : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < kMaxHist; i++)
      if (i < nh) st[i * W + c] = keep[i];
  }
}

// RMS norm + the convolution in one launch, one block per token: h_t = x_t / rms(x_t) * g and
// out_t = h_t + sum_j w[:, j] h_(t - taps + 1 + j).  The block norms its own row and recomputes the norms of the
// earlier rows of its portion that the taps reach (same formula and reduction order as for their own blocks);
// what lies before the portion comes from the state.  ``single``: every sequence brings one token, so the block
// is the only reader of its sequence's state and advances it itself; otherwise canon_state_k follows.
constexpr int kMaxTaps = 16;
template <typename E>
__global__ void __launch_bounds__(1024) norm_canon_k(const float* __restrict__ x, const E* __restrict__ g, int ng,
                                                   float eps, const float* __restrict__ w, int taps,
                                                   float* __restrict__ state, const int32_t* __restrict__ cu,
                                                   const int32_t* __restrict__ seq_of, const int32_t* __restrict__ slots,
                                                   const int64_t* __restrict__ pos, float* __restrict__ h,
                                                   E* __restrict__ ha, E* __restrict__ out, int W, int single) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int b = seq_of[t];
  const int64_t t_start = cu[b];
  const int64_t p = pos[t], p0 = p - (t - t_start);
  const int nh = taps - 1;
  float* st = state + (int64_t)slots[b] * nh * W;
  float rs[kMaxTaps];
#pragma unroll
  for (int r = 0; r < kMaxTaps; r++) {
    rs[r] = 0.f;
    if (r < taps && p - r >= p0) {                  // uniform over the block
      const float* xr = x + (t - r) * W;
      float q = 0.f;
      for (int c = threadIdx.x; c < W; c += blockDim.x) q += xr[c] * xr[c];
      rs[r] = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
    }
  }
  const float g0 = ldf(g);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float gc = ng == 1 ? g0 : ldf(g + c);
    const float own = x[t * W + c] * rs[0] * gc;
    float acc = own;
    float keep[kMaxTaps];
#pragma unroll
    for (int r = 0; r < kMaxTaps; r++) {
      if (r < taps) {
        const int64_t sp = p - r;                   // the tap r positions back: weight column taps - 1 - r
        float v = 0.f;
        if (r == 0) v = own;
        else if (sp >= p0) v = x[(t - r) * W + c] * rs[r] * gc;
        else if (sp >= 0) v = st[(sp - (p0 - nh)) * W + c];
        keep[r] = v;
        acc += w[c * taps + (taps - 1 - r)] * v;
      }
    }
    h[t * W + c] = own;
    if (ha) stf(ha + t * W + c, own);
    stf(out + t * W + c, acc);
    if (single) {                                   // new state: positions p - nh + 1 .. p, oldest first
#pragma unroll
      for (int r = 0; r < kMaxTaps - 1; r++)
        if (r < nh) st[(nh - 1 - r) * W + c] = keep[r];
    }
  }
}

template <typename E>
__global__ void __launch_bounds__(256) relu_sq_k(const E* __restrict__ y, E* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float v = fmaxf(ldf(y + i), 0.f);
    stf(out + i, v * v);
  }
}

template <typename E>
__global__ void __launch_bounds__(256) glu_clamp_k(const E* __restrict__ gu, E* __restrict__ out, int64_t T, int64_t I,
                                                  float limit, float alpha) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < T * I; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / I, c = i - t * I;
    const float g = fminf(ldf(gu + t * 2 * I + c), limit);
    const float u = fminf(fmaxf(ldf(gu + t * 2 * I + I + c), -limit), limit);
    stf(out + i, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

template <typename E>
__global__ void __launch_bounds__(256) side_gate_k(const E* __restrict__ z, const E* __restrict__ table, int64_t ld,
                                                  int64_t vocab, const int64_t* __restrict__ ids, int offset,
                                                  E* __restrict__ out, int T, int n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (int64_t)T * n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / n, c = i - t * n;
    const int64_t id = ids[t];
    const float e = (id >= 0 && id < vocab) ? ldf(table + id * ld + offset + c) : 0.f;
    const float v = ldf(z + i);
    const float a = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    stf(out + i, a * e);
  }
}

// threads of a one-row-per-block kernel.  Few rows (decode): a thread per channel or two, since a thread's loads
// are dependent and the launch is latency-bound; many rows: 256, several blocks per CU
int row_threads(int W, int T) {
  if (T > 64) return 256;
  return W >= 1024 ? 1024 : (W <= 64 ? 64 : (W + 63) / 64 * 64);
}
int grid_for(int64_t n) { return (int)((n + 255) / 256 < 1 ? 1 : ((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256)); }

}  // namespace

void rms_norm_rows(bool bf16, const float* x, const void* w, int nw, float* h, void* ha, int T, int W, float eps,
                   hipStream_t st) {
  if (T <= 0) return;
  if (bf16) rms_norm_rows_k<__bf16><<<T, row_threads(W, T), 0, st>>>(x, (const __bf16*)w, nw, h, (__bf16*)ha, W, eps);
  else rms_norm_rows_k<float><<<T, row_threads(W, T), 0, st>>>(x, (const float*)w, nw, h, nullptr, W, eps);
}

void add_rms_norm(bool bf16, float* x, const void* y, const void* w, void* xa, int T, int W, float eps, hipStream_t st) {
  if (T <= 0) return;
  if (bf16) add_rms_norm_k<__bf16><<<T, row_threads(W, T), 0, st>>>(x, (const __bf16*)y, (const __bf16*)w, (__bf16*)xa, W, eps);
  else add_rms_norm_k<float><<<T, row_threads(W, T), 0, st>>>(x, (const float*)y, (const float*)w, nullptr, W, eps);
}

void add_rms_norm_rows(bool bf16, float* x, const void* y, const void* w, void* out, int T, int W, float eps,
                       hipStream_t st) {
  if (T <= 0) return;
  if (bf16)
    add_rms_norm_rows_k<__bf16><<<T, row_threads(W, T), 0, st>>>(x, (const __bf16*)y, (const __bf16*)w, (__bf16*)out, W, eps);
  else
    add_rms_norm_rows_k<float><<<T, row_threads(W, T), 0, st>>>(x, (const float*)y, (const float*)w, (float*)out, W, eps);
}

void residual_add_scaled(bool bf16, float* x, const void* y1, const float* s1, const void* y2, bool y2_f32,
                         const void* y3, const float* s2, void* xa, int64_t T, int W, hipStream_t st) {
  const int64_t n = T * W;
  if (n <= 0) return;
  if (bf16)
    residual_add_scaled_k<__bf16><<<grid_for(n), 256, 0, st>>>(x, (const __bf16*)y1, s1, y2, y2_f32, (const __bf16*)y3,
                                                               s2, (__bf16*)xa, n, W);
  else
    residual_add_scaled_k<float><<<grid_for(n), 256, 0, st>>>(x, (const float*)y1, s1, y2, true, (const float*)y3, s2,
                                                              nullptr, n, W);
}

void canon_conv(bool bf16, const float* h, const float* w, int taps, float* state, const int32_t* cu,
                const int32_t* seq_of, const int32_t* slots, const int64_t* pos, void* out, int T, int B, int W,
                hipStream_t st) {
  if (T <= 0) return;
  if (bf16) canon_conv_k<__bf16><<<T, 256, 0, st>>>(h, w, taps, state, cu, seq_of, slots, pos, (__bf16*)out, W);
  else canon_conv_k<float><<<T, 256, 0, st>>>(h, w, taps, state, cu, seq_of, slots, pos, (float*)out, W);
  canon_state_k<<<B, 256, 0, st>>>(h, taps, state, cu, slots, pos, W);
}

void norm_canon(bool bf16, const float* x, const void* g, int ng, float eps, const float* w, int taps, float* state,
                const int32_t* cu, const int32_t* seq_of, const int32_t* slots, const int64_t* pos, float* h, void* ha,
                void* out, int T, int B, int W, bool single, hipStream_t st) {
  if (T <= 0) return;
  if (bf16)
    norm_canon_k<__bf16><<<T, row_threads(W, T), 0, st>>>(x, (const __bf16*)g, ng, eps, w, taps, state, cu, seq_of, slots, pos, h,
                                            (__bf16*)ha, (__bf16*)out, W, single ? 1 : 0);
  else
    norm_canon_k<float><<<T, row_threads(W, T), 0, st>>>(x, (const float*)g, ng, eps, w, taps, state, cu, seq_of, slots, pos, h,
                                           nullptr, (float*)out, W, single ? 1 : 0);
  if (!single) canon_state_k<<<B, 256, 0, st>>>(h, taps, state, cu, slots, pos, W);
}

void relu_sq(bool bf16, const void* y, void* out, int64_t n, hipStream_t st) {
  if (n <= 0) return;
  if (bf16) relu_sq_k<__bf16><<<grid_for(n), 256, 0, st>>>((const __bf16*)y, (__bf16*)out, n);
  else relu_sq_k<float><<<grid_for(n), 256, 0, st>>>((const float*)y, (float*)out, n);
}

void glu_clamp(bool bf16, const void* gu, void* out, int64_t T, int64_t I, float limit, float alpha, hipStream_t st) {
  if (T * I <= 0) return;
  if (bf16) glu_clamp_k<__bf16><<<grid_for(T * I), 256, 0, st>>>((const __bf16*)gu, (__bf16*)out, T, I, limit, alpha);
  else glu_clamp_k<float><<<grid_for(T * I), 256, 0, st>>>((const float*)gu, (float*)out, T, I, limit, alpha);
}

void side_gate(bool bf16, const void* z, const void* table, int64_t ld, int64_t vocab, const int64_t* ids, int offset,
               void* out, int T, int n, hipStream_t st) {
  if ((int64_t)T * n <= 0) return;
  if (bf16)
    side_gate_k<__bf16><<<grid_for((int64_t)T * n), 256, 0, st>>>((const __bf16*)z, (const __bf16*)table, ld, vocab, ids,
                                                                   offset, (__bf16*)out, T, n);
  else
    side_gate_k<float><<<grid_for((int64_t)T * n), 256, 0, st>>>((const float*)z, (const float*)table, ld, vocab, ids,
                                                                 offset, (float*)out, T, n);
}

}  // namespace bm
}  // namespace illm
