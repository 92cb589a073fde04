// Sequence-mixing kernels of the hybrid decoders (gfx950, wave64).
//
//   latent attention   one cached row per token [latent c (r) | rotated key
//                      (dr)], shared by all heads; scores, softmax and the
//                      weighted sum of latents in f32; ragged batches (every
//                      token carries its sequence and position), paged rows
//   mLSTM scan         matrix memory S [d, dv] + normaliser n [d] + running
//                      maximum m per (sequence, head), f32, carried in state
//                      slots between steps; token-sequential inside a step
//   element-wise       hashed-bigram embedding, scaled LayerNorm-on-output
//                      residual add (f32 stream), latent RMSNorm + rotary +
//                      cache append, rotary on query rows, per-head RMSNorm *
//                      weight * sigmoid gate, tanh-GELU GLU
//
// Activations are bf16 or f32 (template E); accumulation is always f32.
#include "seqmix.h"

#include <math.h>
#include <stdlib.h>

namespace illm {
namespace sm {
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
// LDS written by some lanes of a wave becomes visible to its other lanes
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
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

// ------------------------------------------------------------------ embedding
template <typename E>
__global__ void __launch_bounds__(256) embed_bigram_k(const int64_t* __restrict__ ids, const int64_t* __restrict__ prev,
                                                     const E* __restrict__ embed, const E* __restrict__ bigram,
                                                     float* __restrict__ out, int W, int64_t vocab, int64_t buckets,
                                                     int64_t mp, int64_t mc) {
  const int t = blockIdx.x;
  const int64_t id = ids[t], p = prev[t];
  float* o = out + (int64_t)t * W;
  if (id < 0 || id >= vocab) {                    // bad id: a zero row, never an out-of-bounds read
    for (int c = threadIdx.x; c < W; c += blockDim.x) o[c] = 0.f;
    return;
  }
  const int64_t row = p < 0 ? buckets : ((p * mp + id * mc) % buckets);
  const E* e = embed + id * W;
  const E* b = bigram + row * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) o[c] = ldf(e + c) + ldf(b + c);
}

// ------------------------------------------------------------------ norms
template <typename E>
__global__ void __launch_bounds__(256) add_sln_k(float* __restrict__ x, const E* __restrict__ y, const E* __restrict__ w,
                                                E* __restrict__ xa, int W, float eps, float mult) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const E* yr = y + t * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += ldf(yr + c);
  const float mean = block_sum(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = ldf(yr + c) - mean;
    q += d * d;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  float* xr = x + t * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = xr[c] + mult * ((ldf(yr + c) - mean) * rs * ldf(w + c));
    xr[c] = v;
    if (xa) stf(xa + t * W + c, v);
  }
}

template <typename E>
__global__ void __launch_bounds__(256) layer_norm_k(const float* __restrict__ x, const E* __restrict__ w,
                                                   E* __restrict__ out, int W, float eps) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const float* xr = x + t * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += xr[c];
  const float mean = block_sum(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = xr[c] - mean;
    q += d * d;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) stf(out + t * W + c, (xr[c] - mean) * rs * ldf(w + c));
}

// ------------------------------------------------------------------ rotary
template <typename E>
__global__ void __launch_bounds__(256) rope_rows_k(E* __restrict__ q, int H, int Dh, int offset,
                                                  const float* __restrict__ table, int max_pos, int dims,
                                                  const int64_t* __restrict__ pos) {
  const int64_t t = blockIdx.x;
  const int64_t p = pos[t];
  if (p < 0 || p >= max_pos) return;
  const int half = dims >> 1;
  const float* cs = table + p * dims;             // [half][2]
  for (int i = threadIdx.x; i < H * half; i += blockDim.x) {
    const int h = i / half, k = i - h * half;
    E* a = q + (t * H + h) * Dh + offset + 2 * k;
    const float u = ldf(a), v = ldf(a + 1), c = cs[2 * k], s = cs[2 * k + 1];
    stf(a, u * c - v * s);
    stf(a + 1, v * c + u * s);
  }
}

template <typename E>
__global__ void __launch_bounds__(128) latent_kv_store_k(const E* __restrict__ dkv, int64_t ld, const E* __restrict__ nw,
                                                        float eps, int r, int dr, const float* __restrict__ table,
                                                        int max_pos, int dims, const int64_t* __restrict__ pos,
                                                        const int64_t* __restrict__ slots, E* __restrict__ rows,
                                                        int64_t num_rows) {
  __shared__ float red[16];
  const int64_t t = blockIdx.x;
  const int64_t slot = slots[t], p = pos[t];
  const E* in = dkv + t * ld;
  float q = 0.f;
  for (int c = threadIdx.x; c < r; c += blockDim.x) {
    const float v = ldf(in + c);
    q += v * v;
  }
  const float rs = 1.0f / sqrtf(block_sum(q, red) / (float)r + eps);
  if (slot < 0 || slot >= num_rows || p < 0 || p >= max_pos) return;      // padded row
  E* out = rows + slot * (int64_t)(r + dr);
  for (int c = threadIdx.x; c < r; c += blockDim.x) stf(out + c, ldf(in + c) * rs * ldf(nw + c));
  const float* cs = table + p * dims;
  const int half = dims >> 1;
  for (int k = threadIdx.x; k < half; k += blockDim.x) {
    const float u = ldf(in + r + 2 * k), v = ldf(in + r + 2 * k + 1), c = cs[2 * k], s = cs[2 * k + 1];
    stf(out + r + 2 * k, u * c - v * s);
    stf(out + r + 2 * k + 1, v * c + u * s);
  }
  for (int c = dims + threadIdx.x; c < dr; c += blockDim.x) stf(out + r + c, ldf(in + r + c));
}

// ------------------------------------------------------------------ latent attention
// One workgroup: one query token x up to HB heads.  Its NW waves walk the
// token's key tiles (KT keys each, tile i -> keys [i KT, (i + 1) KT), always
// inside one cache page) round-robin; a wave stages a tile in LDS, lane j
// scores key j against every head (f32), the wave does the online-softmax
// update per head, and every lane accumulates its latent columns (f32
// weights x latents: the weights are never rounded to 16 bits).  The waves'
// partial (max, sum, out) are merged through LDS at the end.
// LDS rows are padded to DP = 4 (mod 8) elements: 4-element reads of one
// column group by 64 lanes then spread over all banks.
template <typename E> struct Ld4;
template <> struct Ld4<float> {
  static __device__ __forceinline__ void get(const float* p, float* o) {
    const float4 v = *(const float4*)p;
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Ld4<__bf16> {
  static __device__ __forceinline__ void get(const __bf16* p, float* o) {
    const uint2 v = *(const uint2*)p;
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
};

template <typename E> struct Chunk4;
template <> struct Chunk4<float> { typedef uint4 type; };
template <> struct Chunk4<__bf16> { typedef uint2 type; };

template <typename E, int RC, int HB>
__global__ void __launch_bounds__(256) latent_attn_k(const E* __restrict__ q_lat, const E* __restrict__ q_rot,
                                                    int64_t qr_st, int64_t qr_sh, const E* __restrict__ rows, int bs,
                                                    const int32_t* __restrict__ bt, int bt_w,
                                                    const int32_t* __restrict__ seq_of, const int64_t* __restrict__ pos,
                                                    float scale, const E* __restrict__ gate, int64_t g_st,
                                                    E* __restrict__ out, float* __restrict__ part, int H, int r, int dr,
                                                    int KT, int DP, int window) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int D = r + dr, D4 = (D + 3) & ~3;
  const int nsplit = gridDim.z, zs = blockIdx.z;
  const int t = blockIdx.x, h0 = blockIdx.y * HB;
  const int nh = min(HB, H - h0);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  E* qs = (E*)smem;                                                // [HB][D4], zero padded
  const size_t q_bytes = ((size_t)HB * D4 * sizeof(E) + 15) & ~(size_t)15;
  const size_t wave_bytes = ((size_t)KT * DP * sizeof(E) + (size_t)HB * KT * sizeof(float) + 15) & ~(size_t)15;
  unsigned char* wbase = smem + q_bytes + wv * wave_bytes;
  E* kt = (E*)wbase;                                               // [KT][DP]
  float* pb = (float*)(wbase + (size_t)KT * DP * sizeof(E));       // [HB][KT]
  typedef typename Chunk4<E>::type C4;
  if ((((int64_t)r | dr | qr_st | qr_sh) & 3) == 0 && ((uintptr_t)q_rot % sizeof(C4)) == 0) {
    // whole 4-element chunks, every head's loads independent of the others (one latency, not HB x D)
#pragma unroll
    for (int h = 0; h < HB; h++) {
      C4* dst = (C4*)(qs + h * D4);
      if (h < nh) {
        const C4* a = (const C4*)(q_lat + ((int64_t)t * H + h0 + h) * r);
        const C4* b = (const C4*)(q_rot + (int64_t)t * qr_st + (int64_t)(h0 + h) * qr_sh);
        for (int i = threadIdx.x; i < (r >> 2); i += blockDim.x) dst[i] = a[i];
        for (int i = threadIdx.x; i < (dr >> 2); i += blockDim.x) dst[(r >> 2) + i] = b[i];
      } else {
        for (int i = threadIdx.x; i < D4; i += blockDim.x) stf(qs + h * D4 + i, 0.f);
      }
    }
  } else {
    for (int i = threadIdx.x; i < HB * D4; i += blockDim.x) {
      const int h = i / D4, c = i - h * D4;
      float v = 0.f;
      if (h < nh && c < D)
        v = c < r ? ldf(q_lat + ((int64_t)t * H + h0 + h) * r + c)
                  : ldf(q_rot + (int64_t)t * qr_st + (int64_t)(h0 + h) * qr_sh + (c - r));
      stf(qs + i, v);
    }
  }
  // the whole tile buffer starts finite: rows and pad columns a tile does not fill are read with weight 0
  for (int i = lane; i < KT * DP; i += 64) stf(kt + i, 0.f);
  __syncthreads();
  const int64_t p = pos[t];
  const int32_t* tab = bt + (int64_t)seq_of[t] * bt_w;
  const int ntiles = (int)(p / KT) + 1;
  // a window keeps the keys p - window < j <= p: tiles before the first of them are skipped
  const int64_t lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int tile0 = (int)(lo / KT);
  float m[HB], l[HB], o[HB][RC];
#pragma unroll
  for (int h = 0; h < HB; h++) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int c = 0; c < RC; c++) o[h][c] = 0.f;
  }
  for (int ti = tile0 + zs * NW + wv; ti < ntiles; ti += NW * nsplit) {
    const int64_t k0 = (int64_t)ti * KT;
    const int nvalid = (int)min((int64_t)KT, p - k0 + 1);
    const int64_t row0 = (int64_t)tab[k0 / bs] * bs + (k0 % bs);
    const E* src = rows + row0 * D;
    if ((D & 3) == 0) {
      // 4-element chunks of the tile's contiguous rows; (row, column) advance without a division
      const C4* s4 = (const C4*)src;
      const int n4 = nvalid * (D >> 2);
      int j = 0, c = lane * 4;
      while (c >= D) { c -= D; j++; }
      for (int i = lane; i < n4; i += 64 * 4) {
        C4 v[4];
        int jj[4], cc[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          jj[u] = j;
          cc[u] = c;
          if (i + 64 * u < n4) v[u] = s4[i + 64 * u];
          c += 256;
          while (c >= D) { c -= D; j++; }
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
          if (i + 64 * u < n4) *(C4*)(kt + jj[u] * DP + cc[u]) = v[u];
      }
    } else {
      for (int i = lane; i < nvalid * D; i += 64) {
        const int j = i / D, c = i - j * D;
        kt[j * DP + c] = src[i];
      }
    }
    wave_sync();                                                   // the tile is in LDS
    float s[HB];
#pragma unroll
    for (int h = 0; h < HB; h++) s[h] = 0.f;
    // 64 / KT lanes share a key: each takes a slice of the r + dr products, summed by lane exchange
    const int kj = lane & (KT - 1), grp = lane / KT, G = 64 / KT;
    const bool valid = kj < nvalid && k0 + kj >= lo;
    if (valid) {
      const E* kr = kt + kj * DP;
      const int steps = D4 >> 2;
      for (int c4 = grp * steps / G; c4 < (grp + 1) * steps / G; c4++) {
        const int c = c4 * 4;
        float kv[4];
        Ld4<E>::get(kr + c, kv);
#pragma unroll
        for (int h = 0; h < HB; h++) {
          float qv[4];
          Ld4<E>::get(qs + h * D4 + c, qv);
          s[h] = fmaf(qv[0], kv[0], fmaf(qv[1], kv[1], fmaf(qv[2], kv[2], fmaf(qv[3], kv[3], s[h]))));
        }
      }
    }
    for (int off = KT; off < 64; off <<= 1) {
#pragma unroll
      for (int h = 0; h < HB; h++) s[h] += __shfl_xor(s[h], off, 64);
    }
#pragma unroll
    for (int h = 0; h < HB; h++) {
      const float sv = valid ? s[h] * scale : -INFINITY;
      const float mn = fmaxf(m[h], wave_max(sv));
      const float alpha = m[h] == -INFINITY ? 0.f : expf(m[h] - mn);
      const float pv = valid ? expf(sv - mn) : 0.f;
      l[h] = l[h] * alpha + wave_sum(lane < KT ? pv : 0.f);
      m[h] = mn;
#pragma unroll
      for (int c = 0; c < RC; c++) o[h][c] *= alpha;
      if (lane < KT) pb[h * KT + lane] = pv;
    }
    wave_sync();
    const int nv4 = (nvalid + 3) & ~3;                             // weights past nvalid are 0, rows finite
    for (int j = 0; j < nv4; j += 4) {
      float kv[4][RC];
#pragma unroll
      for (int jj = 0; jj < 4; jj++)
#pragma unroll
        for (int c = 0; c < RC; c++) {
          const int col = lane + 64 * c;
          kv[jj][c] = col < r ? ldf(kt + (j + jj) * DP + col) : 0.f;
        }
#pragma unroll
      for (int h = 0; h < HB; h++) {
        const float4 pv = *(const float4*)(pb + h * KT + j);
#pragma unroll
        for (int c = 0; c < RC; c++)
          o[h][c] = fmaf(pv.x, kv[0][c], fmaf(pv.y, kv[1][c], fmaf(pv.z, kv[2][c], fmaf(pv.w, kv[3][c], o[h][c]))));
      }
    }
    wave_sync();
  }
  // merge the waves: once all are done with the query and their tiles, every
  // wave leaves (m, l, o) in its slice of the (re-used) LDS
  __syncthreads();
  const int MS = HB * (r + 2);
  float* mg = (float*)smem + (size_t)wv * MS;                      // [HB][r + 2]
#pragma unroll
  for (int h = 0; h < HB; h++) {
#pragma unroll
    for (int c = 0; c < RC; c++) {
      const int col = lane + 64 * c;
      if (col < r) mg[h * (r + 2) + col] = o[h][c];
    }
    if (lane == 0) {
      mg[h * (r + 2) + r] = m[h];
      mg[h * (r + 2) + r + 1] = l[h];
    }
  }
  __syncthreads();
  const float* m0 = (const float*)smem;
  for (int i = threadIdx.x; i < nh * (r + 2); i += blockDim.x) {
    const int h = i / (r + 2), c = i - h * (r + 2);
    float M = -INFINITY;
    for (int w = 0; w < NW; w++) M = fmaxf(M, m0[(size_t)w * MS + h * (r + 2) + r]);
    float L = 0.f, O = 0.f;
    for (int w = 0; w < NW; w++) {
      const float* g = m0 + (size_t)w * MS + h * (r + 2);
      const float mw = g[r];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      L += g[r + 1] * f;
      if (c < r) O += g[c] * f;
    }
    if (nsplit > 1) {                                              // partial (o, m, l) of this key split
      float* pp = part + (((int64_t)t * H + h0 + h) * nsplit + zs) * (r + 2);
      pp[c] = c < r ? O : (c == r ? M : L);
    } else if (c < r) {
      float v = O / L;
      if (gate) v *= 1.0f / (1.0f + expf(-ldf(gate + (int64_t)t * g_st + h0 + h)));
      stf(out + ((int64_t)t * H + h0 + h) * r + c, v);
    }
  }
}

// bf16 variant with the score products on the matrix cores: S^T = K Q^T as
// 16x16x32 MFMAs (A = 16 key rows of the LDS tile, B = the head rows of the
// staged query, both bf16 as stored; f32 accumulation), which leaves
// (key = 4 g + i, head = lane & 15) in registers.  Softmax runs there in f32;
// the f32 weights and each head's rescale factor go through LDS to the
// weighted sum, which stays on the vector unit in f32 (weights are not
// rounded).  Tiles are 16 keys; rows are padded to round_up(D, 32) + 8
// elements (zero filled), so fragment reads are aligned and conflict-free.
typedef __bf16 sm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float sm_f32x4 __attribute__((ext_vector_type(4)));

template <int RC, int HB>
__global__ void __launch_bounds__(256) latent_attn_mfma_k(const __bf16* __restrict__ q_lat, const __bf16* __restrict__ q_rot,
                                                         int64_t qr_st, int64_t qr_sh, const __bf16* __restrict__ rows,
                                                         int bs, const int32_t* __restrict__ bt, int bt_w,
                                                         const int32_t* __restrict__ seq_of,
                                                         const int64_t* __restrict__ pos, float scale,
                                                         const __bf16* __restrict__ gate, int64_t g_st,
                                                         __bf16* __restrict__ out, float* __restrict__ part, int H, int r,
                                                         int dr, int DP, int window) {
  typedef __bf16 E;
  constexpr int KT = 16;
  extern __shared__ __align__(16) unsigned char smem[];
  const int D = r + dr, KS = (D + 31) >> 5;                        // 32-wide product steps
  const int nsplit = gridDim.z, zs = blockIdx.z;
  const int t = blockIdx.x, h0 = blockIdx.y * HB;
  const int nh = min(HB, H - h0);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  const int r16 = lane & 15, g = lane >> 4;
  E* qs = (E*)smem;                                                // [16][DP], zero padded rows and columns
  const size_t q_bytes = (size_t)16 * DP * sizeof(E);
  const size_t wave_bytes = ((size_t)KT * DP * sizeof(E) + (size_t)HB * KT * sizeof(float) + 16 * sizeof(float) + 15) & ~(size_t)15;
  unsigned char* wbase = smem + q_bytes + wv * wave_bytes;
  E* kt = (E*)wbase;                                               // [KT][DP]
  float* pb = (float*)(wbase + (size_t)KT * DP * sizeof(E));       // [HB][KT] weights
  float* al = pb + HB * KT;                                        // [16] rescale factor per head
  for (int i = threadIdx.x; i < 16 * DP; i += blockDim.x) stf(qs + i, 0.f);
  for (int i = lane; i < KT * DP; i += 64) stf(kt + i, 0.f);
  __syncthreads();
  typedef uint2 C4;
  if ((((int64_t)r | dr | qr_st | qr_sh) & 3) == 0 && ((uintptr_t)q_rot % sizeof(C4)) == 0) {
#pragma unroll
    for (int h = 0; h < HB; h++) {
      if (h < nh) {
        C4* dst = (C4*)(qs + h * DP);
        const C4* a = (const C4*)(q_lat + ((int64_t)t * H + h0 + h) * r);
        const C4* b = (const C4*)(q_rot + (int64_t)t * qr_st + (int64_t)(h0 + h) * qr_sh);
        for (int i = threadIdx.x; i < (r >> 2); i += blockDim.x) dst[i] = a[i];
        for (int i = threadIdx.x; i < (dr >> 2); i += blockDim.x) dst[(r >> 2) + i] = b[i];
      }
    }
  } else {
    for (int i = threadIdx.x; i < nh * D; i += blockDim.x) {
      const int h = i / D, c = i - h * D;
      qs[h * DP + c] = c < r ? q_lat[((int64_t)t * H + h0 + h) * r + c]
                             : q_rot[(int64_t)t * qr_st + (int64_t)(h0 + h) * qr_sh + (c - r)];
    }
  }
  __syncthreads();
  const int64_t p = pos[t];
  const int32_t* tab = bt + (int64_t)seq_of[t] * bt_w;
  const int ntiles = (int)(p / KT) + 1;
  // a window keeps the keys p - window < j <= p: tiles before the first of them are skipped
  const int64_t lo = window > 0 ? (p - window + 1 > 0 ? p - window + 1 : 0) : 0;
  const int tile0 = (int)(lo / KT);
  float m_r = -INFINITY, l_r = 0.f;                                // of head r16 (the same in its four lanes)
  float o[HB][RC];
#pragma unroll
  for (int h = 0; h < HB; h++)
#pragma unroll
    for (int c = 0; c < RC; c++) o[h][c] = 0.f;
  for (int ti = tile0 + zs * NW + wv; ti < ntiles; ti += NW * nsplit) {
    const int64_t k0 = (int64_t)ti * KT;
    const int nvalid = (int)min((int64_t)KT, p - k0 + 1);
    const int64_t row0 = (int64_t)tab[k0 / bs] * bs + (k0 % bs);
    const E* src = rows + row0 * D;
    if ((D & 3) == 0) {
      const C4* s4 = (const C4*)src;
      const int n4 = nvalid * (D >> 2);
      int j = 0, c = lane * 4;
      while (c >= D) { c -= D; j++; }
      for (int i = lane; i < n4; i += 64 * 4) {
        C4 v[4];
        int jj[4], cc[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          jj[u] = j;
          cc[u] = c;
          if (i + 64 * u < n4) v[u] = s4[i + 64 * u];
          c += 256;
          while (c >= D) { c -= D; j++; }
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
          if (i + 64 * u < n4) *(C4*)(kt + jj[u] * DP + cc[u]) = v[u];
      }
    } else {
      for (int i = lane; i < nvalid * D; i += 64) {
        const int j = i / D, c = i - j * D;
        kt[j * DP + c] = src[i];
      }
    }
    wave_sync();
    sm_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    const E* ka = kt + r16 * DP + 8 * g;
    const E* qb = qs + r16 * DP + 8 * g;
    for (int ks = 0; ks < KS; ks++) {
      const sm_bf16x8 a = *(const sm_bf16x8*)(ka + 32 * ks);
      const sm_bf16x8 b = *(const sm_bf16x8*)(qb + 32 * ks);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0);
    }
    // lane: keys 4 g + i (i = 0..3) of head r16
    float sv[4], mloc = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      sv[i] = (4 * g + i) < nvalid && k0 + 4 * g + i >= lo ? acc[i] * scale : -INFINITY;
      mloc = fmaxf(mloc, sv[i]);
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    const float mn = fmaxf(m_r, mloc);
    const float alpha = m_r == -INFINITY ? 0.f : expf(m_r - mn);
    float pv[4], lsum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      pv[i] = sv[i] == -INFINITY ? 0.f : expf(sv[i] - mn);
      lsum += pv[i];
    }
    lsum += __shfl_xor(lsum, 16, 64);
    lsum += __shfl_xor(lsum, 32, 64);
    l_r = l_r * alpha + lsum;
    m_r = mn;
    if (r16 < HB) {
      *(float4*)(pb + r16 * KT + 4 * g) = make_float4(pv[0], pv[1], pv[2], pv[3]);
      if (g == 0) al[r16] = alpha;
    }
    wave_sync();
#pragma unroll
    for (int h = 0; h < HB; h++) {
      const float a = al[h];
#pragma unroll
      for (int c = 0; c < RC; c++) o[h][c] *= a;
    }
    const int nv4 = (nvalid + 3) & ~3;
    for (int j = 0; j < nv4; j += 4) {
      float kv[4][RC];
#pragma unroll
      for (int jj = 0; jj < 4; jj++)
#pragma unroll
        for (int c = 0; c < RC; c++) {
          const int col = lane + 64 * c;
          kv[jj][c] = col < r ? ldf(kt + (j + jj) * DP + col) : 0.f;
        }
#pragma unroll
      for (int h = 0; h < HB; h++) {
        const float4 w4 = *(const float4*)(pb + h * KT + j);
#pragma unroll
        for (int c = 0; c < RC; c++)
          o[h][c] = fmaf(w4.x, kv[0][c], fmaf(w4.y, kv[1][c], fmaf(w4.z, kv[2][c], fmaf(w4.w, kv[3][c], o[h][c]))));
      }
    }
    wave_sync();
  }
  __syncthreads();
  const int MS = HB * (r + 2);
  float* mg = (float*)smem + (size_t)wv * MS;
#pragma unroll
  for (int h = 0; h < HB; h++)
#pragma unroll
    for (int c = 0; c < RC; c++) {
      const int col = lane + 64 * c;
      if (col < r) mg[h * (r + 2) + col] = o[h][c];
    }
  if (g == 0 && r16 < HB) {
    mg[r16 * (r + 2) + r] = m_r;
    mg[r16 * (r + 2) + r + 1] = l_r;
  }
  __syncthreads();
  const float* m0 = (const float*)smem;
  for (int i = threadIdx.x; i < nh * (r + 2); i += blockDim.x) {
    const int h = i / (r + 2), c = i - h * (r + 2);
    float M = -INFINITY;
    for (int w = 0; w < NW; w++) M = fmaxf(M, m0[(size_t)w * MS + h * (r + 2) + r]);
    float L = 0.f, O = 0.f;
    for (int w = 0; w < NW; w++) {
      const float* gp = m0 + (size_t)w * MS + h * (r + 2);
      const float mw = gp[r];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      L += gp[r + 1] * f;
      if (c < r) O += gp[c] * f;
    }
    if (nsplit > 1) {
      float* pp = part + (((int64_t)t * H + h0 + h) * nsplit + zs) * (r + 2);
      pp[c] = c < r ? O : (c == r ? M : L);
    } else if (c < r) {
      float v = O / L;
      if (gate) v *= 1.0f / (1.0f + expf(-ldf(gate + (int64_t)t * g_st + h0 + h)));
      stf(out + ((int64_t)t * H + h0 + h) * r + c, v);
    }
  }
}


// merge of the key splits: part [T, H, nsplit, r + 2] -> out [T, H, r]
template <typename E>
__global__ void __launch_bounds__(128) latent_attn_combine_k(const float* __restrict__ part, const E* __restrict__ gate,
                                                            int64_t g_st, E* __restrict__ out, int H, int r,
                                                            int nsplit) {
  __shared__ float wz[64];                                          // exp(m_z - M) / L * gate, nsplit <= 64
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* pp = part + ((t * H + h) * nsplit) * (int64_t)(r + 2);
  if (threadIdx.x < 64) {
    const int z = threadIdx.x;
    const float mz = z < nsplit ? pp[(int64_t)z * (r + 2) + r] : -INFINITY;
    const float M = wave_max(mz);
    const float e = mz == -INFINITY ? 0.f : expf(mz - M);
    const float L = wave_sum(z < nsplit ? pp[(int64_t)z * (r + 2) + r + 1] * e : 0.f);
    const float g = gate ? 1.0f / (1.0f + expf(-ldf(gate + t * g_st + h))) : 1.0f;
    wz[z] = e / L * g;
  }
  __syncthreads();
  for (int c = threadIdx.x; c < r; c += blockDim.x) {
    float O = 0.f;
    for (int z = 0; z < nsplit; z++) O = fmaf(pp[(int64_t)z * (r + 2) + c], wz[z], O);
    stf(out + (t * H + h) * r + c, O);
  }
}

// Causal softmax over f32 score rows (the library-GEMM prefill path): row i
// belongs to query token i / H at position pos[i / H]; keys j <= pos get
// softmax(scale * s) in f32, the others 0.  E = float: written in place.
// E = bf16: the f32 weight leaves as a pair of bf16 values hi + lo (hi the
// rounded weight, lo the rounded remainder), so the following bf16 products
// carry the weights to ~2^-17 instead of 2^-9.
template <typename E>
__global__ void __launch_bounds__(256) causal_softmax_k(float* __restrict__ sc, int64_t ld, const int64_t* __restrict__ pos,
                                                       int H, float scale, int L, E* __restrict__ hi, E* __restrict__ lo,
                                                       int64_t key0, int window) {
  __shared__ float red[16];
  const int64_t row = blockIdx.x;
  const int64_t p = pos[row / H];
  // column j is key key0 + j; visible: key <= p, and key > p - window with a window
  const int nk = (int)max((int64_t)0, min((int64_t)L, p - key0 + 1));
  const int j0 = window > 0 ? (int)max((int64_t)0, min((int64_t)nk, p - window + 1 - key0)) : 0;
  float* s = sc + row * ld;
  float mx = -INFINITY;
  for (int j = j0 + threadIdx.x; j < nk; j += blockDim.x) mx = fmaxf(mx, s[j] * scale);
  mx = wave_max(mx);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) mx = fmaxf(mx, red[i]);
  float sum = 0.f;
  for (int j = j0 + threadIdx.x; j < nk; j += blockDim.x) {
    const float e = expf(s[j] * scale - mx);
    s[j] = e;
    sum += e;
  }
  const float inv = 1.0f / block_sum(sum, red);
  for (int j = threadIdx.x; j < L; j += blockDim.x) {
    const float w = j >= j0 && j < nk ? s[j] * inv : 0.f;
    if (hi) {
      const E h = (E)w;
      hi[row * ld + j] = h;
      lo[row * ld + j] = (E)(w - (float)h);
    } else {
      s[j] = w;
    }
  }
}

// ------------------------------------------------------------------ mLSTM
// One workgroup: 64 value columns of one (sequence, head).  Wave w keeps the
// key rows [w DS, (w + 1) DS) of those columns in registers (the manner of
// the RWKV-5 WKV kernel, misc.hip, with the key dimension split over up to
// four waves).  Tokens go through LDS in chunks of TC: all threads stage q,
// k, v and the gates; wave 0 runs the scalar recurrences (gates, running
// maximum, normaliser n and its dot with q) once per chunk; every wave then
// updates its rows and leaves a partial numerator per token; the partials are
// summed in a fixed order, so a result never depends on how the tokens were
// cut into steps.
template <typename E, int DS>
__global__ void __launch_bounds__(256) mlstm_scan_k(const E* __restrict__ q, int64_t q_ld, const E* __restrict__ k,
                                                   int64_t k_ld, const E* __restrict__ v, int64_t v_ld,
                                                   const E* __restrict__ ipre, int64_t i_ld, const E* __restrict__ fpre,
                                                   int64_t f_ld, const float* __restrict__ ib, const float* __restrict__ fb,
                                                   float cap, float* __restrict__ Sg, float* __restrict__ ng,
                                                   float* __restrict__ mgl, const int32_t* __restrict__ cu,
                                                   const int32_t* __restrict__ slots, const int64_t* __restrict__ pos,
                                                   float* __restrict__ out, int H, int d, int dv, int TC, bool vec) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, NWV = blockDim.x >> 6, DP = NWV * DS;
  float* qs = (float*)smem;                 // [TC][DP]
  float* ks = qs + (size_t)TC * DP;         // [TC][DP]
  float* vs = ks + (size_t)TC * DP;         // [TC][64]
  float* part = vs + (size_t)TC * 64;       // [NWV][TC][64]
  float* ab = part + (size_t)NWV * TC * 64; // a, b, den [3][TC]
  float* gi = ab + 3 * TC;                  // log gates i, f [2][TC]
  const int b = blockIdx.x, h = blockIdx.y;
  const int j = blockIdx.z * 64 + lane;
  const bool jv = j < dv;
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t0 >= t1) return;
  const int64_t slot = slots[b];
  const bool fresh = pos[t0] == 0;
  float* Ss = Sg + ((slot * H + h) * d) * (int64_t)dv;
  float* ns = ng + (slot * H + h) * (int64_t)d;
  float s[DS];
#pragma unroll
  for (int i = 0; i < DS; i++) {
    const int row = w * DS + i;
    s[i] = (fresh || !jv || row >= d) ? 0.f : Ss[(int64_t)row * dv + j];
  }
  float nreg[4] = {0.f, 0.f, 0.f, 0.f};
  float m = 0.f;
  if (w == 0 && !fresh) {
    m = mgl[slot * H + h];
#pragma unroll
    for (int c = 0; c < 4; c++)
      if (lane + 64 * c < d) nreg[c] = ns[lane + 64 * c];
  }
  const float qscale = 1.0f / sqrtf((float)d);
  for (int tb = t0; tb < t1; tb += TC) {
    const int nt = min(TC, t1 - tb);
    __syncthreads();
    if (vec) {
      // 4-element chunks; a thread's loads are all issued before the first store
      const int c4n = DP >> 2, n4 = nt * c4n;
      float qv[4][4], kv[4][4];
      int at[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int i = threadIdx.x + u * blockDim.x;
        at[u] = -1;
        if (i < n4) {
          const int tt = i / c4n, c = (i - tt * c4n) * 4;
          at[u] = tt * DP + c;
          if (c < d) {
            Ld4<E>::get(q + (int64_t)(tb + tt) * q_ld + h * d + c, qv[u]);
            Ld4<E>::get(k + (int64_t)(tb + tt) * k_ld + h * d + c, kv[u]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++) qv[u][e] = kv[u][e] = 0.f;
          }
        }
      }
      float vv[4];
      const int vi = threadIdx.x;                                     // 16 tokens x 16 chunks = 256 chunks at most
      const int vt = vi >> 4, vc = blockIdx.z * 64 + (vi & 15) * 4;
      const bool vok = vi < nt * 16;
      if (vok) {
        if (vc < dv) Ld4<E>::get(v + (int64_t)(tb + vt) * v_ld + h * dv + vc, vv);
        else vv[0] = vv[1] = vv[2] = vv[3] = 0.f;
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (at[u] >= 0) {
#pragma unroll
          for (int e = 0; e < 4; e++) {
            qs[at[u] + e] = qv[u][e] * qscale;
            ks[at[u] + e] = kv[u][e];
          }
        }
      if (blockDim.x < 256) {                                          // fewer threads than value chunks
        for (int i = threadIdx.x; i < nt * 64; i += blockDim.x) {
          const int tt = i >> 6, col = blockIdx.z * 64 + (i & 63);
          vs[i] = col < dv ? ldf(v + (int64_t)(tb + tt) * v_ld + h * dv + col) : 0.f;
        }
      } else if (vok) {
#pragma unroll
        for (int e = 0; e < 4; e++) vs[vt * 64 + (vi & 15) * 4 + e] = vv[e];
      }
    } else {
      for (int i = threadIdx.x; i < nt * DP; i += blockDim.x) {
        const int tt = i / DP, c = i - tt * DP;
        qs[i] = c < d ? ldf(q + (int64_t)(tb + tt) * q_ld + h * d + c) * qscale : 0.f;
        ks[i] = c < d ? ldf(k + (int64_t)(tb + tt) * k_ld + h * d + c) : 0.f;
      }
      for (int i = threadIdx.x; i < nt * 64; i += blockDim.x) {
        const int tt = i >> 6, col = blockIdx.z * 64 + (i & 63);
        vs[i] = col < dv ? ldf(v + (int64_t)(tb + tt) * v_ld + h * dv + col) : 0.f;
      }
    }
    for (int tt = threadIdx.x; tt < nt; tt += blockDim.x) {
      const float iz = (ldf(ipre + (int64_t)(tb + tt) * i_ld + h) + ib[h]) / cap;
      const float fz = cap * tanhf((ldf(fpre + (int64_t)(tb + tt) * f_ld + h) + fb[h]) / cap);
      gi[tt] = cap * tanhf(iz);
      gi[TC + tt] = fminf(fz, 0.f) - log1pf(expf(-fabsf(fz)));     // logsigmoid
    }
    __syncthreads();
    if (w == 0) {
      for (int tt = 0; tt < nt; tt++) {
        const float ig = gi[tt], fg = gi[TC + tt];
        const float mn = fmaxf(fg + m, ig);
        const float a = expf(fg + m - mn), bb = expf(ig - mn);
        m = mn;
        float pq = 0.f;
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const int row = lane + 64 * c;
          if (row < DP) {
            nreg[c] = a * nreg[c] + bb * ks[tt * DP + row];
            pq = fmaf(nreg[c], qs[tt * DP + row], pq);
          }
        }
        const float nq = wave_sum(pq);
        if (lane == 0) {
          ab[tt] = a;
          ab[TC + tt] = bb;
          ab[2 * TC + tt] = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
        }
      }
    }
    __syncthreads();
    for (int tt = 0; tt < nt; tt++) {
      const float a = ab[tt], bb = ab[TC + tt], vj = vs[tt * 64 + lane];
      const float* kk = ks + tt * DP + w * DS;
      const float* qq = qs + tt * DP + w * DS;
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < DS; i++) {
        s[i] = fmaf(a, s[i], (bb * kk[i]) * vj);
        acc = fmaf(s[i], qq[i], acc);
      }
      part[((size_t)w * TC + tt) * 64 + lane] = acc;
    }
    __syncthreads();
    for (int tt = w; tt < nt; tt += NWV) {
      float sum = 0.f;
      for (int ww = 0; ww < NWV; ww++) sum += part[((size_t)ww * TC + tt) * 64 + lane];
      if (jv) out[((int64_t)(tb + tt) * H + h) * dv + j] = sum / ab[2 * TC + tt];
    }
  }
  if (jv) {
#pragma unroll
    for (int i = 0; i < DS; i++) {
      const int row = w * DS + i;
      if (row < d) Ss[(int64_t)row * dv + j] = s[i];
    }
  }
  if (w == 0 && blockIdx.z == 0) {
#pragma unroll
    for (int c = 0; c < 4; c++)
      if (lane + 64 * c < d) ns[lane + 64 * c] = nreg[c];
    if (lane == 0) mgl[slot * H + h] = m;
  }
}

template <typename E>
__global__ void __launch_bounds__(64) head_rms_gate_k(const float* __restrict__ hh, const E* __restrict__ nw,
                                                     const E* __restrict__ gate, int64_t g_ld, E* __restrict__ out,
                                                     int H, int dv, float eps) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y;
  const float* in = hh + (t * H + h) * dv;
  float q = 0.f;
  for (int c = threadIdx.x; c < dv; c += 64) q += in[c] * in[c];
  const float rs = 1.0f / sqrtf(wave_sum(q) / (float)dv + eps);
  for (int c = threadIdx.x; c < dv; c += 64) {
    const float g = 1.0f / (1.0f + expf(-ldf(gate + t * g_ld + h * dv + c)));
    stf(out + (t * H + h) * dv + c, in[c] * rs * ldf(nw + h * dv + c) * g);
  }
}

template <typename E>
__global__ void __launch_bounds__(256) glu_gelu_k(const E* __restrict__ gu, E* __restrict__ out, int64_t T, int64_t I) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * I) return;
  const int64_t t = i / I, c = i - t * I;
  const float g = ldf(gu + t * 2 * I + c), u = ldf(gu + t * 2 * I + I + c);
  const float a = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  stf(out + i, a * u);
}

// act(gate) * up; ACT 0: tanh-GELU, 1: ReLU, 2: SiLU (f32 math)
template <typename E, int ACT>
__global__ void __launch_bounds__(256) glu_act_k(const E* __restrict__ gu, E* __restrict__ out, int64_t T, int64_t I) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= T * I) return;
  const int64_t t = i / I, c = i - t * I;
  const float g = ldf(gu + t * 2 * I + c), u = ldf(gu + t * 2 * I + I + c);
  float a;
  if (ACT == 1) a = fmaxf(g, 0.f);
  else if (ACT == 2) a = g / (1.0f + expf(-g));
  else a = 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
  stf(out + i, a * u);
}

}  // namespace

#define SM_DISPATCH(bf16, ...)                 \
  if (bf16) {                                  \
    typedef __bf16 E;                          \
    __VA_ARGS__;                               \
  } else {                                     \
    typedef float E;                           \
    __VA_ARGS__;                               \
  }

void embed_bigram(bool bf16, const int64_t* ids, const int64_t* prev, const void* embed, const void* bigram, float* out,
                  int T, int W, int64_t vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(embed_bigram_k<E>, dim3(T), dim3(256), 0, st, ids, prev, (const E*)embed,
                                       (const E*)bigram, out, W, vocab, buckets, mul_prev, mul_cur));
}

void add_scaled_layer_norm(bool bf16, float* x, const void* y, const void* w, void* xa, int T, int W, float eps,
                           float mult, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(add_sln_k<E>, dim3(T), dim3(256), 0, st, x, (const E*)y, (const E*)w, (E*)xa, W,
                                       eps, mult));
}

void layer_norm(bool bf16, const float* x, const void* w, void* out, int T, int W, float eps, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(layer_norm_k<E>, dim3(T), dim3(256), 0, st, x, (const E*)w, (E*)out, W, eps));
}

void rope_rows(bool bf16, void* q, int T, int H, int Dh, int offset, const float* table, int max_pos, int dims,
               const int64_t* pos, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(rope_rows_k<E>, dim3(T), dim3(256), 0, st, (E*)q, H, Dh, offset, table, max_pos,
                                       dims, pos));
}

void latent_kv_store(bool bf16, const void* dkv, int64_t ld, const void* norm_w, float eps, int rank, int rot_dim,
                     const float* table, int max_pos, int dims, const int64_t* pos, const int64_t* slots, void* rows,
                     int64_t num_rows, int T, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(latent_kv_store_k<E>, dim3(T), dim3(128), 0, st, (const E*)dkv, ld,
                                       (const E*)norm_w, eps, rank, rot_dim, table, max_pos, dims, pos, slots, (E*)rows,
                                       num_rows));
}

static int pad_row(int D) {
  // row stride (elements) = 4 (mod 8): 4-element reads of a column group by 64 lanes spread over all banks
  int dp = (D + 3) & ~3;
  return (dp & 7) == 4 ? dp : dp + 4;
}

// LDS plan: heads per workgroup, keys per tile, waves.  The tile buffers, the
// query block and (afterwards, over the same memory) the waves' merge slices
// must fit in 64 KB.
int latent_attention_plan(bool bf16, int H, int r, int dr, int* kt, int* nw, int* hbo) {
  const int esz = bf16 ? 2 : 4, D = r + dr;
  const int DP = pad_row(D), D4 = (D + 3) & ~3;
  // (keys per tile, waves): more waves first -- lanes are never idle whatever the tile size
  static const int opts[][2] = {{64, 4}, {32, 4}, {16, 4}, {64, 2}, {32, 2}, {16, 2}, {64, 1}, {32, 1}, {16, 1}};
  // 16 heads per workgroup only while the f32 accumulators (heads x latent columns per lane) stay in registers
  for (int hb = (H > 8 && r <= 128) ? 16 : 8; hb >= 8; hb -= 8) {
    const size_t qbytes = ((size_t)hb * D4 * esz + 15) & ~(size_t)15;
    for (auto& o : opts) {
      const size_t wave = ((size_t)o[0] * DP * esz + (size_t)hb * o[0] * 4 + 15) & ~(size_t)15;
      const size_t total = qbytes + wave * o[1];
      if (total <= 64 * 1024 && (size_t)o[1] * hb * (r + 2) * 4 <= total) {
        *kt = o[0];
        *nw = o[1];
        *hbo = hb;
        return (int)total;
      }
    }
  }
  return -1;
}

// the bf16 MFMA variant: 16-key tiles, rows of round_up(D, 32) + 8 elements
static int mfma_row(int D) { return ((D + 31) & ~31) + 8; }
static int latent_attention_plan_mfma(int H, int r, int dr, int* nw, int* hbo) {
  const int DP = mfma_row(r + dr);
  for (int hb = (H > 8 && r <= 128) ? 16 : 8; hb >= 8; hb -= 8) {
    const size_t qbytes = (size_t)16 * DP * 2;
    const size_t wave = ((size_t)16 * DP * 2 + (size_t)hb * 16 * 4 + 16 * 4 + 15) & ~(size_t)15;
    for (int w = 4; w >= 1; w--) {
      const size_t total = qbytes + wave * w;
      if (total <= 64 * 1024 && (size_t)w * hb * (r + 2) * 4 <= total) {
        *nw = w;
        *hbo = hb;
        return (int)total;
      }
    }
  }
  return -1;
}

static const bool kUseMfma = []() {
  const char* e = getenv("ILLM_LATENT_MFMA");
  return !(e && e[0] == '0');
}();

int latent_attention_splits(bool bf16, int T, int H, int r, int dr, int max_ctx) {   // with a window: the keys it spans
  int KT = 0, NW = 0, hb = 8;
  if (bf16 && kUseMfma && latent_attention_plan_mfma(H, r, dr, &NW, &hb) > 0) KT = 16;
  else if (latent_attention_plan(bf16, H, r, dr, &KT, &NW, &hb) < 0) return 1;
  const int64_t blocks = (int64_t)T * ((H + hb - 1) / hb);
  const int tiles = (max_ctx + KT - 1) / KT;
  int ns = (int)((1024 + blocks - 1) / blocks);            // ~4 workgroups per CU
  ns = ns > (tiles + NW - 1) / NW ? (tiles + NW - 1) / NW : ns;
  return ns < 1 ? 1 : (ns > 64 ? 64 : ns);
}

void latent_attention(bool bf16, const void* q_lat, const void* q_rot, int64_t qr_st, int64_t qr_sh, const void* rows,
                      int bs, const int32_t* block_tables, int bt_width, const int32_t* seq_of, const int64_t* pos,
                      float scale, const void* gate, int64_t g_st, void* out, float* part, int nsplit, int T, int H,
                      int r, int dr, int window, hipStream_t st) {
  if (T <= 0) return;
  const int rc = (r + 63) / 64;
  int KT = 0, NW = 0, hb = 8;
  if (bf16 && kUseMfma) {
    const int lds = latent_attention_plan_mfma(H, r, dr, &NW, &hb);
    if (lds > 0) {
      const int DP = mfma_row(r + dr);
      dim3 grid(T, (H + hb - 1) / hb, nsplit), block(64 * NW);
#define SM_ATTN_M(RC, HBV)                                                                                            \
  hipLaunchKernelGGL((latent_attn_mfma_k<RC, HBV>), grid, block, lds, st, (const __bf16*)q_lat, (const __bf16*)q_rot,  \
                     qr_st, qr_sh, (const __bf16*)rows, bs, block_tables, bt_width, seq_of, pos, scale,                \
                     (const __bf16*)gate, g_st, (__bf16*)out, part, H, r, dr, DP, window)
      if (hb == 8) {
        if (rc <= 1) { SM_ATTN_M(1, 8); }
        else if (rc <= 2) { SM_ATTN_M(2, 8); }
        else if (rc <= 4) { SM_ATTN_M(4, 8); }
        else { SM_ATTN_M(8, 8); }
      } else {
        if (rc <= 1) { SM_ATTN_M(1, 16); }
        else { SM_ATTN_M(2, 16); }
      }
#undef SM_ATTN_M
      if (nsplit > 1)
        hipLaunchKernelGGL(latent_attn_combine_k<__bf16>, dim3(T, H), dim3(128), 0, st, part, (const __bf16*)gate, g_st,
                           (__bf16*)out, H, r, nsplit);
      return;
    }
  }
  const int lds = latent_attention_plan(bf16, H, r, dr, &KT, &NW, &hb);
  if (lds < 0) return;                     // refused by the caller beforehand
  const int DP = pad_row(r + dr);
  dim3 grid(T, (H + hb - 1) / hb, nsplit), block(64 * NW);
#define SM_ATTN(RC, HBV)                                                                                              \
  SM_DISPATCH(bf16, hipLaunchKernelGGL((latent_attn_k<E, RC, HBV>), grid, block, lds, st, (const E*)q_lat,             \
                                       (const E*)q_rot, qr_st, qr_sh, (const E*)rows, bs, block_tables, bt_width,      \
                                       seq_of, pos, scale, (const E*)gate, g_st, (E*)out, part, H, r, dr, KT, DP,      \
                                       window))
  if (hb == 8) {
    if (rc <= 1) { SM_ATTN(1, 8); }
    else if (rc <= 2) { SM_ATTN(2, 8); }
    else if (rc <= 4) { SM_ATTN(4, 8); }
    else { SM_ATTN(8, 8); }
  } else {
    if (rc <= 1) { SM_ATTN(1, 16); }
    else { SM_ATTN(2, 16); }
  }
#undef SM_ATTN
  if (nsplit > 1) {
    SM_DISPATCH(bf16, hipLaunchKernelGGL(latent_attn_combine_k<E>, dim3(T, H), dim3(128), 0, st, part, (const E*)gate,
                                         g_st, (E*)out, H, r, nsplit));
  }
}

void causal_softmax(bool bf16, float* sc, int64_t ld, const int64_t* pos, int H, float scale, int64_t R, int L, void* hi,
                    void* lo, int64_t key0, int window, hipStream_t st) {
  if (R <= 0 || L <= 0) return;
  if (bf16) {
    hipLaunchKernelGGL(causal_softmax_k<__bf16>, dim3((unsigned)R), dim3(256), 0, st, sc, ld, pos, H, scale, L,
                       (__bf16*)hi, (__bf16*)lo, key0, window);
  } else {
    hipLaunchKernelGGL(causal_softmax_k<float>, dim3((unsigned)R), dim3(256), 0, st, sc, ld, pos, H, scale, L,
                       (float*)nullptr, (float*)nullptr, key0, window);
  }
}

void mlstm_scan(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                const void* ipre, int64_t i_ld, const void* fpre, int64_t f_ld, const float* ib, const float* fb,
                float cap, float* S, float* n, float* m, const int32_t* cu, const int32_t* slots, const int64_t* pos,
                float* out, int B, int H, int d, int dv, hipStream_t st) {
  if (B <= 0 || d > 256) return;           // d checked by the caller
  const int DS = d <= 32 ? 8 : d <= 64 ? 16 : d <= 128 ? 32 : 64;
  const int NWV = (d + DS - 1) / DS, DP = NWV * DS;
  const int TC = 16;                       // tokens staged per chunk (52 KB of LDS at d = 256)
  const size_t lds = ((size_t)2 * TC * DP + (size_t)TC * 64 + (size_t)NWV * TC * 64 + 5 * (size_t)TC) * 4;
  dim3 grid(B, H, (dv + 63) / 64), block(64 * NWV);
  // aligned 4-element loads: sizes, row strides and base addresses all multiples of 4 elements; the
  // chunked staging covers 4 x 256 (q, k) chunks per 16 tokens
  const size_t a4 = bf16 ? 8 : 16;
  const bool vec = ((d | dv | q_ld | k_ld | v_ld) & 3) == 0 && (uintptr_t)q % a4 == 0 && (uintptr_t)k % a4 == 0 &&
                   (uintptr_t)v % a4 == 0 && TC * (DP >> 2) <= 4 * 64 * NWV;
#define SM_SCAN(DSV)                                                                                                  \
  SM_DISPATCH(bf16, hipLaunchKernelGGL((mlstm_scan_k<E, DSV>), grid, block, lds, st, (const E*)q, q_ld, (const E*)k,   \
                                       k_ld, (const E*)v, v_ld, (const E*)ipre, i_ld, (const E*)fpre, f_ld, ib, fb,    \
                                       cap, S, n, m, cu, slots, pos, out, H, d, dv, TC, vec))
  if (DS == 8) { SM_SCAN(8); }
  else if (DS == 16) { SM_SCAN(16); }
  else if (DS == 32) { SM_SCAN(32); }
  else { SM_SCAN(64); }
#undef SM_SCAN
}

void head_rms_gate(bool bf16, const float* h, const void* norm_w, const void* gate, int64_t g_ld, void* out, int T,
                   int H, int dv, float eps, hipStream_t st) {
  if (T <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(head_rms_gate_k<E>, dim3(T, H), dim3(64), 0, st, h, (const E*)norm_w,
                                       (const E*)gate, g_ld, (E*)out, H, dv, eps));
}

void glu_act(bool bf16, const void* gu, void* out, int64_t T, int64_t I, int act, hipStream_t st) {
  const int64_t n = T * I;
  if (n <= 0) return;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (act == 1) {
    SM_DISPATCH(bf16, hipLaunchKernelGGL((glu_act_k<E, 1>), dim3(blocks), dim3(256), 0, st, (const E*)gu, (E*)out, T, I));
  } else if (act == 2) {
    SM_DISPATCH(bf16, hipLaunchKernelGGL((glu_act_k<E, 2>), dim3(blocks), dim3(256), 0, st, (const E*)gu, (E*)out, T, I));
  } else {
    SM_DISPATCH(bf16, hipLaunchKernelGGL((glu_act_k<E, 0>), dim3(blocks), dim3(256), 0, st, (const E*)gu, (E*)out, T, I));
  }
}

void glu_gelu(bool bf16, const void* gu, void* out, int64_t T, int64_t I, hipStream_t st) {
  const int64_t n = T * I;
  if (n <= 0) return;
  SM_DISPATCH(bf16, hipLaunchKernelGGL(glu_gelu_k<E>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                                       (const E*)gu, (E*)out, T, I));
}

}  // namespace sm
}  // namespace illm
