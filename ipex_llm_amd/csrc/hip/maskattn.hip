// Masked grouped-query attention over paged [keys | values] rows (gfx950,
// wave64).
//
//   norm + rotary + append   one workgroup per token: the sums of squares of
//                            every head (per-head norm) or of the whole
//                            projection, then every value normed, turned with
//                            its partner and written: queries as f32, keys
//                            and values into the token's cache row
//   attention                one workgroup: one query token x up to HB query
//                            heads of one key head.  Its waves walk the
//                            token's visible key tiles (16 keys, always inside
//                            one cache page) round-robin from the tile that
//                            holds the first visible key; a wave stages keys
//                            and values of the tile in LDS, four lanes share a
//                            key's dot product with every head (f32 queries,
//                            never rounded), the wave does the online-softmax
//                            update per head and every lane accumulates its
//                            value columns.  The waves' partial (max, sum,
//                            out) are merged through LDS; the sink enters the
//                            denominator at the very end (after the merge of
//                            the key splits, if any)
//   chunk softmax            the softmax (sink, causal inside the chunk)
//                            between the batched library products of whole
//                            chunks
//
// Activations are bf16 or f32 (template E); accumulation is always f32.
#include "maskattn.h"

#include <math.h>

namespace illm {
namespace ma {
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
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ void wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
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

// ------------------------------------------------------------------ norm + rotary + append
// hs: LDS [H + G] sums of squares per head
template <typename EI, typename E>
__device__ __forceinline__ float normed(const EI* x, int i, int head, int d, const E* nw, bool whole, float rs) {
  float v = ldf(x + i);
  if (nw) v = v * rs * ldf(nw + (whole ? head * d + i : i));
  return v;
}

// EI: element type of the projected q / k / v (f32 when a convolution came first), E: of the norm weights and the rows
template <typename EI, typename E>
__global__ void __launch_bounds__(1024) qkv_store_k(const EI* __restrict__ q, int64_t q_ld, const EI* __restrict__ k,
                                                  int64_t k_ld, const EI* __restrict__ v, int64_t v_ld,
                                                  const E* __restrict__ qn, const E* __restrict__ kn, bool whole,
                                                  float eps, const float* __restrict__ table, int dims, int layout,
                                                  const int64_t* __restrict__ pos, const int64_t* __restrict__ slots,
                                                  E* __restrict__ rows, float* __restrict__ qo, int H, int G, int d,
                                                  int dv) {
  extern __shared__ float hs[];                                     // [H + G] (+ 2 totals)
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  const int NH = H + (k ? G : 0);
  const EI* qr = q + t * q_ld;
  const EI* kr = k ? k + t * k_ld : nullptr;
  for (int hh = wv; hh < NH; hh += NW) {
    const EI* x = hh < H ? qr + hh * d : kr + (hh - H) * d;
    float s = 0.f;
    for (int i = lane; i < d; i += 64) {
      const float a = ldf(x + i);
      s += a * a;
    }
    s = wave_sum(s);
    if (lane == 0) hs[hh] = s;
  }
  __syncthreads();
  if (whole && threadIdx.x == 0) {                                  // fixed order: the same sum whatever the launch
    float a = 0.f, b = 0.f;
    for (int i = 0; i < H; i++) a += hs[i];
    for (int i = H; i < NH; i++) b += hs[i];
    hs[NH] = a;
    hs[NH + 1] = b;
  }
  __syncthreads();
  const int64_t p = pos[t];
  const float* cs = table ? table + p * dims : nullptr;             // [dims / 2][2]
  const int half = dims >> 1;
  E* row = k ? rows + slots[t] * ((int64_t)G * (d + dv)) : nullptr;
  for (int e = threadIdx.x; e < NH * d; e += blockDim.x) {
    const int hh = e / d, i = e - hh * d;
    const bool isq = hh < H;
    const int head = isq ? hh : hh - H;
    const EI* x = isq ? qr + head * d : kr + head * d;
    const E* nw = isq ? qn : kn;
    float rs = 1.f;
    if (nw) rs = whole ? 1.0f / sqrtf(hs[isq ? NH : NH + 1] / (float)((isq ? H : G) * d) + eps)
                       : 1.0f / sqrtf(hs[hh] / (float)d + eps);
    float val = normed(x, i, head, d, nw, whole, rs);
    if (cs && i < dims) {
      int pi, partner;
      bool first;
      if (layout == kHalf) {
        first = i < half;
        pi = first ? i : i - half;
        partner = first ? i + half : i - half;
      } else {
        first = !(i & 1);
        pi = i >> 1;
        partner = i ^ 1;
      }
      const float other = normed(x, partner, head, d, nw, whole, rs);
      const float c = cs[2 * pi], s = cs[2 * pi + 1];
      val = first ? val * c - other * s : val * c + other * s;
    }
    if (isq) qo[(t * H + head) * d + i] = val;
    else stf(row + head * d + i, val);
  }
  if (k)
    for (int e = threadIdx.x; e < G * dv; e += blockDim.x) stf(row + (int64_t)G * d + e, ldf(v + t * v_ld + e));
}

// ------------------------------------------------------------------ attention
constexpr int KT = 16;                                              // keys per tile

__device__ __forceinline__ int64_t first_key(int64_t p, int mask, int size) {
  if (mask == kWindow) return p - size + 1 > 0 ? p - size + 1 : 0;
  if (mask == kChunk) return p - p % size;
  return 0;
}

template <typename E> struct Chunk4;
template <> struct Chunk4<float> { typedef uint4 type; };
template <> struct Chunk4<__bf16> { typedef uint2 type; };

// LDS: qs f32 [HB][DQ] | per wave: tile E [KT][DP] (key d | value dv), weights f32 [HB][KT]
template <typename E, int RC, int HB>
__global__ void __launch_bounds__(256) masked_attn_k(const float* __restrict__ q, const E* __restrict__ rows, int bs,
                                                    const int32_t* __restrict__ bt, int bt_w,
                                                    const int32_t* __restrict__ seq_of, const int64_t* __restrict__ pos,
                                                    float scale, int mask, int size, const float* __restrict__ sink,
                                                    E* __restrict__ out, float* __restrict__ part, int H, int G, int d,
                                                    int dv, int DQ, int DP, float softcap, int keep, int cross) {
  extern __shared__ __align__(16) unsigned char smem[];
  typedef typename Chunk4<E>::type C4;
  const int rep = H / G;
  const int nhb = (rep + HB - 1) / HB;                              // head blocks per key head
  const int nsplit = gridDim.z, zs = blockIdx.z;
  // cross: the heads' weights are applied to the values of EVERY value head (grid y also walks the value heads); the
  // unnormalised partial results leave through ``part`` and the mixing of the heads follows in the combine kernel
  const int by = cross ? blockIdx.y / G : blockIdx.y;
  const int t = blockIdx.x, g = by / nhb, h0 = g * rep + (by % nhb) * HB;
  const int vg = cross ? blockIdx.y % G : g;
  const int nh = min(HB, g * rep + rep - h0);
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  float* qs = (float*)smem;
  const size_t q_bytes = (size_t)HB * DQ * sizeof(float);
  const size_t tile_bytes = ((size_t)KT * DP * sizeof(E) + 15) & ~(size_t)15;
  const size_t wave_bytes = tile_bytes + (size_t)HB * KT * sizeof(float);
  unsigned char* wbase = smem + q_bytes + wv * wave_bytes;
  E* kt = (E*)wbase;                                                // [KT][DP]
  float* pb = (float*)(wbase + tile_bytes);                         // [HB][KT]
  for (int i = threadIdx.x; i < HB * DQ; i += blockDim.x) {
    const int h = i / DQ, c = i - h * DQ;
    qs[i] = (h < nh && c < d) ? q[((int64_t)t * H + h0 + h) * d + c] : 0.f;
  }
  for (int i = lane; i < KT * DP; i += 64) stf(kt + i, 0.f);        // pad columns and unfilled rows stay finite
  __syncthreads();
  const int64_t p = pos[t];
  const int64_t lo = first_key(p, mask, size);
  const int32_t* tab = bt + (int64_t)seq_of[t] * bt_w;
  const int tile0 = (int)(lo / KT), ntiles = (int)(p / KT) + 1;
  // a window that keeps the sequence's first tokens: their tiles (those before the window's first) are walked first
  const int nkeep = keep > 0 ? min(tile0, (keep + KT - 1) / KT) : 0;
  const int nwalk = nkeep + ntiles - tile0;
  const int64_t RW = (int64_t)G * (d + dv);                         // cache row width
  const int D = d + dv;
  float m[HB], l[HB], o[HB][RC];
#pragma unroll
  for (int h = 0; h < HB; h++) {
    m[h] = -INFINITY;
    l[h] = 0.f;
#pragma unroll
    for (int c = 0; c < RC; c++) o[h][c] = 0.f;
  }
  const int kj = lane & (KT - 1), grp = lane / KT;                  // 4 lanes share a key
  const int d4 = (d + 3) >> 2;                                      // 4-element steps of a key (LDS pad is zero)
  for (int it = zs * NW + wv; it < nwalk; it += NW * nsplit) {
    const int ti = it < nkeep ? it : tile0 + (it - nkeep);
    const int64_t k0 = (int64_t)ti * KT;
    const int nvalid = (int)min((int64_t)KT, p - k0 + 1);
    const int64_t row0 = (int64_t)tab[k0 / bs] * bs + (k0 % bs);
    if (((d | dv) & 3) == 0) {
      // 4-element chunks (the key part, then the value part of every row), four requests in flight per lane
      const int cd = d >> 2, cpr = (d + dv) >> 2, n4 = nvalid * cpr;
      for (int i0 = lane; i0 < n4; i0 += 256) {
        C4 v[4];
        int dst[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          const int i = i0 + 64 * u;
          if (i < n4) {
            const int j = i / cpr, c = i - j * cpr;
            const E* src = rows + (row0 + j) * RW +
                           (c < cd ? (int64_t)g * d + 4 * c : (int64_t)G * d + (int64_t)vg * dv + 4 * (c - cd));
            v[u] = *(const C4*)src;
            dst[u] = j * DP + (c < cd ? 4 * c : DQ + 4 * (c - cd));
          }
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
          if (i0 + 64 * u < n4) *(C4*)(kt + dst[u]) = v[u];
      }
    } else {
      for (int i = lane; i < nvalid * D; i += 64) {
        const int j = i / D, c = i - j * D;
        const E* src = rows + (row0 + j) * RW + (c < d ? (int64_t)g * d + c : (int64_t)G * d + (int64_t)vg * dv + (c - d));
        kt[j * DP + (c < d ? c : DQ + (c - d))] = *src;
      }
    }
    wave_sync();
    float s[HB];
#pragma unroll
    for (int h = 0; h < HB; h++) s[h] = 0.f;
    const bool valid = kj < nvalid && (k0 + kj >= lo || k0 + kj < keep);
    if (valid) {
      const E* kr = kt + kj * DP;
      for (int c4 = grp * d4 / 4; c4 < (grp + 1) * d4 / 4; c4++) {
        const int c = c4 * 4;
        const float k0v = ldf(kr + c), k1v = ldf(kr + c + 1), k2v = ldf(kr + c + 2), k3v = ldf(kr + c + 3);
#pragma unroll
        for (int h = 0; h < HB; h++) {
          const float4 qv = *(const float4*)(qs + h * DQ + c);
          s[h] = fmaf(qv.x, k0v, fmaf(qv.y, k1v, fmaf(qv.z, k2v, fmaf(qv.w, k3v, s[h]))));
        }
      }
    }
#pragma unroll
    for (int h = 0; h < HB; h++) {
      s[h] += __shfl_xor(s[h], 16, 64);
      s[h] += __shfl_xor(s[h], 32, 64);
    }
#pragma unroll
    for (int h = 0; h < HB; h++) {
      float sv = s[h] * scale;
      if (softcap > 0.f) sv = softcap * tanhf(sv / softcap);
      if (!valid) sv = -INFINITY;
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
    const int nv4 = (nvalid + 3) & ~3;                              // weights past nvalid are 0, rows finite
    for (int j = 0; j < nv4; j += 4) {
      float vv[4][RC];
#pragma unroll
      for (int jj = 0; jj < 4; jj++)
#pragma unroll
        for (int c = 0; c < RC; c++) {
          const int col = lane + 64 * c;
          vv[jj][c] = col < dv ? ldf(kt + (j + jj) * DP + DQ + col) : 0.f;
        }
#pragma unroll
      for (int h = 0; h < HB; h++) {
        const float4 w4 = *(const float4*)(pb + h * KT + j);
#pragma unroll
        for (int c = 0; c < RC; c++)
          o[h][c] = fmaf(w4.x, vv[0][c], fmaf(w4.y, vv[1][c], fmaf(w4.z, vv[2][c], fmaf(w4.w, vv[3][c], o[h][c]))));
      }
    }
    wave_sync();
  }
  // merge the waves through the (re-used) LDS: every wave leaves (o, m, l) per head
  __syncthreads();
  const int MS = HB * (dv + 2);
  float* mg = (float*)smem + (size_t)wv * MS;
#pragma unroll
  for (int h = 0; h < HB; h++) {
#pragma unroll
    for (int c = 0; c < RC; c++) {
      const int col = lane + 64 * c;
      if (col < dv) mg[h * (dv + 2) + col] = o[h][c];
    }
    if (lane == 0) {
      mg[h * (dv + 2) + dv] = m[h];
      mg[h * (dv + 2) + dv + 1] = l[h];
    }
  }
  __syncthreads();
  const float* m0 = (const float*)smem;
  for (int i = threadIdx.x; i < nh * (dv + 2); i += blockDim.x) {
    const int h = i / (dv + 2), c = i - h * (dv + 2);
    float M = -INFINITY;
    for (int w = 0; w < NW; w++) M = fmaxf(M, m0[(size_t)w * MS + h * (dv + 2) + dv]);
    float L = 0.f, O = 0.f;
    for (int w = 0; w < NW; w++) {
      const float* gp = m0 + (size_t)w * MS + h * (dv + 2);
      const float mw = gp[dv];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      L += gp[dv + 1] * f;
      if (c < dv) O += gp[c] * f;
    }
    if (cross) {
      float* pp = part + ((((int64_t)t * H + h0 + h) * G + vg) * nsplit + zs) * (dv + 2);
      pp[c] = c < dv ? O : (c == dv ? M : L);
    } else if (nsplit > 1) {
      float* pp = part + (((int64_t)t * H + h0 + h) * nsplit + zs) * (dv + 2);
      pp[c] = c < dv ? O : (c == dv ? M : L);
    } else if (c < dv) {
      if (sink) {                                                   // one more term of the denominator
        const float sk = sink[h0 + h];
        const float M2 = fmaxf(M, sk);
        const float f = expf(M - M2);
        O *= f;
        L = L * f + expf(sk - M2);
      }
      stf(out + ((int64_t)t * H + h0 + h) * dv + c, O / L);
    }
  }
}

// merge of the key splits: part [T, H, nsplit, dv + 2] -> out [T, H, dv].  One wave per (token, head): lane z
// holds split z's (max, sum) (nsplit <= 64), the wave reduces them, then every lane sums its value columns
template <typename E>
__global__ void __launch_bounds__(64) masked_attn_combine_k(const float* __restrict__ part, const float* __restrict__ sink,
                                                           E* __restrict__ out, int H, int dv, int nsplit) {
  __shared__ float wz[64];
  const int64_t th = (int64_t)blockIdx.x * H + blockIdx.y;
  const float* pp = part + th * nsplit * (dv + 2);
  const int lane = threadIdx.x;
  const float mz = lane < nsplit ? pp[(size_t)lane * (dv + 2) + dv] : -INFINITY;
  const float lz = lane < nsplit ? pp[(size_t)lane * (dv + 2) + dv + 1] : 0.f;
  const float sk = sink ? sink[blockIdx.y] : -INFINITY;
  const float M = fmaxf(wave_max(mz), sk);
  const float f = mz == -INFINITY ? 0.f : expf(mz - M);
  wz[lane] = f;
  // the splits' sums in index order (a fixed order, whatever the lanes do)
  __syncthreads();
  float L = sink ? expf(sk - M) : 0.f;
  for (int z = 0; z < nsplit; z++) L += __shfl(lz, z, 64) * wz[z];
  const float inv = 1.0f / L;
  for (int c = lane; c < dv; c += 64) {
    float O = 0.f;
    for (int z = 0; z < nsplit; z++) O = fmaf(pp[(size_t)z * (dv + 2) + c], wz[z], O);
    stf(out + th * dv + c, O * inv);
  }
}

// merge of the key splits and mixing of the heads' weights after the softmax:
//   out[t, h] = sum_g talk[h, g] (sum_j w_g(j) value_j[c])   with c = h's value head,
// part [T, H, G, nsplit, dv + 2] holds, for query head g and value head c, the unnormalised sums of every key split.
// One wave per (token, output head); dv <= 512
template <typename E>
__global__ void __launch_bounds__(512) masked_attn_talk_combine_k(const float* __restrict__ part,
                                                                 const float* __restrict__ sink,
                                                                 const float* __restrict__ talk, E* __restrict__ out,
                                                                 int H, int G, int dv, int nsplit) {
  extern __shared__ float cs[];                                     // [NW][64] split factors, then [NW][dv] sums
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, c = h / (H / G), lane = threadIdx.x & 63, wv = threadIdx.x >> 6, NW = blockDim.x >> 6;
  float* wz = cs + wv * 64;
  float* sums = cs + NW * 64;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = 0.f;
  for (int g = wv; g < H; g += NW) {                                // wave w: source heads w, w + NW, ...
    const float* pp = part + ((t * H + g) * G + c) * (int64_t)nsplit * (dv + 2);
    const float mz = lane < nsplit ? pp[(size_t)lane * (dv + 2) + dv] : -INFINITY;
    const float lz = lane < nsplit ? pp[(size_t)lane * (dv + 2) + dv + 1] : 0.f;
    const float sk = sink ? sink[g] : -INFINITY;
    const float M = fmaxf(wave_max(mz), sk);
    const float f = mz == -INFINITY ? 0.f : expf(mz - M);
    wave_sync();
    wz[lane] = f;
    wave_sync();
    float L = sink ? expf(sk - M) : 0.f;
    for (int z = 0; z < nsplit; z++) L += __shfl(lz, z, 64) * wz[z];   // index order, whatever the lanes do
    const float coef = talk[h * H + g] / L;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int col = lane + 64 * i;
      if (col < dv) {
        float O = 0.f;
        for (int z = 0; z < nsplit; z++) O = fmaf(pp[(size_t)z * (dv + 2) + col], wz[z], O);
        acc[i] = fmaf(coef, O, acc[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int col = lane + 64 * i;
    if (col < dv) sums[wv * dv + col] = acc[i];
  }
  __syncthreads();
  for (int col = threadIdx.x; col < dv; col += blockDim.x) {
    float o = 0.f;
    for (int w = 0; w < NW; w++) o += sums[w * dv + col];           // the waves in order
    stf(out + (t * H + h) * dv + col, o);
  }
}

// mixing of the heads' weights between the chunk products: w f32 [pieces, G, Lq, rep, L] (normalised softmax
// weights) -> mixed weights of the same layout, w'[.., h, ..] = sum_g talk[h, g] w[.., g, ..] with h = key head * rep +
// r; bf16: as pairs hi + lo in hl [R, 2 L] (a row's hi halves, then its lo halves); f32: out32 [R, L].
// A thread per key column, the piece-and-query's H weights of that column staged in LDS
template <typename E>
__global__ void __launch_bounds__(64) talk_mix_k(const float* __restrict__ w, const float* __restrict__ talk, int Lq, int L,
                                                int G, int rep, E* __restrict__ hl, float* __restrict__ out32) {
  extern __shared__ float col[];                                    // [H][64]
  const int H = G * rep;
  const int piece = blockIdx.x / Lq, qi = blockIdx.x % Lq;
  const int j = blockIdx.y * 64 + threadIdx.x;
  if (j >= L) return;
  const int64_t prow = (int64_t)piece * G * Lq * rep;
  for (int g = 0; g < H; g++) {
    const int64_t row = prow + ((int64_t)(g / rep) * Lq + qi) * rep + g % rep;
    col[g * 64 + threadIdx.x] = w[row * L + j];
  }
  for (int h = 0; h < H; h++) {
    float a = 0.f;
    for (int g = 0; g < H; g++) a = fmaf(talk[h * H + g], col[g * 64 + threadIdx.x], a);
    const int64_t row = prow + ((int64_t)(h / rep) * Lq + qi) * rep + h % rep;
    if (hl) {
      const E hv = (E)a;
      hl[row * 2 * L + j] = hv;
      hl[row * 2 * L + L + j] = (E)(a - (float)hv);
    } else {
      out32[row * L + j] = a;
    }
  }
}

// ------------------------------------------------------------------ softmax between the chunk products
// window == 0: a piece of a chunk (query tok sees keys 0 .. L - Lq + tok).  window > 0: a block of queries of a
// sliding window: query tok stands at position q0 + tok; the first nkeep columns are kept first tokens (always
// visible), column nkeep + jj is the key at position k0 + jj, visible when it is not ahead of the query and inside
// the window (or before position ``keep``)
template <typename E>
__global__ void __launch_bounds__(256) chunk_softmax_k(float* __restrict__ sc, int Lq, int L, int G, int rep, float scale,
                                                      const float* __restrict__ sink, E* __restrict__ hi, float softcap,
                                                      int window, int keep, int nkeep, int64_t q0, int64_t k0) {
  __shared__ float red[16];
  const int64_t row = blockIdx.x;
  const int tok = (int)((row / rep) % Lq);                          // the piece's queries are its last Lq positions
  const int h = (int)((row / ((int64_t)rep * Lq)) % G) * rep + (int)(row % rep);
  const int64_t p = q0 + tok;
  const int nk = window > 0 ? (int)min((int64_t)L, nkeep + (p - k0) + 1) : L - Lq + tok + 1;
  // the first column of the window's own keys (columns nkeep .. first - 1 are seen only if kept)
  const int first = window > 0 ? nkeep + (int)max((int64_t)0, p - window + 1 - k0) : 0;
  auto vis = [&](int j) -> bool { return window <= 0 || j < nkeep || j >= first || k0 + (j - nkeep) < keep; };
  float* s = sc + row * L;
  const float sk = sink ? sink[h] : -INFINITY;
  float mx = sk;
  for (int j = threadIdx.x; j < nk; j += blockDim.x) {
    float v = s[j] * scale;
    if (softcap > 0.f) v = softcap * tanhf(v / softcap);
    if (!vis(j)) v = -INFINITY;
    s[j] = v;
    mx = fmaxf(mx, v);
  }
  mx = wave_max(mx);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
  __syncthreads();
  for (int i = 0; i < (int)(blockDim.x >> 6); i++) mx = fmaxf(mx, red[i]);
  float sum = 0.f;
  for (int j = threadIdx.x; j < nk; j += blockDim.x) {
    const float e = expf(s[j] - mx);                               // a masked column: exp(-inf) = 0
    s[j] = e;
    sum += e;
  }
  const float inv = 1.0f / (block_sum(sum, red) + (sink ? expf(sk - mx) : 0.f));
  for (int j = threadIdx.x; j < L; j += blockDim.x) {
    const float w = j < nk ? s[j] * inv : 0.f;
    if (hi) {                                                      // [R, 2 L]: hi halves, then lo halves
      const E hv = (E)w;
      hi[row * 2 * L + j] = hv;
      hi[row * 2 * L + L + j] = (E)(w - (float)hv);
    } else {
      s[j] = w;
    }
  }
}

template <typename E>
__global__ void __launch_bounds__(256) sigmoid_gate_k(E* __restrict__ o, const E* __restrict__ g, int64_t g_ld, int64_t n,
                                                     int C) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / C;
    const int c = (int)(i - t * C);
    stf(o + i, ldf(o + i) / (1.0f + expf(-ldf(g + t * g_ld + c))));
  }
}

int pad4(int n) { return (n + 3) & ~3; }
// key | value row of a tile: the key part padded to DQ (a multiple of 4, zero filled), the row to 4 (mod 8) elements
int tile_row(int d, int dv) {
  const int n = pad4(d) + pad4(dv);
  return n + ((12 - (n & 7)) & 7);
}

}  // namespace

void qkv_norm_rope_store(bool in_bf16, bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld,
                         const void* v, int64_t v_ld, const void* qn, const void* kn, bool whole, float eps,
                         const float* table, int max_pos, int dims, int layout, const int64_t* pos, const int64_t* slots,
                         void* rows, int64_t num_rows, float* qo, int T, int H, int G, int d, int dv, hipStream_t st) {
  (void)max_pos;
  (void)num_rows;
  if (T <= 0) return;
  const size_t lds = (size_t)(H + G + 2) * sizeof(float);
  // few tokens (decode): a thread per value or two, so that no thread walks a chain of dependent loads
  const int64_t vals = (int64_t)(H + G) * d;
  const int nt = T > 64 ? 256 : (vals >= 1024 ? 1024 : (int)((vals + 63) / 64 * 64));
#define MA_STORE(EI, E)                                                                                                 \
  qkv_store_k<EI, E><<<T, nt, lds, st>>>((const EI*)q, q_ld, (const EI*)k, k_ld, (const EI*)v, v_ld, (const E*)qn,      \
                                         (const E*)kn, whole, eps, table, dims, layout, pos, slots, (E*)rows, qo, H, G, \
                                         d, dv)
  if (bf16 && in_bf16) MA_STORE(__bf16, __bf16);
  else if (bf16) MA_STORE(float, __bf16);
  else MA_STORE(float, float);
#undef MA_STORE
}

int masked_attention_plan(bool bf16, int rep, int d, int dv, int* nw, int* hbo) {
  if (d < 1 || dv < 1 || dv > 512) return -1;
  const int hb = rep >= 8 ? 8 : (rep >= 4 ? 4 : (rep >= 2 ? 2 : 1));
  const size_t eb = bf16 ? 2 : 4;
  const size_t q_bytes = (size_t)hb * pad4(d) * 4;
  const size_t wave = (((size_t)KT * tile_row(d, dv) * eb + 15) & ~(size_t)15) + (size_t)hb * KT * 4;
  for (int w = 4; w >= 1; w--) {
    const size_t tiles = q_bytes + (size_t)w * wave;
    const size_t merge = (size_t)w * hb * (dv + 2) * 4;
    const size_t total = tiles > merge ? tiles : merge;
    if (total <= 64 * 1024) {
      *nw = w;
      *hbo = hb;
      return (int)total;
    }
  }
  return -1;
}

int masked_attention_splits(bool bf16, int T, int H, int G, int d, int dv, int max_keys, bool cross) {
  int NW = 0, hb = 0;
  if (masked_attention_plan(bf16, H / G, d, dv, &NW, &hb) < 0) return 1;
  const int64_t blocks = (int64_t)T * G * ((H / G + hb - 1) / hb) * (cross ? G : 1);
  const int tiles = (max_keys + KT - 1) / KT + 1;
  int ns = (int)((1024 + blocks - 1) / blocks);                    // ~4 workgroups per CU
  ns = ns > (tiles + NW - 1) / NW ? (tiles + NW - 1) / NW : ns;
  return ns < 1 ? 1 : (ns > 64 ? 64 : ns);
}

void masked_attention(bool bf16, const float* q, const void* rows, int bs, const int32_t* block_tables, int bt_width,
                      const int32_t* seq_of, const int64_t* pos, float scale, int mask, int size, const float* sink,
                      void* out, float* part, int nsplit, int T, int H, int G, int d, int dv, float softcap, int keep,
                      const float* talk, hipStream_t st) {
  if (T <= 0) return;
  const int cross = talk ? 1 : 0;
  if (mask != kWindow) keep = 0;
  int NW = 0, hb = 0;
  const int rep = H / G;
  const int lds = masked_attention_plan(bf16, rep, d, dv, &NW, &hb);
  if (lds < 0) return;                       // refused by the caller beforehand
  const int DQ = pad4(d), DP = tile_row(d, dv);
  const int rc = (dv + 63) / 64;
  dim3 grid(T, G * ((rep + hb - 1) / hb) * (cross ? G : 1), nsplit), block(64 * NW);
#define MA_LAUNCH(E, RC, HBV)                                                                                          \
  masked_attn_k<E, RC, HBV><<<grid, block, lds, st>>>(q, (const E*)rows, bs, block_tables, bt_width, seq_of, pos, scale, \
                                                      mask, size, sink, (E*)out, part, H, G, d, dv, DQ, DP, softcap,   \
                                                      keep, cross)
#define MA_RC(E, HBV)                                 \
  if (rc <= 1) MA_LAUNCH(E, 1, HBV);                  \
  else if (rc <= 2) MA_LAUNCH(E, 2, HBV);             \
  else if (rc <= 4) MA_LAUNCH(E, 4, HBV);             \
  else MA_LAUNCH(E, 8, HBV)
#define MA_HB(E)                                      \
  if (hb == 8) { MA_RC(E, 8); }                       \
  else if (hb == 4) { MA_RC(E, 4); }                  \
  else if (hb == 2) { MA_RC(E, 2); }                  \
  else { MA_RC(E, 1); }
  if (bf16) { MA_HB(__bf16) } else { MA_HB(float) }
#undef MA_HB
#undef MA_RC
#undef MA_LAUNCH
  if (cross) {
    const int cw = H < 8 ? H : 8;                                   // waves: each merges some of the source heads
    const size_t cl = (size_t)cw * (64 + dv) * sizeof(float);
    if (bf16)
      masked_attn_talk_combine_k<__bf16><<<dim3(T, H), 64 * cw, cl, st>>>(part, sink, talk, (__bf16*)out, H, G, dv, nsplit);
    else
      masked_attn_talk_combine_k<float><<<dim3(T, H), 64 * cw, cl, st>>>(part, sink, talk, (float*)out, H, G, dv, nsplit);
  } else if (nsplit > 1) {
    if (bf16) masked_attn_combine_k<__bf16><<<dim3(T, H), 64, 0, st>>>(part, sink, (__bf16*)out, H, dv, nsplit);
    else masked_attn_combine_k<float><<<dim3(T, H), 64, 0, st>>>(part, sink, (float*)out, H, dv, nsplit);
  }
}

void chunk_softmax(bool bf16, float* sc, int64_t R, int Lq, int L, int G, int rep, float scale, const float* sink,
                   void* hl, float softcap, int window, int keep, int nkeep, int64_t q0, int64_t k0, hipStream_t st) {
  if (R <= 0 || L <= 0) return;
  if (bf16)
    chunk_softmax_k<__bf16><<<(unsigned)R, 256, 0, st>>>(sc, Lq, L, G, rep, scale, sink, (__bf16*)hl, softcap, window,
                                                         keep, nkeep, q0, k0);
  else
    chunk_softmax_k<float><<<(unsigned)R, 256, 0, st>>>(sc, Lq, L, G, rep, scale, sink, (float*)nullptr, softcap, window,
                                                        keep, nkeep, q0, k0);
}

void talk_mix(bool bf16, const float* w, const float* talk, int64_t pieces, int Lq, int L, int G, int rep, void* hl,
              float* out32, hipStream_t st) {
  if (pieces <= 0 || L <= 0) return;
  const dim3 grid((unsigned)(pieces * Lq), (L + 63) / 64);
  const size_t lds = (size_t)G * rep * 64 * sizeof(float);
  if (bf16) talk_mix_k<__bf16><<<grid, 64, lds, st>>>(w, talk, Lq, L, G, rep, (__bf16*)hl, nullptr);
  else talk_mix_k<float><<<grid, 64, lds, st>>>(w, talk, Lq, L, G, rep, (float*)nullptr, out32);
}

void sigmoid_gate(bool bf16, void* o, const void* g, int64_t g_ld, int64_t T, int C, hipStream_t st) {
  const int64_t n = T * C;
  if (n <= 0) return;
  const int blocks = (int)((n + 255) / 256 > 65535 ? 65535 : (n + 255) / 256);
  if (bf16) sigmoid_gate_k<__bf16><<<blocks, 256, 0, st>>>((__bf16*)o, (const __bf16*)g, g_ld, n, C);
  else sigmoid_gate_k<float><<<blocks, 256, 0, st>>>((float*)o, (const float*)g, g_ld, n, C);
}

}  // namespace ma
}  // namespace illm
