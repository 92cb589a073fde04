// Launchers of the state-space mixer's kernels (ssm.hip): the short causal
// convolution with bias and SiLU over per-sequence state, the selective scan
// over f32 state slots, and the gated group norm.  ``bf16`` selects the
// activation element type (bf16 when true, f32 when false); everything the
// kernels accumulate is f32 either way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace illm {
namespace ssm {

// out f32 [T, C] = silu(b + sum_j w[:, j] u_(t - taps + 1 + j)) (b null: no bias; act false: no SiLU); u rows of u_ld
// elements; w f32 [C, taps], b f32 [C];
// state f32 [slots, taps - 1, C], advanced afterwards (by the same launch when ``single``: every sequence brings
// exactly one token)
void conv_silu(bool bf16, const void* u, int64_t u_ld, const float* w, const float* b, int taps, float* state,
               const int32_t* cu, const int32_t* seq_of, const int32_t* slots, const int64_t* pos, float* out, int T,
               int B, int C, bool single, bool act, hipStream_t st);

// largest state size N the scan holds
constexpr int kScanMaxState = 1024;
// x f32 [T, H, P] (rows of x_ld), Bm / Cm f32 [T, G, N] (rows of b_ld / c_ld), dt [T, H] activation type (rows of
// dt_ld); S f32 [slots, H, N, P]; out f32 [T, H, P] contiguous
void selective_scan(bool bf16, const float* x, int64_t x_ld, const float* Bm, int64_t b_ld, const float* Cm,
                    int64_t c_ld, const void* dt, int64_t dt_ld, const float* dt_bias, const float* a_log,
                    const float* d_skip, float* S, const int32_t* cu, const int32_t* slots, const int64_t* pos,
                    float* out, int B, int H, int P, int G, int N, hipStream_t st);

// out [T, C] = group_rms_norm(y * silu(z)) * w; y f32 [T, C], z rows of z_ld elements
void gated_group_norm(bool bf16, const float* y, const void* z, int64_t z_ld, const void* w, void* out, int T, int C,
                      int groups, float eps, hipStream_t st);

}  // namespace ssm
}  // namespace illm
