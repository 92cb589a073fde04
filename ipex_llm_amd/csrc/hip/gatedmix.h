// Launchers of the kernels of the gated recurrent mixers and the two-norm
// parallel blocks (gatedmix.hip): a pair of LayerNorms with the token shift,
// the minGRU recurrence, the gated-linear-attention recurrence, the per-head
// RMS norm with a SiLU gate, the mean of two RMS-normed results and the tanh
// cap.  ``bf16`` selects the activation element type (bf16 when true, f32
// when false); everything the kernels accumulate is f32 either way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace illm {
namespace gm {

// x f32 [T, W]; w1 / w2 [W] (w2 null: one norm); mu f32 [W] or null (no shift: state, cu, seq_of, slots, pos, last
// unused); state f32 [slots, W]; h1 / h2 [T, W]; last: f32 scratch [B, W] (used unless ``single``)
void layer_norm_pair_shift(bool bf16, const float* x, const void* w1, const void* w2, const float* mu, float eps,
                           float* state, const int32_t* cu, const int32_t* seq_of, const int32_t* slots,
                           const int64_t* pos, void* h1, void* h2, float* last, int T, int B, int W, bool single,
                           hipStream_t st);

// y [T, 3 width] rows of y_ld elements = [z_pre | u | g_pre]; state f32 [slots, width]; out [T, width];
// max_n: the longest portion (chooses the pieces per portion)
void mingru_scan(bool bf16, const void* y, int64_t y_ld, int width, float* state, const int32_t* cu,
                 const int32_t* slots, const int64_t* pos, void* out, int B, int max_n, hipStream_t st);

// largest key size per head the scan holds
constexpr int kGlaMaxDim = 1024;
// q / k / a [T, H, d], v [T, H, dv] (rows of *_ld elements, heads contiguous); S f32 [slots, H, d, dv]; out f32 [T, H, dv]
void gla_scan(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
              const void* a, int64_t a_ld, float tau, float q_scale, float* S, const int32_t* cu, const int32_t* slots,
              const int64_t* pos, float* out, int B, int H, int d, int dv, hipStream_t st);

// a long portion cut into pieces that run side by side: P f32 [NP, H, d] = the product of every piece's decays
// (cu int32 [NP + 1]: the pieces' token borders), and the chain of the pieces' start states: Z / Sin f32
// [NP + 1, H, d, dv] (Z: every piece's end state from the first pass), seqs int32 [nseq, 2] = first piece, pieces
void gla_piece_decay(bool bf16, const void* a, int64_t a_ld, const int32_t* cu, float tau, float* P, int NP, int H, int d,
                     hipStream_t st);
void gla_chain(const float* Z, float* Sin, const float* P, const int32_t* seqs, int nseq, int H, int d, int dv,
               hipStream_t st);

// o f32 [T, H, dv]; w [dv]; gate rows of g_ld elements; out [T, H dv]
void head_rms_silu(bool bf16, const float* o, const void* w, const void* gate, int64_t g_ld, void* out, int T, int H,
                   int dv, float eps, hipStream_t st);

// out = (rms_norm(a) wa + rms_norm(b) wb) / 2, rows [T, W]
void rms_pair_mean(bool bf16, const void* a, const void* b, const void* wa, const void* wb, void* out, int T, int W,
                   float eps, hipStream_t st);

// x <- cap tanh(x / cap)
void softcap(float* x, int64_t n, float cap, hipStream_t st);

}  // namespace gm
}  // namespace illm
