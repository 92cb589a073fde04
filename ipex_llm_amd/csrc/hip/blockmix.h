// Launchers of the kernels of the parallel-residual hybrid blocks
// (blockmix_elem.hip, blockmix_attn.hip, blockmix_moe.hip): RMS norms, the
// short causal convolution with its per-sequence state, grouped-query
// attention with mixed head scores over paged [keys | values] rows, and
// clamped-GLU experts behind a sigmoid router.  ``bf16`` selects the
// activation element type (bf16 when true, f32 when false); everything the
// kernels accumulate is f32 either way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace illm {
namespace bm {

// ---- element-wise (blockmix_elem.hip)
// h = x / sqrt(mean(x^2) + eps) * w; w holds nw = 1 or W numbers; ha: h in the activation type (bf16 only)
void rms_norm_rows(bool bf16, const float* x, const void* w, int nw, float* h, void* ha, int T, int W, float eps,
                   hipStream_t st);
// x += y / sqrt(mean(y^2) + eps) * w; xa: x in the activation type (bf16 only, may be null)
void add_rms_norm(bool bf16, float* x, const void* y, const void* w, void* xa, int T, int W, float eps, hipStream_t st);
// x += y (y in the activation type, may be null), then out = x / sqrt(mean(x^2) + eps) * w in the activation type
void add_rms_norm_rows(bool bf16, float* x, const void* y, const void* w, void* out, int T, int W, float eps,
                       hipStream_t st);
// x += s1 * y1 + s2 * (y2 + y3); s1, s2 f32 [W] or null; y2 f32 when y2_f32 else activation type; y2, y3 may be null
void residual_add_scaled(bool bf16, float* x, const void* y1, const float* s1, const void* y2, bool y2_f32,
                         const void* y3, const float* s2, void* xa, int64_t T, int W, hipStream_t st);
// out = h + conv(h) over time, per channel; state f32 [slots, taps - 1, W]; then the state is advanced
void canon_conv(bool bf16, const float* h, const float* w, int taps, float* state, const int32_t* cu,
                const int32_t* seq_of, const int32_t* slots, const int64_t* pos, void* out, int T, int B, int W,
                hipStream_t st);
// rms_norm_rows + canon_conv in one launch (h f32, ha: h in the activation type (bf16 only), out = h + conv(h));
// single: every sequence brings exactly one token (the state is advanced by the same launch)
void norm_canon(bool bf16, const float* x, const void* g, int ng, float eps, const float* w, int taps, float* state,
                const int32_t* cu, const int32_t* seq_of, const int32_t* slots, const int64_t* pos, float* h, void* ha,
                void* out, int T, int B, int W, bool single, hipStream_t st);
void relu_sq(bool bf16, const void* y, void* out, int64_t n, hipStream_t st);
void glu_clamp(bool bf16, const void* gu, void* out, int64_t T, int64_t I, float limit, float alpha, hipStream_t st);
// out = gelu_tanh(z) * table[ids, offset : offset + n]
void side_gate(bool bf16, const void* z, const void* table, int64_t ld, int64_t vocab, const int64_t* ids, int offset,
               void* out, int T, int n, hipStream_t st);

// ---- attention (blockmix_attn.hip)
// q [T, H, d] / k [T, G, d] rows of q_ld / k_ld elements; norm weights [d] or null; table f32 [max_pos, dims / 2, 2];
// rows [num_rows, 2 G d]; qo f32 [T, H, d]
void qk_norm_rope_store(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* qn,
                        const void* kn, float eps, const float* table, int max_pos, int dims, const int64_t* pos,
                        const int64_t* slots, void* rows, int64_t num_rows, float* qo, int T, int H, int G, int d,
                        hipStream_t st);
// dynamic LDS of the flash kernel (and its key tile); < 0: these sizes do not fit
int talk_attention_plan(bool bf16, int H, int G, int d, int* kt);
int talk_attention_splits(bool bf16, int T, int H, int G, int d, int max_ctx);
// part: f32 scratch [T, nsplit, H, d + 2] when nsplit > 1
void talk_attention(bool bf16, const float* q, const void* rows, int bs, const int32_t* block_tables, int bt_width,
                    const int32_t* seq_of, const int64_t* pos, float scale, const float* talk, const void* gate,
                    int64_t g_st, void* out, float* part, int nsplit, int T, int H, int G, int d, hipStream_t st);
// long portions of one sequence on the matrix cores (bf16 rows): tokens t0 .. t0 + n - 1 of the step at consecutive
// positions, bt: the sequence's block table row; writes out rows t0 .. t0 + n - 1 ([T, H d] bf16)
bool talk_prefill_fits(int H, int G, int d);
// part: f32 scratch [n, nsplit, H, d + 2] when nsplit > 1 (talk_prefill_splits)
int talk_prefill_splits(int n, int max_keys);
void talk_prefill(const float* q, const void* rows, int bs, const int32_t* bt, const int64_t* pos, int t0, int n,
                  float scale, const float* talk, const void* gate, int64_t g_st, void* out, float* part, int nsplit,
                  int H, int G, int d, hipStream_t st);
// rows [R, L] of raw scores (row i = token i / H, head i % H): scaled, mixed over the heads of a token, masked by
// pos[i / H], softmax; bf16: weights leave as hi + lo bf16 pairs (row stride L), f32 (hi == null): in place
void talk_softmax(bool bf16, float* sc, const int64_t* pos, int H, float scale, const float* talk, int64_t nt, int L,
                  void* hi, void* lo, hipStream_t st);

// ---- experts (blockmix_moe.hip)
// mode 0: the largest sigmoid(z) win and are the weights; 1: the largest logits win, softmax over the winners (top <= 64)
void moe_route(const float* z, int T, int E, int top, int32_t* idx, float* w, int mode, hipStream_t st);
// off int32 [E + 1], sorted int32 [P]: pair ids (token * top + k) grouped by expert
void moe_align(const int32_t* idx, int P, int E, int32_t* off, int32_t* sorted, hipStream_t st);
// y [P, ff] (sorted order) = glu(W_gu[e] (w_p h_token)), glu = g sigmoid(alpha g) (u + up_shift) with the clamps;
// weigh_out: the input is h_token itself (the routing weight multiplies the result of moe_down instead)
void moe_glu(bool bf16, const void* h, const int32_t* off, const int32_t* sorted, const float* wts, int top,
             const void* w_gu, void* y, int P, int E, int ff, int W, float limit, float alpha, float up_shift,
             bool weigh_out, hipStream_t st);
// out f32 [P, W] (by pair id) = W_down[e] y_p (times wts[pair] when wts is not null)
void moe_down(bool bf16, const void* y, const int32_t* off, const int32_t* sorted, const void* w_down, float* out,
              int P, int E, int ff, int W, const float* wts, hipStream_t st);

}  // namespace bm
}  // namespace illm
