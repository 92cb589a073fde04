// Launchers of the sequence-mixing kernels (seqmix.hip): latent attention
// over a paged latent cache, the mLSTM matrix-memory scan over state slots,
// and the fused element-wise steps of the hybrid decoders.  ``bf16`` selects
// the activation element type (bf16 when true, f32 when false); everything
// the kernels accumulate is f32 either way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace illm {
namespace sm {

void embed_bigram(bool bf16, const int64_t* ids, const int64_t* prev, const void* embed, const void* bigram, float* out,
                  int T, int W, int64_t vocab, int64_t buckets, int64_t mul_prev, int64_t mul_cur, hipStream_t st);

// x += mult * LN(y) * w (f32 residual rows); xa: x in the activation type (bf16 only, may be null)
void add_scaled_layer_norm(bool bf16, float* x, const void* y, const void* w, void* xa, int T, int W, float eps,
                           float mult, hipStream_t st);
void layer_norm(bool bf16, const float* x, const void* w, void* out, int T, int W, float eps, hipStream_t st);

// table f32 [max_pos, dims / 2, 2]
void rope_rows(bool bf16, void* q, int T, int H, int Dh, int offset, const float* table, int max_pos, int dims,
               const int64_t* pos, hipStream_t st);
// dkv rows of ``ld`` elements: [rank | rot_dim] used
void latent_kv_store(bool bf16, const void* dkv, int64_t ld, const void* norm_w, float eps, int rank, int rot_dim,
                     const float* table, int max_pos, int dims, const int64_t* pos, const int64_t* slots, void* rows,
                     int64_t num_rows, int T, hipStream_t st);

// how much dynamic LDS the attention launch takes (and its tile / wave / head-group sizes); < 0: does not fit
int latent_attention_plan(bool bf16, int H, int r, int dr, int* kt, int* nw, int* hb);
// key splits (grid z) for T query tokens whose longest context is max_ctx
int latent_attention_splits(bool bf16, int T, int H, int r, int dr, int max_ctx);
// part: f32 scratch [T, H, nsplit, r + 2] when nsplit > 1; window > 0: only the keys pos - window < j <= pos count
void latent_attention(bool bf16, const void* q_lat, const void* q_rot, int64_t qr_st, int64_t qr_sh, const void* rows,
                      int bs, const int32_t* block_tables, int bt_width, const int32_t* seq_of, const int64_t* pos,
                      float scale, const void* gate, int64_t g_st, void* out, float* part, int nsplit, int T, int H,
                      int r, int dr, int window, hipStream_t st);

// causal softmax of f32 score rows [R, L] (row stride ld), row i -> position pos[i / H], column j -> key key0 + j,
// window > 0: only the keys pos - window < key <= pos count; bf16: weights leave as hi + lo bf16 pairs (same row
// stride), f32 (hi == null): in place
void causal_softmax(bool bf16, float* sc, int64_t ld, const int64_t* pos, int H, float scale, int64_t R, int L, void* hi,
                    void* lo, int64_t key0, int window, hipStream_t st);

// q, k [T, H, d], v [T, H, dv], gate pre-activations [T, H]: rows of *_ld elements
void mlstm_scan(bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld, const void* v, int64_t v_ld,
                const void* ipre, int64_t i_ld, const void* fpre, int64_t f_ld, const float* ib, const float* fb,
                float cap, float* S, float* n, float* m, const int32_t* cu, const int32_t* slots, const int64_t* pos,
                float* out, int B, int H, int d, int dv, hipStream_t st);
void head_rms_gate(bool bf16, const float* h, const void* norm_w, const void* gate, int64_t g_ld, void* out, int T,
                   int H, int dv, float eps, hipStream_t st);
void glu_gelu(bool bf16, const void* gu, void* out, int64_t T, int64_t I, hipStream_t st);
// act(gate) * up; act 0: tanh-GELU, 1: ReLU, 2: SiLU
void glu_act(bool bf16, const void* gu, void* out, int64_t T, int64_t I, int act, hipStream_t st);

}  // namespace sm
}  // namespace illm
