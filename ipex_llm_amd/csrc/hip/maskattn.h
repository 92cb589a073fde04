// Launchers of the masked grouped-query attention kernels (maskattn.hip):
// norm + rotary + cache append of a step's queries, keys and values, and
// attention over paged [keys | values] rows with a causal, sliding-window or
// chunked view of the past and an optional sink in the softmax.  ``bf16``
// selects the activation element type (bf16 when true, f32 when false);
// everything the kernels accumulate is f32 either way.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace illm {
namespace ma {

enum Mask { kCausal = 0, kWindow = 1, kChunk = 2 };
enum Layout { kPairs = 0, kHalf = 1 };     // rotary pairs (2 i, 2 i + 1) or (i, i + dims / 2)

// q [T, H, d] / k [T, G, d] / v [T, G, dv]: rows of q_ld / k_ld / v_ld elements (k, v, rows null: queries only);
// qn / kn: norm weights ([H d] / [G d] when whole, else [d]) or null; table f32 [max_pos, dims / 2, 2] or null;
// rows [num_rows, G d + G dv]; qo f32 [T, H, d].  in_bf16: the element type of q / k / v (f32 inputs beside bf16
// weights and rows are allowed: the result of a convolution), bf16: of the norm weights and the rows
void qkv_norm_rope_store(bool in_bf16, bool bf16, const void* q, int64_t q_ld, const void* k, int64_t k_ld,
                         const void* v, int64_t v_ld, const void* qn, const void* kn, bool whole, float eps,
                         const float* table, int max_pos, int dims, int layout, const int64_t* pos, const int64_t* slots,
                         void* rows, int64_t num_rows, float* qo, int T, int H, int G, int d, int dv, hipStream_t st);

// dynamic LDS of the attention launch (waves and heads per workgroup out); < 0: these sizes do not fit
int masked_attention_plan(bool bf16, int rep, int d, int dv, int* nw, int* hb);
// key splits (grid z) for T query tokens that see at most max_keys keys
int masked_attention_splits(bool bf16, int T, int H, int G, int d, int dv, int max_keys, bool cross);
// q f32 [T, H, d]; rows [., bs, G d + G dv]; sink f32 [H] or null; out [T, H dv];
// part: f32 scratch [T, H, nsplit, dv + 2] when nsplit > 1.  softcap > 0: scores capped by softcap tanh(s / softcap);
// keep > 0 (window): the keys before position ``keep`` stay visible; talk f32 [H, H] or null: the heads' weights
// mixed after the softmax -- part is then [T, H, G, nsplit, dv + 2] whatever nsplit is
void masked_attention(bool bf16, const float* q, const void* rows, int bs, const int32_t* block_tables, int bt_width,
                      const int32_t* seq_of, const int64_t* pos, float scale, int mask, int size, const float* sink,
                      void* out, float* part, int nsplit, int T, int H, int G, int d, int dv, float softcap, int keep,
                      const float* talk, hipStream_t st);

// rows [R, L] of raw scores of pieces of chunks: a piece is L keys from a chunk's first position on, its queries are
// its last Lq positions (Lq == L: a whole chunk).  Row i: head (i / (rep Lq)) % G * rep + i % rep, query
// (i / rep) % Lq, which sees keys 0 .. L - Lq + query.  Scaled, softmax with the head's sink; bf16: the f32 weights
// leave as bf16 pairs hi + lo in hl [R, 2 L] (a row's hi halves, then its lo halves); f32 (hl == null): in place
// (hl null with bf16: in place as well); softcap as above.  window > 0: the rows are a block of Lq queries of a sliding
// window instead (query i at position q0 + i): the first nkeep columns are kept first tokens, column nkeep + j is the
// key at position k0 + j, seen when not ahead of the query and closer than ``window`` (or before position ``keep``)
void chunk_softmax(bool bf16, float* sc, int64_t R, int Lq, int L, int G, int rep, float scale, const float* sink,
                   void* hl, float softcap, int window, int keep, int nkeep, int64_t q0, int64_t k0, hipStream_t st);

// w f32 [pieces, G, Lq, rep, L] normalised weights -> the heads' weights mixed by talk f32 [H, H] (H = G rep), same
// layout: bf16 pairs hi + lo in hl [R, 2 L], or f32 in out32 [R, L]
void talk_mix(bool bf16, const float* w, const float* talk, int64_t pieces, int Lq, int L, int G, int rep, void* hl,
              float* out32, hipStream_t st);

// o[t, c] *= sigmoid(g[t, c]); g rows of g_ld elements
void sigmoid_gate(bool bf16, void* o, const void* g, int64_t g_ld, int64_t T, int C, hipStream_t st);

}  // namespace ma
}  // namespace illm
