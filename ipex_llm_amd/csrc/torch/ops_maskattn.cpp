// torch.ops.ipex_llm_amd.ma_*: masked grouped-query attention
// (csrc/hip/maskattn.hip).  Every entry checks on the host that the operand
// shapes, dtypes and strides are what its kernel and grid assume.
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include <algorithm>
#include <tuple>

#include "../hip/maskattn.h"

using at::Tensor;

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }
bool is_act(const Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
bool bf(const Tensor& t) { return t.scalar_type() == at::kBFloat16; }
bool has(const c10::optional<Tensor>& t) { return t.has_value() && t->defined(); }

void check_idx(const Tensor& t, at::ScalarType ty, int64_t n, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == ty && t.is_contiguous() && t.numel() >= n, what);
}
// [T, heads, n] view of a projection's rows: heads contiguous inside a row
bool head_rows(const Tensor& t, at::ScalarType ty) {
  return t.is_cuda() && t.dim() == 3 && t.scalar_type() == ty && t.stride(2) == 1 && t.stride(1) == t.size(2) &&
         t.stride(0) >= t.size(1) * t.size(2);
}

Tensor ma_qkv_norm_rope_store(const Tensor& q, const c10::optional<Tensor>& k, const c10::optional<Tensor>& v,
                              const c10::optional<Tensor>& qn, const c10::optional<Tensor>& kn, bool whole, double eps,
                              const c10::optional<Tensor>& table, int64_t layout, const Tensor& pos, const Tensor& slots,
                              const c10::optional<Tensor>& rows) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(is_act(q) && head_rows(q, q.scalar_type()), "ma_qkv_norm_rope_store: q [T, H, d] (heads contiguous in a row)");
  const auto in_ty = q.scalar_type();
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  const bool store = has(k);
  TORCH_CHECK(store == has(v) && store == has(rows), "ma_qkv_norm_rope_store: k, v and rows come together");
  // q / k / v may be f32 beside 16-bit rows and norm weights (the result of a convolution in front)
  const auto ty = store ? rows->scalar_type() : (has(qn) ? qn->scalar_type() : in_ty);
  TORCH_CHECK(ty == in_ty || in_ty == at::kFloat, "ma_qkv_norm_rope_store: q / k / v of the rows' dtype, or f32");
  int64_t G = 0, dv = 0, num_rows = 0;
  if (store) {
    TORCH_CHECK(head_rows(*k, in_ty) && k->size(0) == T && k->size(2) == d, "ma_qkv_norm_rope_store: k [T, G, d] like q");
    TORCH_CHECK(head_rows(*v, in_ty) && v->size(0) == T && v->size(1) == k->size(1), "ma_qkv_norm_rope_store: v [T, G, dv]");
    G = k->size(1);
    dv = v->size(2);
    TORCH_CHECK(rows->is_cuda() && rows->scalar_type() == ty && rows->is_contiguous() && rows->dim() == 3 &&
                    rows->size(2) == G * (d + dv),
                "ma_qkv_norm_rope_store: rows [blocks, bs, G d + G dv] of q's dtype");
    num_rows = rows->size(0) * rows->size(1);
  }
  auto norm_ok = [&](const c10::optional<Tensor>& w, int64_t heads) {
    return !has(w) || (w->is_cuda() && w->scalar_type() == ty && w->is_contiguous() && w->numel() == (whole ? heads * d : d));
  };
  TORCH_CHECK(norm_ok(qn, H) && (!store || norm_ok(kn, G)),
              "ma_qkv_norm_rope_store: norm weights [heads d] (whole) or [d] of q's dtype");
  int64_t dims = 0, max_pos = 0;
  if (has(table)) {
    TORCH_CHECK(table->is_cuda() && table->scalar_type() == at::kFloat && table->is_contiguous() && table->dim() == 3 &&
                    table->size(2) == 2 && 2 * table->size(1) <= d,
                "ma_qkv_norm_rope_store: table f32 [max_pos, dims / 2, 2], dims <= d");
    dims = 2 * table->size(1);
    max_pos = table->size(0);
  }
  TORCH_CHECK(layout == 0 || layout == 1, "ma_qkv_norm_rope_store: layout 0 (pairs) or 1 (half)");
  TORCH_CHECK(H + G <= 8192, "ma_qkv_norm_rope_store: too many heads");
  check_idx(pos, at::kLong, T, "ma_qkv_norm_rope_store: pos int64 [T]");
  check_idx(slots, at::kLong, T, "ma_qkv_norm_rope_store: slots int64 [T]");
  Tensor qo = at::empty({T, H, d}, q.options().dtype(at::kFloat));
  illm::ma::qkv_norm_rope_store(bf(q), ty == at::kBFloat16, q.data_ptr(), q.stride(0), store ? k->data_ptr() : nullptr,
                                store ? k->stride(0) : 0, store ? v->data_ptr() : nullptr, store ? v->stride(0) : 0,
                                has(qn) ? qn->data_ptr() : nullptr, store && has(kn) ? kn->data_ptr() : nullptr, whole,
                                (float)eps, has(table) ? table->data_ptr<float>() : nullptr, (int)max_pos, (int)dims,
                                (int)layout, pos.data_ptr<int64_t>(), slots.data_ptr<int64_t>(),
                                store ? rows->data_ptr() : nullptr, num_rows, qo.data_ptr<float>(), (int)T, (int)H, (int)G,
                                (int)d, (int)dv, stream());
  return qo;
}

Tensor ma_masked_attention(const Tensor& q, const Tensor& rows, int64_t G, int64_t dv, const Tensor& block_tables,
                           const Tensor& seq_of, const Tensor& pos, double scale, int64_t mask, int64_t size,
                           const c10::optional<Tensor>& sink, int64_t max_ctx, bool act_f32, double softcap,
                           int64_t keep_first, const c10::optional<Tensor>& talk) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.scalar_type() == at::kFloat && q.is_contiguous(),
              "ma_masked_attention: q f32 [T, H, d] contiguous");
  TORCH_CHECK(softcap >= 0 && keep_first >= 0 && keep_first < (int64_t)1 << 30 && (keep_first == 0 || mask == 1),
              "ma_masked_attention: softcap >= 0; keep_first >= 0 and only with a window");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  TORCH_CHECK(G >= 1 && H % G == 0 && dv >= 1, "ma_masked_attention: heads must be a multiple of key heads");
  const auto at_ = act_f32 ? at::kFloat : at::kBFloat16;
  TORCH_CHECK(rows.is_cuda() && rows.dim() == 3 && rows.scalar_type() == at_ && rows.is_contiguous() &&
                  rows.size(2) == G * (d + dv) && rows.size(1) % 64 == 0,
              "ma_masked_attention: rows [blocks, bs (multiple of 64), G d + G dv] in the activation dtype");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
                  block_tables.is_contiguous(),
              "ma_masked_attention: block tables int32 [B, W]");
  TORCH_CHECK(max_ctx >= 1 && max_ctx <= block_tables.size(1) * rows.size(1),
              "ma_masked_attention: block tables narrower than the longest context");
  TORCH_CHECK(mask >= 0 && mask <= 2 && (mask == 0 || (size >= 1 && size < (int64_t)1 << 30)),
              "ma_masked_attention: mask 0 (causal), 1 (window) or 2 (chunk) with a size of at least 1");
  check_idx(seq_of, at::kInt, T, "ma_masked_attention: seq_of int32 [T]");
  check_idx(pos, at::kLong, T, "ma_masked_attention: pos int64 [T]");
  const float* sk = nullptr;
  if (has(sink)) {
    TORCH_CHECK(sink->is_cuda() && sink->scalar_type() == at::kFloat && sink->is_contiguous() && sink->numel() == H,
                "ma_masked_attention: sink f32 [H]");
    sk = sink->data_ptr<float>();
  }
  const float* tk = nullptr;
  if (has(talk)) {
    TORCH_CHECK(talk->is_cuda() && talk->scalar_type() == at::kFloat && talk->is_contiguous() && talk->numel() == H * H,
                "ma_masked_attention: talk f32 [H, H]");
    tk = talk->data_ptr<float>();
  }
  int nw = 0, hb = 0;
  TORCH_CHECK(illm::ma::masked_attention_plan(!act_f32, (int)(H / G), (int)d, (int)dv, &nw, &hb) > 0,
              "ma_masked_attention: a key tile of d + dv = ", d + dv, " does not fit in LDS");
  TORCH_CHECK(G * ((H / G + hb - 1) / hb) * (tk ? G : 1) <= 65535, "ma_masked_attention: too many heads for one launch");
  Tensor out = at::empty({T, H * dv}, q.options().dtype(at_));
  if (T == 0) return out;
  const int64_t span = mask == 0 ? max_ctx : std::min<int64_t>(max_ctx, size + keep_first + 16);
  const int nsplit =
      illm::ma::masked_attention_splits(!act_f32, (int)T, (int)H, (int)G, (int)d, (int)dv, (int)span, tk != nullptr);
  Tensor part;
  if (tk) part = at::empty({T, H, G, nsplit, dv + 2}, q.options());
  else if (nsplit > 1) part = at::empty({T, H, nsplit, dv + 2}, q.options());
  illm::ma::masked_attention(!act_f32, q.data_ptr<float>(), rows.data_ptr(), (int)rows.size(1),
                             block_tables.data_ptr<int32_t>(), (int)block_tables.size(1), seq_of.data_ptr<int32_t>(),
                             pos.data_ptr<int64_t>(), (float)scale, (int)mask, (int)size, sk, out.data_ptr(),
                             part.defined() ? part.data_ptr<float>() : nullptr, nsplit, (int)T, (int)H, (int)G, (int)d,
                             (int)dv, (float)softcap, (int)keep_first, tk, stream());
  return out;
}

int64_t ma_masked_attention_fits(bool bf16, int64_t rep, int64_t d, int64_t dv) {
  int nw = 0, hb = 0;
  return illm::ma::masked_attention_plan(bf16, (int)rep, (int)d, (int)dv, &nw, &hb);
}

// scores f32 [R, L] of whole chunks -> softmax weights with the sink: bf16 [R, 2 L] (hi halves | lo halves), or in
// place (f32)
Tensor ma_chunk_softmax(Tensor& scores, int64_t Lq, int64_t G, int64_t rep, double scale,
                        const c10::optional<Tensor>& sink, bool act_f32, double softcap, bool in_place, int64_t window,
                        int64_t keep, int64_t nkeep, int64_t q0, int64_t k0) {
  c10::DeviceGuard g(scores.device());
  TORCH_CHECK(scores.is_cuda() && scores.dim() == 2 && scores.scalar_type() == at::kFloat && scores.is_contiguous(),
              "ma_chunk_softmax: scores f32 [R, L] contiguous");
  const int64_t R = scores.size(0), L = scores.size(1);
  TORCH_CHECK(G >= 1 && rep >= 1 && Lq >= 1 && (window > 0 || Lq <= L) && R % (G * rep * Lq) == 0,
              "ma_chunk_softmax: rows must be pieces x key heads x Lq x rep, Lq <= L");
  TORCH_CHECK(window >= 0 && window < (int64_t)1 << 30 && keep >= 0 && keep < (int64_t)1 << 30 && nkeep >= 0 &&
                  nkeep <= L && q0 >= 0 && k0 >= 0 && k0 <= q0 && (window == 0 || nkeep + (q0 - k0) + Lq <= L),
              "ma_chunk_softmax: a window's block holds its kept columns and every key from k0 to its last query");
  const float* sk = nullptr;
  if (has(sink)) {
    TORCH_CHECK(sink->is_cuda() && sink->scalar_type() == at::kFloat && sink->is_contiguous() && sink->numel() == G * rep,
                "ma_chunk_softmax: sink f32 [H]");
    sk = sink->data_ptr<float>();
  }
  Tensor hl;
  const bool pairs = !act_f32 && !in_place;
  if (pairs) hl = at::empty({R, 2 * L}, scores.options().dtype(at::kBFloat16));
  illm::ma::chunk_softmax(!act_f32, scores.data_ptr<float>(), R, (int)Lq, (int)L, (int)G, (int)rep, (float)scale, sk,
                          pairs ? hl.data_ptr() : nullptr, (float)softcap, (int)window, (int)keep, (int)nkeep, q0, k0,
                          stream());
  return pairs ? hl : scores;
}

// normalised weights f32 [R, L] (R = pieces x G x Lq x rep) -> the heads' weights mixed by talk [H, H]: bf16 pairs
// [R, 2 L] or f32 [R, L]
Tensor ma_talk_mix(const Tensor& w, const Tensor& talk, int64_t Lq, int64_t G, int64_t rep, bool act_f32) {
  c10::DeviceGuard g(w.device());
  TORCH_CHECK(w.is_cuda() && w.dim() == 2 && w.scalar_type() == at::kFloat && w.is_contiguous(),
              "ma_talk_mix: weights f32 [R, L] contiguous");
  const int64_t R = w.size(0), L = w.size(1), H = G * rep;
  TORCH_CHECK(G >= 1 && rep >= 1 && Lq >= 1 && R % (H * Lq) == 0, "ma_talk_mix: rows must be pieces x key heads x Lq x rep");
  TORCH_CHECK(talk.is_cuda() && talk.scalar_type() == at::kFloat && talk.is_contiguous() && talk.numel() == H * H &&
                  H * 64 * 4 <= 64 * 1024,
              "ma_talk_mix: talk f32 [H, H], H <= 256");
  TORCH_CHECK((L + 63) / 64 <= 65535, "ma_talk_mix: too many keys for one launch");
  Tensor out = act_f32 ? at::empty({R, L}, w.options()) : at::empty({R, 2 * L}, w.options().dtype(at::kBFloat16));
  illm::ma::talk_mix(!act_f32, w.data_ptr<float>(), talk.data_ptr<float>(), R / (H * Lq), (int)Lq, (int)L, (int)G,
                     (int)rep, act_f32 ? nullptr : out.data_ptr(), act_f32 ? out.data_ptr<float>() : nullptr, stream());
  return out;
}

Tensor ma_sigmoid_gate(Tensor& o, const Tensor& gate) {
  c10::DeviceGuard g(o.device());
  TORCH_CHECK(o.is_cuda() && o.dim() == 2 && is_act(o) && o.is_contiguous(), "ma_sigmoid_gate: o [T, C] contiguous");
  const int64_t T = o.size(0), C = o.size(1);
  TORCH_CHECK(gate.is_cuda() && gate.dim() == 2 && gate.scalar_type() == o.scalar_type() && gate.size(0) == T &&
                  gate.size(1) == C && (C == 1 || gate.stride(1) == 1),
              "ma_sigmoid_gate: gate [T, C] of o's dtype (unit inner stride)");
  illm::ma::sigmoid_gate(bf(o), o.data_ptr(), gate.data_ptr(), gate.stride(0), T, (int)C, stream());
  return o;
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(ipex_llm_amd, m) {
  m.def("ma_qkv_norm_rope_store(Tensor q, Tensor? k, Tensor? v, Tensor? qn, Tensor? kn, bool whole, float eps, "
        "Tensor? table, int layout, Tensor pos, Tensor slots, Tensor(a!)? rows) -> Tensor");
  m.def("ma_masked_attention(Tensor q, Tensor rows, int G, int dv, Tensor block_tables, Tensor seq_of, Tensor pos, "
        "float scale, int mask, int size, Tensor? sink, int max_ctx, bool act_f32, float softcap, int keep_first, "
        "Tensor? talk) -> Tensor");
  m.def("ma_masked_attention_fits(bool bf16, int rep, int d, int dv) -> int");
  m.def("ma_chunk_softmax(Tensor(a!) scores, int Lq, int G, int rep, float scale, Tensor? sink, bool act_f32, "
        "float softcap, bool in_place, int window, int keep, int nkeep, int q0, int k0) -> Tensor");
  m.def("ma_talk_mix(Tensor w, Tensor talk, int Lq, int G, int rep, bool act_f32) -> Tensor");
  m.def("ma_sigmoid_gate(Tensor(a!) o, Tensor gate) -> Tensor(a!)");
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CompositeExplicitAutograd, m) {
  m.impl("ma_masked_attention_fits", &ma_masked_attention_fits);
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CUDA, m) {
  m.impl("ma_qkv_norm_rope_store", &ma_qkv_norm_rope_store);
  m.impl("ma_masked_attention", &ma_masked_attention);
  m.impl("ma_chunk_softmax", &ma_chunk_softmax);
  m.impl("ma_talk_mix", &ma_talk_mix);
  m.impl("ma_sigmoid_gate", &ma_sigmoid_gate);
}
