// torch.ops.ipex_llm_amd.sm_*: the sequence-mixing kernels of the hybrid
// decoders (csrc/hip/seqmix.hip).  Every entry checks on the host that the
// operand shapes, dtypes and strides are what its kernel and grid assume.
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include <algorithm>

#include "../hip/seqmix.h"

using at::Tensor;

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }

bool is_act(const Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
bool bf(const Tensor& t) { return t.scalar_type() == at::kBFloat16; }

void check_idx(const Tensor& t, at::ScalarType ty, int64_t n, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == ty && t.is_contiguous() && t.numel() >= n, what);
}

Tensor sm_embed_bigram(const Tensor& ids, const Tensor& prev, const Tensor& embed, const Tensor& bigram,
                       int64_t mul_prev, int64_t mul_cur) {
  c10::DeviceGuard g(embed.device());
  const int64_t T = ids.numel(), W = embed.size(1);
  check_idx(ids, at::kLong, T, "sm_embed_bigram: ids int64 on the GPU");
  check_idx(prev, at::kLong, T, "sm_embed_bigram: prev ids int64 [T]");
  TORCH_CHECK(embed.is_cuda() && embed.dim() == 2 && is_act(embed) && embed.is_contiguous() && bigram.dim() == 2 &&
                  bigram.scalar_type() == embed.scalar_type() && bigram.is_contiguous() && bigram.size(1) == W &&
                  bigram.size(0) >= 2 && bigram.is_cuda(),
              "sm_embed_bigram: embed [V, W] and bigram [buckets + 1, W] of one dtype (bf16 / f32)");
  Tensor out = at::empty({T, W}, embed.options().dtype(at::kFloat));
  illm::sm::embed_bigram(bf(embed), ids.data_ptr<int64_t>(), prev.data_ptr<int64_t>(), embed.data_ptr(),
                         bigram.data_ptr(), out.data_ptr<float>(), (int)T, (int)W, embed.size(0), bigram.size(0) - 1,
                         mul_prev, mul_cur, stream());
  return out;
}

Tensor sm_add_scaled_layer_norm(Tensor& x, const Tensor& y, const Tensor& w, double eps, double mult, bool act_f32) {
  c10::DeviceGuard g(x.device());
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.scalar_type() == at::kFloat && x.is_contiguous(),
              "sm_add_scaled_layer_norm: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(y.is_cuda() && is_act(y) && y.is_contiguous() && y.dim() == 2 && y.size(0) == T && y.size(1) == W,
              "sm_add_scaled_layer_norm: y [T, W] bf16 / f32");
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == y.scalar_type() && w.is_contiguous() && w.numel() == W,
              "sm_add_scaled_layer_norm: w [W] of y's dtype");
  TORCH_CHECK(act_f32 == (y.scalar_type() == at::kFloat), "sm_add_scaled_layer_norm: activation dtype mismatch");
  Tensor xa;
  if (!act_f32) xa = at::empty({T, W}, y.options());
  illm::sm::add_scaled_layer_norm(bf(y), x.data_ptr<float>(), y.data_ptr(), w.data_ptr(),
                                  act_f32 ? nullptr : xa.data_ptr(), (int)T, (int)W, (float)eps, (float)mult, stream());
  return act_f32 ? x : xa;
}

Tensor sm_layer_norm(const Tensor& x, const Tensor& w, double eps, bool act_f32) {
  c10::DeviceGuard g(x.device());
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.scalar_type() == at::kFloat && x.is_contiguous(),
              "sm_layer_norm: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(w.is_cuda() && is_act(w) && w.is_contiguous() && w.numel() == W &&
                  act_f32 == (w.scalar_type() == at::kFloat),
              "sm_layer_norm: w [W] in the activation dtype");
  Tensor out = at::empty({T, W}, w.options());
  illm::sm::layer_norm(bf(w), x.data_ptr<float>(), w.data_ptr(), out.data_ptr(), (int)T, (int)W, (float)eps, stream());
  return out;
}

void check_table(const Tensor& table, const char* who) {
  TORCH_CHECK(table.is_cuda() && table.scalar_type() == at::kFloat && table.is_contiguous() && table.dim() == 3 &&
                  table.size(2) == 2 && table.size(1) >= 1,
              who, ": rotary table f32 [max_pos, dims / 2, 2]");
}

void sm_rope_rows_(Tensor& q, int64_t offset, const Tensor& table, const Tensor& pos) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && is_act(q) && q.is_contiguous(), "sm_rope_rows_: q [T, H, D] contiguous");
  check_table(table, "sm_rope_rows_");
  const int64_t T = q.size(0), H = q.size(1), Dh = q.size(2), dims = 2 * table.size(1);
  TORCH_CHECK(offset >= 0 && offset + dims <= Dh, "sm_rope_rows_: rotated range outside the head");
  check_idx(pos, at::kLong, T, "sm_rope_rows_: pos int64 [T]");
  illm::sm::rope_rows(bf(q), q.data_ptr(), (int)T, (int)H, (int)Dh, (int)offset, table.data_ptr<float>(),
                      (int)table.size(0), (int)dims, pos.data_ptr<int64_t>(), stream());
}

void sm_latent_kv_store(const Tensor& dkv, const Tensor& norm_w, double eps, int64_t rank, const Tensor& table,
                        const Tensor& pos, const Tensor& slots, Tensor& rows) {
  c10::DeviceGuard g(dkv.device());
  TORCH_CHECK(dkv.is_cuda() && dkv.dim() == 2 && is_act(dkv) && dkv.stride(1) == 1, "sm_latent_kv_store: dkv [T, r + dr]");
  const int64_t T = dkv.size(0), D = dkv.size(1), dr = D - rank;
  check_table(table, "sm_latent_kv_store");
  const int64_t dims = 2 * table.size(1);
  TORCH_CHECK(rank > 0 && dr >= 0 && dims <= dr, "sm_latent_kv_store: rank / rotated sizes");
  TORCH_CHECK(rows.is_cuda() && rows.dim() == 3 && rows.scalar_type() == dkv.scalar_type() && rows.is_contiguous() &&
                  rows.size(2) == D,
              "sm_latent_kv_store: rows [blocks, bs, r + dr] of dkv's dtype");
  TORCH_CHECK(norm_w.is_cuda() && norm_w.scalar_type() == dkv.scalar_type() && norm_w.is_contiguous() &&
                  norm_w.numel() == rank,
              "sm_latent_kv_store: norm weight [rank]");
  check_idx(pos, at::kLong, T, "sm_latent_kv_store: pos int64 [T]");
  check_idx(slots, at::kLong, T, "sm_latent_kv_store: slots int64 [T]");
  illm::sm::latent_kv_store(bf(dkv), dkv.data_ptr(), dkv.stride(0), norm_w.data_ptr(), (float)eps, (int)rank, (int)dr,
                            table.data_ptr<float>(), (int)table.size(0), (int)dims, pos.data_ptr<int64_t>(),
                            slots.data_ptr<int64_t>(), rows.data_ptr(), rows.size(0) * rows.size(1), (int)T, stream());
}

// dynamic LDS the flash kernel would take for these sizes; -1: they do not fit (callers then take the
// library-product path, which has no size limits)
int64_t sm_latent_attention_fits(bool bf16, int64_t H, int64_t r, int64_t dr) {
  if (r < 1 || r > 512) return -1;
  int kt = 0, nw = 0, hb = 0;
  return illm::sm::latent_attention_plan(bf16, (int)H, (int)r, (int)dr, &kt, &nw, &hb);
}

Tensor sm_latent_attention(const Tensor& q_lat, const Tensor& q_rot, const Tensor& rows, const Tensor& block_tables,
                           const Tensor& seq_of, const Tensor& pos, double scale, const c10::optional<Tensor>& gate,
                           int64_t max_ctx, bool act_f32, int64_t window) {
  c10::DeviceGuard g(q_lat.device());
  TORCH_CHECK(q_lat.is_cuda() && q_lat.dim() == 3 && is_act(q_lat) && q_lat.is_contiguous(),
              "sm_latent_attention: q_lat [T, H, r] contiguous");
  TORCH_CHECK(window >= 0 && window < (int64_t)1 << 30, "sm_latent_attention: window >= 0");
  TORCH_CHECK(act_f32 == (q_lat.scalar_type() == at::kFloat), "sm_latent_attention: activation dtype mismatch");
  const int64_t T = q_lat.size(0), H = q_lat.size(1), r = q_lat.size(2);
  TORCH_CHECK(q_rot.is_cuda() && q_rot.dim() == 3 && q_rot.scalar_type() == q_lat.scalar_type() && q_rot.size(0) == T &&
                  q_rot.size(1) == H && (q_rot.size(2) == 0 || q_rot.stride(2) == 1),
              "sm_latent_attention: q_rot [T, H, dr] (unit inner stride)");
  const int64_t dr = q_rot.size(2);
  TORCH_CHECK(rows.is_cuda() && rows.dim() == 3 && rows.scalar_type() == q_lat.scalar_type() && rows.is_contiguous() &&
                  rows.size(2) == r + dr && rows.size(1) % 64 == 0,
              "sm_latent_attention: rows [blocks, bs (multiple of 64), r + dr] of q's dtype");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
                  block_tables.is_contiguous(),
              "sm_latent_attention: block tables int32 [B, W]");
  TORCH_CHECK(max_ctx >= 1 && max_ctx <= block_tables.size(1) * rows.size(1),
              "sm_latent_attention: block tables narrower than the longest context");
  check_idx(seq_of, at::kInt, T, "sm_latent_attention: seq_of int32 [T]");
  check_idx(pos, at::kLong, T, "sm_latent_attention: pos int64 [T]");
  TORCH_CHECK(r >= 1 && r <= 512, "sm_latent_attention: latent size must be 1..512");
  const void* gp = nullptr;
  int64_t gst = 0;
  if (gate.has_value() && gate->defined()) {
    TORCH_CHECK(gate->is_cuda() && gate->dim() == 2 && gate->size(0) == T && gate->size(1) == H &&
                    gate->scalar_type() == q_lat.scalar_type() && (H == 1 || gate->stride(1) == 1),
                "sm_latent_attention: gate [T, H] of q's dtype");
    gp = gate->data_ptr();
    gst = gate->stride(0);
  }
  int kt = 0, nw = 0, hb = 0;
  TORCH_CHECK(illm::sm::latent_attention_plan(bf(q_lat), (int)H, (int)r, (int)dr, &kt, &nw, &hb) > 0,
              "sm_latent_attention: a key tile of r + dr = ", r + dr, " does not fit in LDS");
  Tensor out = at::empty({T, H, r}, q_lat.options());
  if (T == 0) return out;
  // a window spans at most window keys plus the rest of its first tile
  const int64_t span = window > 0 ? std::min<int64_t>(max_ctx, window + 64) : max_ctx;
  const int nsplit = illm::sm::latent_attention_splits(bf(q_lat), (int)T, (int)H, (int)r, (int)dr, (int)span);
  Tensor part;
  if (nsplit > 1) part = at::empty({T, H, nsplit, r + 2}, q_lat.options().dtype(at::kFloat));
  illm::sm::latent_attention(bf(q_lat), q_lat.data_ptr(), q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1),
                             rows.data_ptr(), (int)rows.size(1), block_tables.data_ptr<int32_t>(),
                             (int)block_tables.size(1), seq_of.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), (float)scale,
                             gp, gst, out.data_ptr(), nsplit > 1 ? part.data_ptr<float>() : nullptr, nsplit, (int)T,
                             (int)H, (int)r, (int)dr, (int)window, stream());
  return out;
}

// scores f32 [R, L] (R = tokens x H rows) -> causal softmax weights; bf16 pair (hi, lo) or in place (f32)
std::tuple<Tensor, Tensor> sm_causal_softmax(Tensor& scores, const Tensor& pos, int64_t H, double scale, bool act_f32,
                                             int64_t key0, int64_t window) {
  c10::DeviceGuard g(scores.device());
  TORCH_CHECK(scores.is_cuda() && scores.dim() == 2 && scores.scalar_type() == at::kFloat && scores.is_contiguous(),
              "sm_causal_softmax: scores f32 [R, L] contiguous");
  const int64_t R = scores.size(0), L = scores.size(1);
  TORCH_CHECK(H >= 1 && R % H == 0, "sm_causal_softmax: rows must be tokens x heads");
  TORCH_CHECK(key0 >= 0 && window >= 0 && window < (int64_t)1 << 30, "sm_causal_softmax: key0 >= 0, window >= 0");
  check_idx(pos, at::kLong, R / H, "sm_causal_softmax: pos int64 [R / H]");
  Tensor hi, lo;
  if (!act_f32) {
    hi = at::empty({R, L}, scores.options().dtype(at::kBFloat16));
    lo = at::empty({R, L}, scores.options().dtype(at::kBFloat16));
  }
  illm::sm::causal_softmax(!act_f32, scores.data_ptr<float>(), L, pos.data_ptr<int64_t>(), (int)H, (float)scale, R, (int)L,
                           act_f32 ? nullptr : hi.data_ptr(), act_f32 ? nullptr : lo.data_ptr(), key0, (int)window,
                           stream());
  if (act_f32) return {scores, scores};
  return {hi, lo};
}

Tensor sm_mlstm_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& ipre, const Tensor& fpre,
                     const Tensor& ib, const Tensor& fb, double cap, Tensor& S, Tensor& n, Tensor& m, const Tensor& cu,
                     const Tensor& slots, const Tensor& pos, int64_t max_q) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && is_act(q) && q.stride(2) == 1 && q.stride(1) == q.size(2),
              "sm_mlstm_scan: q [T, H, d] (heads contiguous in a row)");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2), dv = v.size(2);
  auto same = [&](const Tensor& t) { return t.is_cuda() && t.scalar_type() == q.scalar_type(); };
  TORCH_CHECK(same(k) && k.sizes() == q.sizes() && k.stride(2) == 1 && k.stride(1) == d, "sm_mlstm_scan: k like q");
  TORCH_CHECK(same(v) && v.dim() == 3 && v.size(0) == T && v.size(1) == H && v.stride(2) == 1 && v.stride(1) == dv,
              "sm_mlstm_scan: v [T, H, dv]");
  TORCH_CHECK(same(ipre) && same(fpre) && ipre.dim() == 2 && fpre.dim() == 2 && ipre.size(0) == T && fpre.size(0) == T &&
                  ipre.size(1) == H && fpre.size(1) == H && (H == 1 || (ipre.stride(1) == 1 && fpre.stride(1) == 1)),
              "sm_mlstm_scan: gate pre-activations [T, H]");
  TORCH_CHECK(ib.is_cuda() && fb.is_cuda() && ib.scalar_type() == at::kFloat && fb.scalar_type() == at::kFloat &&
                  ib.is_contiguous() && fb.is_contiguous() && ib.numel() == H && fb.numel() == H,
              "sm_mlstm_scan: gate biases f32 [H]");
  const int64_t B = cu.numel() - 1;
  TORCH_CHECK(B >= 0 && cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous(), "sm_mlstm_scan: cu int32 [B + 1]");
  check_idx(slots, at::kInt, B, "sm_mlstm_scan: state slots int32 [B]");
  check_idx(pos, at::kLong, T, "sm_mlstm_scan: pos int64 [T]");
  TORCH_CHECK(S.is_cuda() && S.scalar_type() == at::kFloat && S.is_contiguous() && S.dim() == 4 && S.size(1) == H &&
                  S.size(2) == d && S.size(3) == dv && n.is_cuda() && n.scalar_type() == at::kFloat && n.is_contiguous() &&
                  n.dim() == 3 && n.size(0) == S.size(0) && n.size(1) == H && n.size(2) == d && m.is_cuda() &&
                  m.scalar_type() == at::kFloat && m.is_contiguous() && m.dim() == 2 && m.size(0) == S.size(0) &&
                  m.size(1) == H,
              "sm_mlstm_scan: state S [slots, H, d, dv], n [slots, H, d], m [slots, H] f32");
  TORCH_CHECK(d >= 1 && d <= 256, "sm_mlstm_scan: key size per head must be 1..256 (register-resident state rows)");
  TORCH_CHECK(max_q >= 0 && max_q <= T, "sm_mlstm_scan: max_q");
  Tensor out = at::empty({T, H, dv}, q.options().dtype(at::kFloat));
  if (T == 0 || B == 0) return out;
  illm::sm::mlstm_scan(bf(q), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                       ipre.data_ptr(), ipre.stride(0), fpre.data_ptr(), fpre.stride(0), ib.data_ptr<float>(),
                       fb.data_ptr<float>(), (float)cap, S.data_ptr<float>(), n.data_ptr<float>(), m.data_ptr<float>(),
                       cu.data_ptr<int32_t>(), slots.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), out.data_ptr<float>(),
                       (int)B, (int)H, (int)d, (int)dv, stream());
  return out;
}

Tensor sm_head_rms_gate(const Tensor& h, const Tensor& norm_w, const Tensor& gate, double eps, bool act_f32) {
  c10::DeviceGuard g(h.device());
  TORCH_CHECK(h.is_cuda() && h.dim() == 3 && h.scalar_type() == at::kFloat && h.is_contiguous(),
              "sm_head_rms_gate: h f32 [T, H, dv]");
  const int64_t T = h.size(0), H = h.size(1), dv = h.size(2);
  TORCH_CHECK(norm_w.is_cuda() && is_act(norm_w) && norm_w.is_contiguous() && norm_w.numel() == H * dv &&
                  act_f32 == (norm_w.scalar_type() == at::kFloat),
              "sm_head_rms_gate: norm weight [H * dv] in the activation dtype");
  TORCH_CHECK(gate.is_cuda() && gate.scalar_type() == norm_w.scalar_type() && gate.dim() == 2 && gate.size(0) == T &&
                  gate.size(1) == H * dv && gate.stride(1) == 1,
              "sm_head_rms_gate: gate [T, H * dv]");
  Tensor out = at::empty({T, H * dv}, norm_w.options());
  illm::sm::head_rms_gate(bf(norm_w), h.data_ptr<float>(), norm_w.data_ptr(), gate.data_ptr(), gate.stride(0),
                          out.data_ptr(), (int)T, (int)H, (int)dv, (float)eps, stream());
  return out;
}

Tensor sm_glu_gelu(const Tensor& gu) {
  c10::DeviceGuard g(gu.device());
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && is_act(gu) && gu.is_contiguous() && gu.size(1) % 2 == 0,
              "sm_glu_gelu: [T, 2 I] contiguous bf16 / f32");
  const int64_t T = gu.size(0), I = gu.size(1) / 2;
  Tensor out = at::empty({T, I}, gu.options());
  illm::sm::glu_gelu(bf(gu), gu.data_ptr(), out.data_ptr(), T, I, stream());
  return out;
}

Tensor sm_glu_act(const Tensor& gu, int64_t act) {
  c10::DeviceGuard g(gu.device());
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && is_act(gu) && gu.is_contiguous() && gu.size(1) % 2 == 0,
              "sm_glu_act: [T, 2 I] contiguous bf16 / f32");
  TORCH_CHECK(act >= 0 && act <= 2, "sm_glu_act: act 0 (tanh-GELU), 1 (ReLU) or 2 (SiLU)");
  const int64_t T = gu.size(0), I = gu.size(1) / 2;
  Tensor out = at::empty({T, I}, gu.options());
  illm::sm::glu_act(bf(gu), gu.data_ptr(), out.data_ptr(), T, I, (int)act, stream());
  return out;
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(ipex_llm_amd, m) {
  m.def("sm_embed_bigram(Tensor ids, Tensor prev, Tensor embed, Tensor bigram, int mul_prev, int mul_cur) -> Tensor");
  m.def("sm_add_scaled_layer_norm(Tensor(a!) x, Tensor y, Tensor w, float eps, float mult, bool act_f32) -> Tensor");
  m.def("sm_layer_norm(Tensor x, Tensor w, float eps, bool act_f32) -> Tensor");
  m.def("sm_rope_rows_(Tensor(a!) q, int offset, Tensor table, Tensor pos) -> ()");
  m.def("sm_latent_kv_store(Tensor dkv, Tensor norm_w, float eps, int rank, Tensor table, Tensor pos, Tensor slots, "
        "Tensor(a!) rows) -> ()");
  m.def("sm_latent_attention(Tensor q_lat, Tensor q_rot, Tensor rows, Tensor block_tables, Tensor seq_of, Tensor pos, "
        "float scale, Tensor? gate, int max_ctx, bool act_f32, int window=0) -> Tensor");
  m.def("sm_latent_attention_fits(bool bf16, int H, int r, int dr) -> int");
  m.def("sm_mlstm_scan(Tensor q, Tensor k, Tensor v, Tensor ipre, Tensor fpre, Tensor ib, Tensor fb, float cap, "
        "Tensor(a!) S, Tensor(b!) n, Tensor(c!) m, Tensor cu, Tensor slots, Tensor pos, int max_q) -> Tensor");
  m.def("sm_causal_softmax(Tensor(a!) scores, Tensor pos, int H, float scale, bool act_f32, int key0=0, int window=0) "
        "-> (Tensor, Tensor)");
  m.def("sm_head_rms_gate(Tensor h, Tensor norm_w, Tensor gate, float eps, bool act_f32) -> Tensor");
  m.def("sm_glu_gelu(Tensor gu) -> Tensor");
  m.def("sm_glu_act(Tensor gu, int act) -> Tensor");
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CompositeExplicitAutograd, m) {
  m.impl("sm_latent_attention_fits", &sm_latent_attention_fits);
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CUDA, m) {
  m.impl("sm_embed_bigram", &sm_embed_bigram);
  m.impl("sm_add_scaled_layer_norm", &sm_add_scaled_layer_norm);
  m.impl("sm_layer_norm", &sm_layer_norm);
  m.impl("sm_rope_rows_", &sm_rope_rows_);
  m.impl("sm_latent_kv_store", &sm_latent_kv_store);
  m.impl("sm_latent_attention", &sm_latent_attention);
  m.impl("sm_mlstm_scan", &sm_mlstm_scan);
  m.impl("sm_causal_softmax", &sm_causal_softmax);
  m.impl("sm_head_rms_gate", &sm_head_rms_gate);
  m.impl("sm_glu_gelu", &sm_glu_gelu);
  m.impl("sm_glu_act", &sm_glu_act);
}
