// torch.ops.ipex_llm_amd.bm_*: the kernels of the parallel-residual hybrid
// blocks (csrc/hip/blockmix_*.hip).  Every entry checks on the host that the
// operand shapes, dtypes and strides are what its kernel and grid assume.
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include <tuple>

#include "../hip/blockmix.h"

using at::Tensor;

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }

bool is_act(const Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
bool bf(const Tensor& t) { return t.scalar_type() == at::kBFloat16; }
at::ScalarType act_type(bool act_f32) { return act_f32 ? at::kFloat : at::kBFloat16; }

void check_idx(const Tensor& t, at::ScalarType ty, int64_t n, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == ty && t.is_contiguous() && t.numel() >= n, what);
}
void check_f32_rows(const Tensor& x, const char* what) {
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.scalar_type() == at::kFloat && x.is_contiguous(), what);
}
const float* opt_scale(const c10::optional<Tensor>& s, int64_t W, const char* what) {
  if (!s.has_value() || !s->defined()) return nullptr;
  TORCH_CHECK(s->is_cuda() && s->scalar_type() == at::kFloat && s->is_contiguous() && s->numel() == W, what);
  return s->data_ptr<float>();
}

std::tuple<Tensor, Tensor> bm_rms_norm_rows(const Tensor& x, const Tensor& w, double eps, bool act_f32) {
  c10::DeviceGuard g(x.device());
  check_f32_rows(x, "bm_rms_norm_rows: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(w.is_cuda() && w.is_contiguous() && (w.numel() == 1 || w.numel() == W) &&
                  w.scalar_type() == act_type(act_f32),
              "bm_rms_norm_rows: w [1] or [W] in the activation dtype");
  Tensor h = at::empty({T, W}, x.options());
  Tensor ha = act_f32 ? h : at::empty({T, W}, x.options().dtype(at::kBFloat16));
  illm::bm::rms_norm_rows(!act_f32, x.data_ptr<float>(), w.data_ptr(), (int)w.numel(), h.data_ptr<float>(),
                          act_f32 ? nullptr : ha.data_ptr(), (int)T, (int)W, (float)eps, stream());
  return {h, ha};
}

Tensor bm_add_rms_norm(Tensor& x, const Tensor& y, const Tensor& w, double eps, bool act_f32) {
  c10::DeviceGuard g(x.device());
  check_f32_rows(x, "bm_add_rms_norm: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(y.is_cuda() && y.scalar_type() == act_type(act_f32) && y.is_contiguous() && y.dim() == 2 &&
                  y.size(0) == T && y.size(1) == W,
              "bm_add_rms_norm: y [T, W] in the activation dtype");
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == y.scalar_type() && w.is_contiguous() && w.numel() == W,
              "bm_add_rms_norm: w [W] of y's dtype");
  Tensor xa;
  if (!act_f32) xa = at::empty({T, W}, y.options());
  illm::bm::add_rms_norm(!act_f32, x.data_ptr<float>(), y.data_ptr(), w.data_ptr(), act_f32 ? nullptr : xa.data_ptr(),
                         (int)T, (int)W, (float)eps, stream());
  return act_f32 ? x : xa;
}

Tensor bm_add_rms_norm_rows(Tensor& x, const c10::optional<Tensor>& y, const Tensor& w, double eps, bool act_f32) {
  c10::DeviceGuard g(x.device());
  check_f32_rows(x, "bm_add_rms_norm_rows: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  const void* yp = nullptr;
  if (y.has_value() && y->defined()) {
    TORCH_CHECK(y->is_cuda() && y->scalar_type() == act_type(act_f32) && y->is_contiguous() && y->dim() == 2 &&
                    y->size(0) == T && y->size(1) == W,
                "bm_add_rms_norm_rows: y [T, W] in the activation dtype");
    yp = y->data_ptr();
  }
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == act_type(act_f32) && w.is_contiguous() && w.numel() == W,
              "bm_add_rms_norm_rows: w [W] in the activation dtype");
  Tensor out = at::empty({T, W}, x.options().dtype(act_type(act_f32)));
  illm::bm::add_rms_norm_rows(!act_f32, x.data_ptr<float>(), yp, w.data_ptr(), out.data_ptr(), (int)T, (int)W,
                              (float)eps, stream());
  return out;
}

Tensor bm_residual_add_scaled(Tensor& x, const Tensor& y1, const c10::optional<Tensor>& s1,
                              const c10::optional<Tensor>& y2, const c10::optional<Tensor>& y3,
                              const c10::optional<Tensor>& s2, bool act_f32) {
  c10::DeviceGuard g(x.device());
  check_f32_rows(x, "bm_residual_add_scaled: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  const auto at_ = act_type(act_f32);
  auto same = [&](const Tensor& y) {
    return y.is_cuda() && y.is_contiguous() && y.dim() == 2 && y.size(0) == T && y.size(1) == W;
  };
  TORCH_CHECK(same(y1) && y1.scalar_type() == at_, "bm_residual_add_scaled: y1 [T, W] in the activation dtype");
  const void *p2 = nullptr, *p3 = nullptr;
  bool y2_f32 = true;
  if (y2.has_value() && y2->defined()) {
    TORCH_CHECK(same(*y2) && (y2->scalar_type() == at_ || y2->scalar_type() == at::kFloat),
                "bm_residual_add_scaled: y2 [T, W] f32 or the activation dtype");
    p2 = y2->data_ptr();
    y2_f32 = y2->scalar_type() == at::kFloat;
  }
  if (y3.has_value() && y3->defined()) {
    TORCH_CHECK(same(*y3) && y3->scalar_type() == at_, "bm_residual_add_scaled: y3 [T, W] in the activation dtype");
    p3 = y3->data_ptr();
  }
  Tensor xa;
  if (!act_f32) xa = at::empty({T, W}, y1.options());
  illm::bm::residual_add_scaled(!act_f32, x.data_ptr<float>(), y1.data_ptr(),
                                opt_scale(s1, W, "bm_residual_add_scaled: s1 f32 [W]"), p2, y2_f32, p3,
                                opt_scale(s2, W, "bm_residual_add_scaled: s2 f32 [W]"),
                                act_f32 ? nullptr : xa.data_ptr(), T, (int)W, stream());
  return act_f32 ? x : xa;
}

Tensor bm_canon_conv(const Tensor& h, const Tensor& w, Tensor& state, const Tensor& cu, const Tensor& seq_of,
                     const Tensor& slots, const Tensor& pos, bool act_f32) {
  c10::DeviceGuard g(h.device());
  check_f32_rows(h, "bm_canon_conv: h f32 [T, W]");
  const int64_t T = h.size(0), W = h.size(1);
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == at::kFloat && w.is_contiguous() && w.dim() == 2 && w.size(0) == W &&
                  w.size(1) >= 2 && w.size(1) <= 16,
              "bm_canon_conv: w f32 [W, taps], 2 <= taps <= 16");
  const int64_t taps = w.size(1);
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 3 &&
                  state.size(1) == taps - 1 && state.size(2) == W,
              "bm_canon_conv: state f32 [slots, taps - 1, W]");
  TORCH_CHECK(cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous() && cu.numel() >= 2,
              "bm_canon_conv: cu int32 [B + 1]");
  const int64_t B = cu.numel() - 1;
  check_idx(seq_of, at::kInt, T, "bm_canon_conv: seq_of int32 [T]");
  check_idx(slots, at::kInt, B, "bm_canon_conv: state slots int32 [B]");
  check_idx(pos, at::kLong, T, "bm_canon_conv: pos int64 [T]");
  Tensor out = at::empty({T, W}, h.options().dtype(act_type(act_f32)));
  illm::bm::canon_conv(!act_f32, h.data_ptr<float>(), w.data_ptr<float>(), (int)taps, state.data_ptr<float>(),
                       cu.data_ptr<int32_t>(), seq_of.data_ptr<int32_t>(), slots.data_ptr<int32_t>(),
                       pos.data_ptr<int64_t>(), out.data_ptr(), (int)T, (int)B, (int)W, stream());
  return out;
}

std::tuple<Tensor, Tensor, Tensor> bm_norm_canon(const Tensor& x, const Tensor& g, double eps, const Tensor& w,
                                                 Tensor& state, const Tensor& cu, const Tensor& seq_of,
                                                 const Tensor& slots, const Tensor& pos, bool single, bool act_f32) {
  c10::DeviceGuard gd(x.device());
  check_f32_rows(x, "bm_norm_canon: x f32 [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  TORCH_CHECK(g.is_cuda() && g.is_contiguous() && (g.numel() == 1 || g.numel() == W) &&
                  g.scalar_type() == act_type(act_f32),
              "bm_norm_canon: norm weight [1] or [W] in the activation dtype");
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == at::kFloat && w.is_contiguous() && w.dim() == 2 && w.size(0) == W &&
                  w.size(1) >= 2 && w.size(1) <= 16,
              "bm_norm_canon: w f32 [W, taps], 2 <= taps <= 16");
  const int64_t taps = w.size(1);
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 3 &&
                  state.size(1) == taps - 1 && state.size(2) == W,
              "bm_norm_canon: state f32 [slots, taps - 1, W]");
  TORCH_CHECK(cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous() && cu.numel() >= 2,
              "bm_norm_canon: cu int32 [B + 1]");
  const int64_t B = cu.numel() - 1;
  TORCH_CHECK(!single || B == T, "bm_norm_canon: single needs one token per sequence");
  check_idx(seq_of, at::kInt, T, "bm_norm_canon: seq_of int32 [T]");
  check_idx(slots, at::kInt, B, "bm_norm_canon: state slots int32 [B]");
  check_idx(pos, at::kLong, T, "bm_norm_canon: pos int64 [T]");
  Tensor h = at::empty({T, W}, x.options());
  Tensor ha = act_f32 ? h : at::empty({T, W}, x.options().dtype(at::kBFloat16));
  Tensor out = at::empty({T, W}, x.options().dtype(act_type(act_f32)));
  illm::bm::norm_canon(!act_f32, x.data_ptr<float>(), g.data_ptr(), (int)g.numel(), (float)eps, w.data_ptr<float>(),
                       (int)taps, state.data_ptr<float>(), cu.data_ptr<int32_t>(), seq_of.data_ptr<int32_t>(),
                       slots.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), h.data_ptr<float>(),
                       act_f32 ? nullptr : ha.data_ptr(), out.data_ptr(), (int)T, (int)B, (int)W, single, stream());
  return {h, ha, out};
}

Tensor bm_relu_sq(const Tensor& y) {
  c10::DeviceGuard g(y.device());
  TORCH_CHECK(y.is_cuda() && is_act(y) && y.is_contiguous(), "bm_relu_sq: contiguous bf16 / f32");
  Tensor out = at::empty_like(y);
  illm::bm::relu_sq(bf(y), y.data_ptr(), out.data_ptr(), y.numel(), stream());
  return out;
}

Tensor bm_glu_clamp(const Tensor& gu, double limit, double alpha) {
  c10::DeviceGuard g(gu.device());
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && is_act(gu) && gu.is_contiguous() && gu.size(1) % 2 == 0,
              "bm_glu_clamp: [T, 2 I] contiguous bf16 / f32");
  const int64_t T = gu.size(0), I = gu.size(1) / 2;
  Tensor out = at::empty({T, I}, gu.options());
  illm::bm::glu_clamp(bf(gu), gu.data_ptr(), out.data_ptr(), T, I, (float)limit, (float)alpha, stream());
  return out;
}

Tensor bm_side_gate(const Tensor& z, const Tensor& table, const Tensor& ids, int64_t offset) {
  c10::DeviceGuard g(z.device());
  TORCH_CHECK(z.is_cuda() && z.dim() == 2 && is_act(z) && z.is_contiguous(), "bm_side_gate: z [T, n] contiguous");
  const int64_t T = z.size(0), n = z.size(1);
  TORCH_CHECK(table.is_cuda() && table.dim() == 2 && table.scalar_type() == z.scalar_type() && table.is_contiguous() &&
                  offset >= 0 && offset + n <= table.size(1),
              "bm_side_gate: table [V, >= offset + n] of z's dtype");
  check_idx(ids, at::kLong, T, "bm_side_gate: ids int64 [T]");
  Tensor out = at::empty_like(z);
  illm::bm::side_gate(bf(z), z.data_ptr(), table.data_ptr(), table.size(1), table.size(0), ids.data_ptr<int64_t>(),
                      (int)offset, out.data_ptr(), (int)T, (int)n, stream());
  return out;
}

Tensor bm_qk_norm_rope_store(const Tensor& q, const Tensor& k, const c10::optional<Tensor>& qn,
                             const c10::optional<Tensor>& kn, double eps, const Tensor& table, const Tensor& pos,
                             const Tensor& slots, Tensor& rows) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && is_act(q) && q.stride(2) == 1 && q.stride(1) == q.size(2),
              "bm_qk_norm_rope_store: q [T, H, d] with dense heads");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  TORCH_CHECK(k.is_cuda() && k.dim() == 3 && k.scalar_type() == q.scalar_type() && k.size(0) == T && k.size(2) == d &&
                  k.stride(2) == 1 && k.stride(1) == d,
              "bm_qk_norm_rope_store: k [T, G, d] of q's dtype with dense heads");
  const int64_t G = k.size(1);
  TORCH_CHECK(table.is_cuda() && table.scalar_type() == at::kFloat && table.is_contiguous() && table.dim() == 3 &&
                  table.size(2) == 2 && table.size(1) >= 1 && 2 * table.size(1) <= d,
              "bm_qk_norm_rope_store: rotary table f32 [max_pos, dims / 2, 2], dims <= d");
  TORCH_CHECK(rows.is_cuda() && rows.dim() == 3 && rows.scalar_type() == q.scalar_type() && rows.is_contiguous() &&
                  rows.size(2) == 2 * G * d,
              "bm_qk_norm_rope_store: rows [blocks, bs, 2 G d] of q's dtype");
  auto normw = [&](const c10::optional<Tensor>& n) -> const void* {
    if (!n.has_value() || !n->defined()) return nullptr;
    TORCH_CHECK(n->is_cuda() && n->scalar_type() == q.scalar_type() && n->is_contiguous() && n->numel() == d,
                "bm_qk_norm_rope_store: norm weight [d] of q's dtype");
    return n->data_ptr();
  };
  check_idx(pos, at::kLong, T, "bm_qk_norm_rope_store: pos int64 [T]");
  check_idx(slots, at::kLong, T, "bm_qk_norm_rope_store: slots int64 [T]");
  TORCH_CHECK(d <= 4096, "bm_qk_norm_rope_store: head size");
  Tensor qo = at::empty({T, H, d}, q.options().dtype(at::kFloat));
  illm::bm::qk_norm_rope_store(bf(q), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), normw(qn), normw(kn),
                               (float)eps, table.data_ptr<float>(), (int)table.size(0), (int)(2 * table.size(1)),
                               pos.data_ptr<int64_t>(), slots.data_ptr<int64_t>(), rows.data_ptr(),
                               rows.size(0) * rows.size(1), qo.data_ptr<float>(), (int)T, (int)H, (int)G, (int)d,
                               stream());
  return qo;
}

int64_t bm_talk_attention_fits(bool bf16, int64_t H, int64_t G, int64_t d) {
  int kt = 0;
  return illm::bm::talk_attention_plan(bf16, (int)H, (int)G, (int)d, &kt);
}

const float* talk_ptr(const c10::optional<Tensor>& talk, int64_t H, const char* what) {
  if (!talk.has_value() || !talk->defined()) return nullptr;
  TORCH_CHECK(talk->is_cuda() && talk->scalar_type() == at::kFloat && talk->is_contiguous() && talk->dim() == 2 &&
                  talk->size(0) == H && talk->size(1) == H,
              what);
  return talk->data_ptr<float>();
}

Tensor bm_talk_attention(const Tensor& q, const Tensor& rows, const Tensor& block_tables, const Tensor& seq_of,
                         const Tensor& pos, double scale, const c10::optional<Tensor>& talk,
                         const c10::optional<Tensor>& gate, int64_t G, int64_t max_ctx, bool act_f32) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.scalar_type() == at::kFloat && q.is_contiguous(),
              "bm_talk_attention: q f32 [T, H, d] contiguous");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  TORCH_CHECK(G >= 1 && H % G == 0, "bm_talk_attention: heads must be a multiple of the key / value heads");
  TORCH_CHECK(rows.is_cuda() && rows.dim() == 3 && rows.scalar_type() == act_type(act_f32) && rows.is_contiguous() &&
                  rows.size(2) == 2 * G * d && rows.size(1) % 64 == 0,
              "bm_talk_attention: rows [blocks, bs (multiple of 64), 2 G d] in the activation dtype");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
                  block_tables.is_contiguous(),
              "bm_talk_attention: block tables int32 [B, W]");
  TORCH_CHECK(max_ctx >= 1 && max_ctx <= block_tables.size(1) * rows.size(1),
              "bm_talk_attention: block tables narrower than the longest context");
  check_idx(seq_of, at::kInt, T, "bm_talk_attention: seq_of int32 [T]");
  check_idx(pos, at::kLong, T, "bm_talk_attention: pos int64 [T]");
  const float* tp = talk_ptr(talk, H, "bm_talk_attention: talk f32 [H, H]");
  const void* gp = nullptr;
  int64_t gst = 0;
  if (gate.has_value() && gate->defined()) {
    TORCH_CHECK(gate->is_cuda() && gate->dim() == 2 && gate->size(0) == T && gate->size(1) == H * d &&
                    gate->scalar_type() == rows.scalar_type() && gate->stride(1) == 1,
                "bm_talk_attention: gate [T, H d] in the activation dtype");
    gp = gate->data_ptr();
    gst = gate->stride(0);
  }
  int kt = 0;
  TORCH_CHECK(illm::bm::talk_attention_plan(!act_f32, (int)H, (int)G, (int)d, &kt) > 0,
              "bm_talk_attention: these sizes do not fit the kernel (callers take the library-product path)");
  const int ns = illm::bm::talk_attention_splits(!act_f32, (int)T, (int)H, (int)G, (int)d, (int)max_ctx);
  Tensor out = at::empty({T, H * d}, rows.options());
  Tensor part;
  if (ns > 1) part = at::empty({T, ns, H, d + 2}, q.options());
  illm::bm::talk_attention(!act_f32, q.data_ptr<float>(), rows.data_ptr(), (int)rows.size(1),
                           block_tables.data_ptr<int32_t>(), (int)block_tables.size(1), seq_of.data_ptr<int32_t>(),
                           pos.data_ptr<int64_t>(), (float)scale, tp, gp, gst, out.data_ptr(),
                           ns > 1 ? part.data_ptr<float>() : nullptr, ns, (int)T, (int)H, (int)G, (int)d, stream());
  return out;
}

int64_t bm_talk_prefill_fits(int64_t H, int64_t G, int64_t d) {
  return illm::bm::talk_prefill_fits((int)H, (int)G, (int)d) ? 1 : 0;
}

void bm_talk_prefill(const Tensor& q, const Tensor& rows, const Tensor& table_row, const Tensor& pos, int64_t t0,
                     int64_t n, int64_t max_keys, double scale, const c10::optional<Tensor>& talk,
                     const c10::optional<Tensor>& gate, int64_t G, Tensor& out) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.scalar_type() == at::kFloat && q.is_contiguous(),
              "bm_talk_prefill: q f32 [T, H, d] contiguous");
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  TORCH_CHECK(illm::bm::talk_prefill_fits((int)H, (int)G, (int)d), "bm_talk_prefill: sizes outside the kernel's set");
  TORCH_CHECK(t0 >= 0 && n >= 1 && t0 + n <= T, "bm_talk_prefill: portion outside the step");
  TORCH_CHECK(rows.is_cuda() && rows.dim() == 3 && rows.scalar_type() == at::kBFloat16 && rows.is_contiguous() &&
                  rows.size(2) == 2 * G * d && rows.size(1) % 64 == 0,
              "bm_talk_prefill: rows bf16 [blocks, bs (multiple of 64), 2 G d]");
  TORCH_CHECK(table_row.is_cuda() && table_row.scalar_type() == at::kInt && table_row.dim() == 1 &&
                  table_row.is_contiguous(),
              "bm_talk_prefill: block table row int32 [W]");
  check_idx(pos, at::kLong, T, "bm_talk_prefill: pos int64 [T]");
  const float* tp = talk_ptr(talk, H, "bm_talk_prefill: talk f32 [H, H]");
  const void* gp = nullptr;
  int64_t gst = 0;
  if (gate.has_value() && gate->defined()) {
    TORCH_CHECK(gate->is_cuda() && gate->dim() == 2 && gate->size(0) == T && gate->size(1) == H * d &&
                    gate->scalar_type() == at::kBFloat16 && gate->stride(1) == 1,
                "bm_talk_prefill: gate bf16 [T, H d]");
    gp = gate->data_ptr();
    gst = gate->stride(0);
  }
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == at::kBFloat16 && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == T && out.size(1) == H * d,
              "bm_talk_prefill: out bf16 [T, H d]");
  TORCH_CHECK(max_keys >= n && max_keys <= table_row.numel() * rows.size(1),
              "bm_talk_prefill: block table row narrower than the portion's context");
  const int ns = illm::bm::talk_prefill_splits((int)n, (int)max_keys);
  Tensor part;
  if (ns > 1) part = at::empty({n, ns, H, d + 2}, q.options());
  illm::bm::talk_prefill(q.data_ptr<float>(), rows.data_ptr(), (int)rows.size(1), table_row.data_ptr<int32_t>(),
                         pos.data_ptr<int64_t>(), (int)t0, (int)n, (float)scale, tp, gp, gst, out.data_ptr(),
                         ns > 1 ? part.data_ptr<float>() : nullptr, ns, (int)H, (int)G, (int)d, stream());
}

std::tuple<Tensor, Tensor> bm_talk_softmax(Tensor& sc, const Tensor& pos, int64_t H, double scale,
                                           const c10::optional<Tensor>& talk, bool act_f32) {
  c10::DeviceGuard g(sc.device());
  check_f32_rows(sc, "bm_talk_softmax: scores f32 [nt H, L] contiguous");
  TORCH_CHECK(H >= 1 && H <= 64 && sc.size(0) % H == 0, "bm_talk_softmax: 1 <= H <= 64 rows per token");
  const int64_t nt = sc.size(0) / H, L = sc.size(1);
  check_idx(pos, at::kLong, nt, "bm_talk_softmax: pos int64 [nt]");
  const float* tp = talk_ptr(talk, H, "bm_talk_softmax: talk f32 [H, H]");
  Tensor hi, lo;
  if (act_f32) {
    hi = sc;
    lo = at::empty({0}, sc.options());
  } else {
    hi = at::empty({nt * H, L}, sc.options().dtype(at::kBFloat16));
    lo = at::empty({nt * H, L}, sc.options().dtype(at::kBFloat16));
  }
  illm::bm::talk_softmax(!act_f32, sc.data_ptr<float>(), pos.data_ptr<int64_t>(), (int)H, (float)scale, tp, nt, (int)L,
                         act_f32 ? nullptr : hi.data_ptr(), act_f32 ? nullptr : lo.data_ptr(), stream());
  return {hi, lo};
}

std::tuple<Tensor, Tensor> bm_moe_route(const Tensor& z, int64_t top, int64_t mode) {
  c10::DeviceGuard g(z.device());
  check_f32_rows(z, "bm_moe_route: router logits f32 [T, E]");
  const int64_t T = z.size(0), E = z.size(1);
  TORCH_CHECK(E >= 1 && E <= 512 && top >= 1 && top <= E, "bm_moe_route: 1 <= top <= experts <= 512");
  TORCH_CHECK(mode == 0 || (mode == 1 && top <= 64), "bm_moe_route: mode 0 (sigmoid) or 1 (softmax over the chosen, top <= 64)");
  Tensor idx = at::empty({T, top}, z.options().dtype(at::kInt));
  Tensor w = at::empty({T, top}, z.options());
  illm::bm::moe_route(z.data_ptr<float>(), (int)T, (int)E, (int)top, idx.data_ptr<int32_t>(), w.data_ptr<float>(),
                      (int)mode, stream());
  return {idx, w};
}

Tensor bm_moe_experts(const Tensor& h, const Tensor& idx, const Tensor& wts, const Tensor& w_gu, const Tensor& w_down,
                      double limit, double alpha, double up_shift, bool weigh_out) {
  c10::DeviceGuard g(h.device());
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && is_act(h) && h.is_contiguous(), "bm_moe_experts: h [T, W] contiguous");
  const int64_t T = h.size(0), W = h.size(1);
  TORCH_CHECK(idx.is_cuda() && idx.scalar_type() == at::kInt && idx.is_contiguous() && idx.dim() == 2 &&
                  idx.size(0) == T && idx.size(1) >= 1,
              "bm_moe_experts: idx int32 [T, top]");
  const int64_t top = idx.size(1), P = T * top;
  TORCH_CHECK(wts.is_cuda() && wts.scalar_type() == at::kFloat && wts.is_contiguous() && wts.numel() == P,
              "bm_moe_experts: weights f32 [T, top]");
  TORCH_CHECK(w_gu.is_cuda() && w_gu.dim() == 3 && w_gu.scalar_type() == h.scalar_type() && w_gu.is_contiguous() &&
                  w_gu.size(2) == W && w_gu.size(1) % 2 == 0,
              "bm_moe_experts: w_gu [E, 2 ff, W] of h's dtype");
  const int64_t E = w_gu.size(0), ff = w_gu.size(1) / 2;
  TORCH_CHECK(E <= 1024, "bm_moe_experts: at most 1024 experts");
  TORCH_CHECK(w_down.is_cuda() && w_down.dim() == 3 && w_down.scalar_type() == h.scalar_type() &&
                  w_down.is_contiguous() && w_down.size(0) == E && w_down.size(1) == W && w_down.size(2) == ff,
              "bm_moe_experts: w_down [E, W, ff] of h's dtype");
  auto iopt = h.options().dtype(at::kInt);
  Tensor off = at::empty({E + 1}, iopt), sorted = at::empty({P}, iopt);
  Tensor y = at::empty({P, ff}, h.options());
  Tensor out = at::empty({P, W}, h.options().dtype(at::kFloat));
  if (P == 0) return out.view({T, W});
  auto st = stream();
  illm::bm::moe_align(idx.data_ptr<int32_t>(), (int)P, (int)E, off.data_ptr<int32_t>(), sorted.data_ptr<int32_t>(), st);
  illm::bm::moe_glu(bf(h), h.data_ptr(), off.data_ptr<int32_t>(), sorted.data_ptr<int32_t>(), wts.data_ptr<float>(),
                    (int)top, w_gu.data_ptr(), y.data_ptr(), (int)P, (int)E, (int)ff, (int)W, (float)limit,
                    (float)alpha, (float)up_shift, weigh_out, st);
  illm::bm::moe_down(bf(h), y.data_ptr(), off.data_ptr<int32_t>(), sorted.data_ptr<int32_t>(), w_down.data_ptr(),
                     out.data_ptr<float>(), (int)P, (int)E, (int)ff, (int)W, weigh_out ? wts.data_ptr<float>() : nullptr,
                     st);
  if (top == 1) return out;
  return out.view({T, top, W}).sum(1);
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(ipex_llm_amd, m) {
  m.def("bm_rms_norm_rows(Tensor x, Tensor w, float eps, bool act_f32) -> (Tensor, Tensor)");
  m.def("bm_add_rms_norm(Tensor(a!) x, Tensor y, Tensor w, float eps, bool act_f32) -> Tensor");
  m.def("bm_add_rms_norm_rows(Tensor(a!) x, Tensor? y, Tensor w, float eps, bool act_f32) -> Tensor");
  m.def("bm_residual_add_scaled(Tensor(a!) x, Tensor y1, Tensor? s1, Tensor? y2, Tensor? y3, Tensor? s2, "
        "bool act_f32) -> Tensor");
  m.def("bm_canon_conv(Tensor h, Tensor w, Tensor(a!) state, Tensor cu, Tensor seq_of, Tensor slots, Tensor pos, "
        "bool act_f32) -> Tensor");
  m.def("bm_norm_canon(Tensor x, Tensor g, float eps, Tensor w, Tensor(a!) state, Tensor cu, Tensor seq_of, Tensor slots, "
        "Tensor pos, bool single, bool act_f32) -> (Tensor, Tensor, Tensor)");
  m.def("bm_relu_sq(Tensor y) -> Tensor");
  m.def("bm_glu_clamp(Tensor gu, float limit, float alpha) -> Tensor");
  m.def("bm_side_gate(Tensor z, Tensor table, Tensor ids, int offset) -> Tensor");
  m.def("bm_qk_norm_rope_store(Tensor q, Tensor k, Tensor? qn, Tensor? kn, float eps, Tensor table, Tensor pos, "
        "Tensor slots, Tensor(a!) rows) -> Tensor");
  m.def("bm_talk_attention_fits(bool bf16, int H, int G, int d) -> int");
  m.def("bm_talk_attention(Tensor q, Tensor rows, Tensor block_tables, Tensor seq_of, Tensor pos, float scale, "
        "Tensor? talk, Tensor? gate, int G, int max_ctx, bool act_f32) -> Tensor");
  m.def("bm_talk_prefill_fits(int H, int G, int d) -> int");
  m.def("bm_talk_prefill(Tensor q, Tensor rows, Tensor table_row, Tensor pos, int t0, int n, int max_keys, float scale, "
        "Tensor? talk, Tensor? gate, int G, Tensor(a!) out) -> ()");
  m.def("bm_talk_softmax(Tensor(a!) scores, Tensor pos, int H, float scale, Tensor? talk, bool act_f32) -> "
        "(Tensor, Tensor)");
  m.def("bm_moe_route(Tensor z, int top, int mode) -> (Tensor, Tensor)");
  m.def("bm_moe_experts(Tensor h, Tensor idx, Tensor wts, Tensor w_gu, Tensor w_down, float limit, float alpha, "
        "float up_shift, bool weigh_out) -> Tensor");
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CompositeExplicitAutograd, m) {
  m.impl("bm_talk_attention_fits", &bm_talk_attention_fits);
  m.impl("bm_talk_prefill_fits", &bm_talk_prefill_fits);
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CUDA, m) {
  m.impl("bm_rms_norm_rows", &bm_rms_norm_rows);
  m.impl("bm_add_rms_norm", &bm_add_rms_norm);
  m.impl("bm_add_rms_norm_rows", &bm_add_rms_norm_rows);
  m.impl("bm_residual_add_scaled", &bm_residual_add_scaled);
  m.impl("bm_canon_conv", &bm_canon_conv);
  m.impl("bm_norm_canon", &bm_norm_canon);
  m.impl("bm_relu_sq", &bm_relu_sq);
  m.impl("bm_glu_clamp", &bm_glu_clamp);
  m.impl("bm_side_gate", &bm_side_gate);
  m.impl("bm_qk_norm_rope_store", &bm_qk_norm_rope_store);
  m.impl("bm_talk_attention", &bm_talk_attention);
  m.impl("bm_talk_prefill", &bm_talk_prefill);
  m.impl("bm_talk_softmax", &bm_talk_softmax);
  m.impl("bm_moe_route", &bm_moe_route);
  m.impl("bm_moe_experts", &bm_moe_experts);
}
