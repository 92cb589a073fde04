// torch.ops.ipex_llm_amd.gm_*: the kernels of the gated recurrent mixers and
// the two-norm parallel blocks (csrc/hip/gatedmix.hip).  Every entry checks
// on the host that the operand shapes, dtypes and strides are what its kernel
// and grid assume.
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include <tuple>

#include "../hip/gatedmix.h"

using at::Tensor;

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }
bool is_act(const Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
bool bf(const Tensor& t) { return t.scalar_type() == at::kBFloat16; }
bool has(const c10::optional<Tensor>& t) { return t.has_value() && t->defined(); }
at::ScalarType act_type(bool act_f32) { return act_f32 ? at::kFloat : at::kBFloat16; }

void check_idx(const Tensor& t, at::ScalarType ty, int64_t n, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == ty && t.is_contiguous() && t.numel() >= n, what);
}
bool vec(const Tensor& t, at::ScalarType ty, int64_t n) {
  return t.is_cuda() && t.scalar_type() == ty && t.is_contiguous() && t.numel() == n;
}
// [T, heads, n] view of a projection's rows: heads contiguous inside a row
bool head_rows(const Tensor& t, at::ScalarType ty) {
  return t.is_cuda() && t.dim() == 3 && t.scalar_type() == ty && t.stride(2) == 1 && t.stride(1) == t.size(2) &&
         t.stride(0) >= t.size(1) * t.size(2);
}
// the slots a step names must exist: one read of the step's (small) slot list on the host would cost a
// synchronisation, so the callers pass slots the allocator handed out; the pools' sizes are checked here
void check_step(const Tensor& cu, const Tensor& slots, const Tensor& pos, int64_t T, const char* what) {
  TORCH_CHECK(cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous() && cu.numel() >= 2, what);
  check_idx(slots, at::kInt, cu.numel() - 1, what);
  check_idx(pos, at::kLong, T, what);
}

std::tuple<Tensor, Tensor> gm_layer_norm_pair_shift(const Tensor& x, const Tensor& w1, const c10::optional<Tensor>& w2,
                                                    const c10::optional<Tensor>& mu, double eps,
                                                    const c10::optional<Tensor>& state, const Tensor& cu,
                                                    const Tensor& seq_of, const Tensor& slots, const Tensor& pos,
                                                    bool single, bool act_f32) {
  c10::DeviceGuard g(x.device());
  TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.scalar_type() == at::kFloat && x.is_contiguous(),
              "gm_layer_norm_pair_shift: x f32 [T, W] contiguous");
  const int64_t T = x.size(0), W = x.size(1);
  const auto ty = act_type(act_f32);
  TORCH_CHECK(vec(w1, ty, W) && (!has(w2) || vec(*w2, ty, W)),
              "gm_layer_norm_pair_shift: norm weights [W] in the activation dtype");
  int64_t B = 0;
  if (has(mu)) {
    TORCH_CHECK(vec(*mu, at::kFloat, W), "gm_layer_norm_pair_shift: shift f32 [W]");
    TORCH_CHECK(has(state) && state->is_cuda() && state->scalar_type() == at::kFloat && state->is_contiguous() &&
                    state->dim() == 2 && state->size(1) == W,
                "gm_layer_norm_pair_shift: state f32 [slots, W]");
    check_step(cu, slots, pos, T, "gm_layer_norm_pair_shift: cu int32 [B + 1], slots int32 [B], pos int64 [T]");
    check_idx(seq_of, at::kInt, T, "gm_layer_norm_pair_shift: seq_of int32 [T]");
    B = cu.numel() - 1;
    TORCH_CHECK(!single || B == T, "gm_layer_norm_pair_shift: single means one token per sequence");
  }
  Tensor h1 = at::empty({T, W}, x.options().dtype(ty));
  Tensor h2 = has(w2) ? at::empty({T, W}, x.options().dtype(ty)) : at::empty({0}, x.options().dtype(ty));
  Tensor last;
  if (has(mu) && !single) last = at::empty({B, W}, x.options());
  illm::gm::layer_norm_pair_shift(!act_f32, x.data_ptr<float>(), w1.data_ptr(), has(w2) ? w2->data_ptr() : nullptr,
                                  has(mu) ? mu->data_ptr<float>() : nullptr, (float)eps,
                                  has(mu) ? state->data_ptr<float>() : nullptr,
                                  has(mu) ? cu.data_ptr<int32_t>() : nullptr, has(mu) ? seq_of.data_ptr<int32_t>() : nullptr,
                                  has(mu) ? slots.data_ptr<int32_t>() : nullptr, has(mu) ? pos.data_ptr<int64_t>() : nullptr,
                                  h1.data_ptr(), has(w2) ? h2.data_ptr() : nullptr,
                                  last.defined() ? last.data_ptr<float>() : nullptr, (int)T, (int)B, (int)W, single,
                                  stream());
  return {h1, h2};
}

Tensor gm_mingru_scan(const Tensor& y, int64_t width, Tensor& state, const Tensor& cu, const Tensor& slots,
                      const Tensor& pos, int64_t max_n) {
  c10::DeviceGuard g(y.device());
  TORCH_CHECK(y.is_cuda() && y.dim() == 2 && is_act(y) && y.size(1) == 3 * width && width >= 1 && y.stride(1) == 1 &&
                  y.stride(0) >= y.size(1),
              "gm_mingru_scan: y [T, 3 width] (unit inner stride)");
  const int64_t T = y.size(0);
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 2 &&
                  state.size(1) == width,
              "gm_mingru_scan: state f32 [slots, width]");
  check_step(cu, slots, pos, T, "gm_mingru_scan: cu int32 [B + 1], slots int32 [B], pos int64 [T]");
  const int64_t B = cu.numel() - 1;
  TORCH_CHECK(B <= 65535, "gm_mingru_scan: too many sequences for one launch");
  Tensor out = at::empty({T, width}, y.options());
  if (T == 0) return out;
  illm::gm::mingru_scan(bf(y), y.data_ptr(), y.stride(0), (int)width, state.data_ptr<float>(), cu.data_ptr<int32_t>(),
                        slots.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), out.data_ptr(), (int)B, (int)max_n, stream());
  return out;
}

Tensor gm_gla_scan(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& a, double tau, double q_scale,
                   Tensor& S, const Tensor& cu, const Tensor& slots, const Tensor& pos) {
  c10::DeviceGuard g(q.device());
  TORCH_CHECK(is_act(q) && head_rows(q, q.scalar_type()), "gm_gla_scan: q [T, H, d] (heads contiguous in a row)");
  const auto ty = q.scalar_type();
  const int64_t T = q.size(0), H = q.size(1), d = q.size(2);
  TORCH_CHECK(head_rows(k, ty) && k.sizes() == q.sizes() && head_rows(a, ty) && a.sizes() == q.sizes(),
              "gm_gla_scan: k and the decay's input [T, H, d] like q");
  TORCH_CHECK(head_rows(v, ty) && v.size(0) == T && v.size(1) == H, "gm_gla_scan: v [T, H, dv]");
  const int64_t dv = v.size(2);
  TORCH_CHECK(d >= 1 && d <= illm::gm::kGlaMaxDim && dv >= 1 && tau > 0, "gm_gla_scan: key size 1..", illm::gm::kGlaMaxDim);
  TORCH_CHECK(S.is_cuda() && S.scalar_type() == at::kFloat && S.is_contiguous() && S.dim() == 4 && S.size(1) == H &&
                  S.size(2) == d && S.size(3) == dv,
              "gm_gla_scan: state f32 [slots, H, d, dv]");
  check_step(cu, slots, pos, T, "gm_gla_scan: cu int32 [B + 1], slots int32 [B], pos int64 [T]");
  const int64_t B = cu.numel() - 1;
  TORCH_CHECK(H <= 65535 && (dv + 63) / 64 <= 65535, "gm_gla_scan: too many heads for one launch");
  Tensor out = at::empty({T, H, dv}, q.options().dtype(at::kFloat));
  if (T == 0) return out;
  illm::gm::gla_scan(bf(q), q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), a.data_ptr(),
                     a.stride(0), (float)tau, (float)q_scale, S.data_ptr<float>(), cu.data_ptr<int32_t>(),
                     slots.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), out.data_ptr<float>(), (int)B, (int)H, (int)d,
                     (int)dv, stream());
  return out;
}

Tensor gm_gla_piece_decay(const Tensor& a, const Tensor& cu, double tau) {
  c10::DeviceGuard g(a.device());
  TORCH_CHECK(is_act(a) && head_rows(a, a.scalar_type()), "gm_gla_piece_decay: a [T, H, d] (heads contiguous in a row)");
  TORCH_CHECK(cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous() && cu.numel() >= 2 && tau > 0,
              "gm_gla_piece_decay: cu int32 [NP + 1], tau > 0");
  const int64_t NP = cu.numel() - 1, H = a.size(1), d = a.size(2);
  TORCH_CHECK(H <= 65535, "gm_gla_piece_decay: too many heads for one launch");
  Tensor P = at::empty({NP, H, d}, a.options().dtype(at::kFloat));
  illm::gm::gla_piece_decay(bf(a), a.data_ptr(), a.stride(0), cu.data_ptr<int32_t>(), (float)tau, P.data_ptr<float>(),
                            (int)NP, (int)H, (int)d, stream());
  return P;
}

void gm_gla_chain_(const Tensor& Z, Tensor& Sin, const Tensor& P, const Tensor& seqs) {
  c10::DeviceGuard g(Z.device());
  TORCH_CHECK(Z.is_cuda() && Z.scalar_type() == at::kFloat && Z.is_contiguous() && Z.dim() == 4,
              "gm_gla_chain_: Z f32 [pieces + 1, H, d, dv]");
  TORCH_CHECK(Sin.is_cuda() && Sin.scalar_type() == at::kFloat && Sin.is_contiguous() && Sin.sizes() == Z.sizes(),
              "gm_gla_chain_: Sin like Z");
  const int64_t H = Z.size(1), d = Z.size(2), dv = Z.size(3);
  TORCH_CHECK(P.is_cuda() && P.scalar_type() == at::kFloat && P.is_contiguous() && P.dim() == 3 &&
                  P.size(0) + 1 == Z.size(0) && P.size(1) == H && P.size(2) == d,
              "gm_gla_chain_: P f32 [pieces, H, d]");
  TORCH_CHECK(seqs.is_cuda() && seqs.scalar_type() == at::kInt && seqs.is_contiguous() && seqs.dim() == 2 &&
                  seqs.size(1) == 2 && seqs.size(0) <= 65535,
              "gm_gla_chain_: seqs int32 [n, 2]");
  illm::gm::gla_chain(Z.data_ptr<float>(), Sin.data_ptr<float>(), P.data_ptr<float>(), seqs.data_ptr<int32_t>(),
                      (int)seqs.size(0), (int)H, (int)d, (int)dv, stream());
}

Tensor gm_head_rms_silu(const Tensor& o, const Tensor& w, const Tensor& gate, double eps, bool act_f32) {
  c10::DeviceGuard g(o.device());
  TORCH_CHECK(o.is_cuda() && o.dim() == 3 && o.scalar_type() == at::kFloat && o.is_contiguous(),
              "gm_head_rms_silu: o f32 [T, H, dv] contiguous");
  const int64_t T = o.size(0), H = o.size(1), dv = o.size(2);
  const auto ty = act_type(act_f32);
  TORCH_CHECK(vec(w, ty, dv), "gm_head_rms_silu: weight [dv] in the activation dtype");
  TORCH_CHECK(gate.is_cuda() && gate.dim() == 2 && gate.scalar_type() == ty && gate.size(0) == T &&
                  gate.size(1) == H * dv && (H * dv == 1 || gate.stride(1) == 1),
              "gm_head_rms_silu: gate [T, H dv] in the activation dtype (unit inner stride)");
  TORCH_CHECK(H <= 65535, "gm_head_rms_silu: too many heads for one launch");
  Tensor out = at::empty({T, H * dv}, o.options().dtype(ty));
  illm::gm::head_rms_silu(!act_f32, o.data_ptr<float>(), w.data_ptr(), gate.data_ptr(), gate.stride(0), out.data_ptr(),
                          (int)T, (int)H, (int)dv, (float)eps, stream());
  return out;
}

Tensor gm_rms_pair_mean(const Tensor& a, const Tensor& b, const Tensor& wa, const Tensor& wb, double eps, bool act_f32) {
  c10::DeviceGuard g(a.device());
  const auto ty = a.scalar_type();
  TORCH_CHECK(a.is_cuda() && a.dim() == 2 && is_act(a) && a.is_contiguous() && b.is_cuda() && b.scalar_type() == ty &&
                  b.is_contiguous() && b.sizes() == a.sizes(),
              "gm_rms_pair_mean: a, b [T, W] contiguous, one dtype");
  TORCH_CHECK(ty == act_type(act_f32), "gm_rms_pair_mean: the result has the inputs' dtype");
  const int64_t T = a.size(0), W = a.size(1);
  TORCH_CHECK(vec(wa, ty, W) && vec(wb, ty, W), "gm_rms_pair_mean: weights [W] of a's dtype");
  Tensor out = at::empty({T, W}, a.options());
  illm::gm::rms_pair_mean(bf(a), a.data_ptr(), b.data_ptr(), wa.data_ptr(), wb.data_ptr(), out.data_ptr(), (int)T,
                          (int)W, (float)eps, stream());
  return out;
}

Tensor gm_softcap_(Tensor& x, double cap) {
  c10::DeviceGuard g(x.device());
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kFloat && x.is_contiguous() && cap > 0,
              "gm_softcap_: x f32 contiguous, cap > 0");
  illm::gm::softcap(x.data_ptr<float>(), x.numel(), (float)cap, stream());
  return x;
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(ipex_llm_amd, m) {
  m.def("gm_layer_norm_pair_shift(Tensor x, Tensor w1, Tensor? w2, Tensor? mu, float eps, Tensor(a!)? state, Tensor cu, "
        "Tensor seq_of, Tensor slots, Tensor pos, bool single, bool act_f32) -> (Tensor, Tensor)");
  m.def("gm_mingru_scan(Tensor y, int width, Tensor(a!) state, Tensor cu, Tensor slots, Tensor pos, int max_n) -> Tensor");
  m.def("gm_gla_scan(Tensor q, Tensor k, Tensor v, Tensor a, float tau, float q_scale, Tensor(a!) S, Tensor cu, "
        "Tensor slots, Tensor pos) -> Tensor");
  m.def("gm_gla_piece_decay(Tensor a, Tensor cu, float tau) -> Tensor");
  m.def("gm_gla_chain_(Tensor Z, Tensor(a!) Sin, Tensor P, Tensor seqs) -> ()");
  m.def("gm_head_rms_silu(Tensor o, Tensor w, Tensor gate, float eps, bool act_f32) -> Tensor");
  m.def("gm_rms_pair_mean(Tensor a, Tensor b, Tensor wa, Tensor wb, float eps, bool act_f32) -> Tensor");
  m.def("gm_softcap_(Tensor(a!) x, float cap) -> Tensor(a!)");
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CUDA, m) {
  m.impl("gm_layer_norm_pair_shift", &gm_layer_norm_pair_shift);
  m.impl("gm_mingru_scan", &gm_mingru_scan);
  m.impl("gm_gla_scan", &gm_gla_scan);
  m.impl("gm_gla_piece_decay", &gm_gla_piece_decay);
  m.impl("gm_gla_chain_", &gm_gla_chain_);
  m.impl("gm_head_rms_silu", &gm_head_rms_silu);
  m.impl("gm_rms_pair_mean", &gm_rms_pair_mean);
  m.impl("gm_softcap_", &gm_softcap_);
}
