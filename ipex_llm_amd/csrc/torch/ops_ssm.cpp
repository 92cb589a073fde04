// torch.ops.ipex_llm_amd.ssm_*: the kernels of the state-space mixer
// (csrc/hip/ssm.hip).  Every entry checks on the host that the operand
// shapes, dtypes and strides are what its kernel and grid assume.
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include "../hip/ssm.h"

using at::Tensor;

namespace {

hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }
bool is_act(const Tensor& t) { return t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat; }
bool bf(const Tensor& t) { return t.scalar_type() == at::kBFloat16; }

void check_idx(const Tensor& t, at::ScalarType ty, int64_t n, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == ty && t.is_contiguous() && t.numel() >= n, what);
}
void check_f32_vec(const Tensor& t, int64_t n, const char* what) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous() && t.numel() == n, what);
}

Tensor ssm_conv_silu(const Tensor& u, const Tensor& w, const c10::optional<Tensor>& b, Tensor& state, const Tensor& cu,
                     const Tensor& seq_of, const Tensor& slots, const Tensor& pos, bool single, bool act) {
  c10::DeviceGuard g(u.device());
  TORCH_CHECK(u.is_cuda() && u.dim() == 2 && is_act(u) && (u.size(1) <= 1 || u.stride(1) == 1) && u.stride(0) >= u.size(1),
              "ssm_conv_silu: u [T, C] (unit inner stride)");
  const int64_t T = u.size(0), C = u.size(1);
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == at::kFloat && w.is_contiguous() && w.dim() == 2 && w.size(0) == C &&
                  w.size(1) >= 1 && w.size(1) <= 16,
              "ssm_conv_silu: w f32 [C, taps], 1 <= taps <= 16");
  const int64_t taps = w.size(1);
  const bool has_b = b.has_value() && b->defined();
  if (has_b) check_f32_vec(*b, C, "ssm_conv_silu: bias f32 [C]");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 3 &&
                  state.size(1) == taps - 1 && state.size(2) == C,
              "ssm_conv_silu: state f32 [slots, taps - 1, C]");
  TORCH_CHECK(cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous() && cu.numel() >= 2,
              "ssm_conv_silu: cu int32 [B + 1]");
  const int64_t B = cu.numel() - 1;
  TORCH_CHECK(!single || B == T, "ssm_conv_silu: single means one token per sequence");
  TORCH_CHECK((C + 255) / 256 <= 65535, "ssm_conv_silu: too many channels for one launch");
  check_idx(seq_of, at::kInt, T, "ssm_conv_silu: seq_of int32 [T]");
  check_idx(slots, at::kInt, B, "ssm_conv_silu: state slots int32 [B]");
  check_idx(pos, at::kLong, T, "ssm_conv_silu: pos int64 [T]");
  Tensor out = at::empty({T, C}, u.options().dtype(at::kFloat));
  illm::ssm::conv_silu(bf(u), u.data_ptr(), u.stride(0), w.data_ptr<float>(), has_b ? b->data_ptr<float>() : nullptr, (int)taps,
                       state.data_ptr<float>(), cu.data_ptr<int32_t>(), seq_of.data_ptr<int32_t>(),
                       slots.data_ptr<int32_t>(), pos.data_ptr<int64_t>(), out.data_ptr<float>(), (int)T, (int)B, (int)C,
                       single, act, stream());
  return out;
}

Tensor ssm_selective_scan(const Tensor& x, const Tensor& Bm, const Tensor& Cm, const Tensor& dt, const Tensor& dt_bias,
                          const Tensor& a_log, const Tensor& d_skip, Tensor& S, const Tensor& cu, const Tensor& slots,
                          const Tensor& pos) {
  c10::DeviceGuard g(x.device());
  auto rows3 = [](const Tensor& t) {
    return t.is_cuda() && t.dim() == 3 && t.scalar_type() == at::kFloat && t.stride(2) == 1 && t.stride(1) == t.size(2) &&
           t.stride(0) >= t.size(1) * t.size(2);
  };
  TORCH_CHECK(rows3(x), "ssm_selective_scan: x f32 [T, H, P] (heads contiguous in a row)");
  const int64_t T = x.size(0), H = x.size(1), P = x.size(2);
  TORCH_CHECK(rows3(Bm) && rows3(Cm) && Bm.size(0) == T && Cm.sizes() == Bm.sizes(),
              "ssm_selective_scan: B / C f32 [T, G, N] (groups contiguous in a row)");
  const int64_t G = Bm.size(1), N = Bm.size(2);
  TORCH_CHECK(G >= 1 && H % G == 0, "ssm_selective_scan: heads must be a multiple of groups");
  TORCH_CHECK(N >= 1 && N <= illm::ssm::kScanMaxState, "ssm_selective_scan: state size 1..", illm::ssm::kScanMaxState);
  TORCH_CHECK(dt.is_cuda() && dt.dim() == 2 && is_act(dt) && dt.size(0) == T && dt.size(1) == H &&
                  (H == 1 || dt.stride(1) == 1),
              "ssm_selective_scan: dt [T, H] bf16 / f32");
  check_f32_vec(dt_bias, H, "ssm_selective_scan: dt_bias f32 [H]");
  check_f32_vec(a_log, H, "ssm_selective_scan: a_log f32 [H]");
  check_f32_vec(d_skip, H, "ssm_selective_scan: d_skip f32 [H]");
  TORCH_CHECK(S.is_cuda() && S.scalar_type() == at::kFloat && S.is_contiguous() && S.dim() == 4 && S.size(1) == H &&
                  S.size(2) == N && S.size(3) == P,
              "ssm_selective_scan: state f32 [slots, H, N, P]");
  TORCH_CHECK(cu.is_cuda() && cu.scalar_type() == at::kInt && cu.is_contiguous() && cu.numel() >= 2,
              "ssm_selective_scan: cu int32 [B + 1]");
  const int64_t B = cu.numel() - 1;
  TORCH_CHECK(H <= 65535 && (P + 63) / 64 <= 65535, "ssm_selective_scan: too many heads for one launch");
  check_idx(slots, at::kInt, B, "ssm_selective_scan: state slots int32 [B]");
  check_idx(pos, at::kLong, T, "ssm_selective_scan: pos int64 [T]");
  Tensor out = at::empty({T, H, P}, x.options());
  if (T == 0) return out;
  illm::ssm::selective_scan(bf(dt), x.data_ptr<float>(), x.stride(0), Bm.data_ptr<float>(), Bm.stride(0),
                            Cm.data_ptr<float>(), Cm.stride(0), dt.data_ptr(), dt.stride(0), dt_bias.data_ptr<float>(),
                            a_log.data_ptr<float>(), d_skip.data_ptr<float>(), S.data_ptr<float>(),
                            cu.data_ptr<int32_t>(), slots.data_ptr<int32_t>(), pos.data_ptr<int64_t>(),
                            out.data_ptr<float>(), (int)B, (int)H, (int)P, (int)G, (int)N, stream());
  return out;
}

Tensor ssm_gated_group_norm(const Tensor& y, const Tensor& z, const Tensor& w, int64_t groups, double eps, bool act_f32) {
  c10::DeviceGuard g(y.device());
  TORCH_CHECK(y.is_cuda() && y.dim() == 2 && y.scalar_type() == at::kFloat && y.is_contiguous(),
              "ssm_gated_group_norm: y f32 [T, C]");
  const int64_t T = y.size(0), C = y.size(1);
  const auto at_ = act_f32 ? at::kFloat : at::kBFloat16;
  TORCH_CHECK(z.is_cuda() && z.dim() == 2 && z.scalar_type() == at_ && z.size(0) == T && z.size(1) == C &&
                  (C == 1 || z.stride(1) == 1),
              "ssm_gated_group_norm: z [T, C] in the activation dtype (unit inner stride)");
  TORCH_CHECK(w.is_cuda() && w.scalar_type() == at_ && w.is_contiguous() && w.numel() == C,
              "ssm_gated_group_norm: w [C] in the activation dtype");
  TORCH_CHECK(groups >= 1 && groups <= 65535 && C % groups == 0, "ssm_gated_group_norm: C must split into the groups");
  Tensor out = at::empty({T, C}, y.options().dtype(at_));
  illm::ssm::gated_group_norm(!act_f32, y.data_ptr<float>(), z.data_ptr(), z.stride(0), w.data_ptr(), out.data_ptr(),
                              (int)T, (int)C, (int)groups, (float)eps, stream());
  return out;
}

}  // namespace

TORCH_LIBRARY_FRAGMENT(ipex_llm_amd, m) {
  m.def("ssm_conv_silu(Tensor u, Tensor w, Tensor? b, Tensor(a!) state, Tensor cu, Tensor seq_of, Tensor slots, Tensor pos, "
        "bool single, bool act) -> Tensor");
  m.def("ssm_selective_scan(Tensor x, Tensor Bm, Tensor Cm, Tensor dt, Tensor dt_bias, Tensor a_log, Tensor d_skip, "
        "Tensor(a!) S, Tensor cu, Tensor slots, Tensor pos) -> Tensor");
  m.def("ssm_gated_group_norm(Tensor y, Tensor z, Tensor w, int groups, float eps, bool act_f32) -> Tensor");
}

TORCH_LIBRARY_IMPL(ipex_llm_amd, CUDA, m) {
  m.impl("ssm_conv_silu", &ssm_conv_silu);
  m.impl("ssm_selective_scan", &ssm_selective_scan);
  m.impl("ssm_gated_group_norm", &ssm_gated_group_norm);
}
