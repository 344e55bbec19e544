// torch op registration for the "moe" kernel group of kaito_amd's gfx950
// extension (one shared library per group, loaded on first use).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace kaito {
void moe_gate_silu(at::Tensor act, at::Tensor x, at::Tensor w_gate_up,
                   at::Tensor sorted_ids, at::Tensor offsets, at::Tensor bias,
                   int64_t act_mode, int64_t e_base, int64_t n_local_experts,
                   double act_limit);
void moe_down_scatter(at::Tensor out, at::Tensor act, at::Tensor w_down,
                      at::Tensor sorted_ids, at::Tensor gates,
                      at::Tensor offsets, at::Tensor bias, int64_t e_base,
                      int64_t n_local_experts);
}  // namespace kaito

TORCH_LIBRARY_FRAGMENT(kaito, m) {
  m.def("moe_gate_silu(Tensor(a!) act, Tensor x, Tensor w_gate_up, Tensor sorted_ids, Tensor offsets, Tensor bias, int act_mode, int e_base, int n_local_experts, float act_limit) -> ()");
  m.def("moe_down_scatter(Tensor(a!) out, Tensor act, Tensor w_down, Tensor sorted_ids, Tensor gates, Tensor offsets, Tensor bias, int e_base, int n_local_experts) -> ()");
}

TORCH_LIBRARY_IMPL(kaito, CUDA, m) {
  m.impl("moe_gate_silu", &kaito::moe_gate_silu);
  m.impl("moe_down_scatter", &kaito::moe_down_scatter);
}
