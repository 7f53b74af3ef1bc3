// pybind11 bindings: post-norm residual, short convolutions with a
// per-sequence tail, matrix-memory recurrences, head norm + gate,
// group-limited softmax routing, clamped gated experts.
#include <torch/extension.h>

using OptT = c10::optional<torch::Tensor>;

void postln_rmsnorm_residual(torch::Tensor x, OptT y, double y_scale, OptT y2,
                             double y2_scale, double alpha, OptT row_add,
                             torch::Tensor w1p, double eps, torch::Tensor h);
void short_conv_state(torch::Tensor out, torch::Tensor u, torch::Tensor w,
                      torch::Tensor tail, torch::Tensor state_slots,
                      torch::Tensor seq_lens, OptT query_starts,
                      OptT query_lens, bool silu, long norm_channels,
                      long head_dim, long lead_channels, double lead_scale,
                      double l2_eps);
void matrix_memory_scan(long kind, torch::Tensor out, torch::Tensor q,
                        torch::Tensor k, torch::Tensor v, torch::Tensor gate,
                        OptT gate_bias, OptT head_rate, OptT beta,
                        double q_scale, double gate_param, torch::Tensor S,
                        OptT n_state, OptT m_state, torch::Tensor state_slots,
                        torch::Tensor seq_lens, OptT query_starts,
                        OptT query_lens, long lanes);
void head_rmsnorm_gate(torch::Tensor out, torch::Tensor o, torch::Tensor w,
                       torch::Tensor gate, double eps, bool silu_gate);
void grouped_softmax_route(torch::Tensor weight, torch::Tensor logits,
                           OptT correction, long top, long n_groups,
                           long keep_groups, double scale);
void routed_clamped_glu(torch::Tensor out, torch::Tensor gu,
                        torch::Tensor weight, long n_experts, double limit,
                        double slope);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "agentainer_amd CDNA4 (gfx950) recurrent-family kernels";
  m.def("postln_rmsnorm_residual", &postln_rmsnorm_residual,
        "x <- rms_norm(a x + s1 y + s2 y2) * w; h = x in the compute dtype");
  m.def("short_conv_state", &short_conv_state,
        "depthwise causal convolution with a per-sequence tail");
  m.def("matrix_memory_scan", &matrix_memory_scan,
        "gated linear attention / gated delta rule / mLSTM over state");
  m.def("head_rmsnorm_gate", &head_rmsnorm_gate,
        "per-head RMS norm, weight and output gate");
  m.def("grouped_softmax_route", &grouped_softmax_route,
        "softmax scores, group-limited top-k, renormalized weights");
  m.def("routed_clamped_glu", &routed_clamped_glu,
        "stacked clamped gated expert activation times routing weight");
}
