// pybind11 bindings: hashed bigram embedding, gated residual + layer norm,
// xIELU, token-side gate, sigmoid group-limited routing, output-weighted
// gated experts, latent rotary append, plain K/V append, output gate.
#include <torch/extension.h>

using OptT = c10::optional<torch::Tensor>;

void bigram_embed(torch::Tensor x, torch::Tensor ids, torch::Tensor embed,
                  OptT bigram, double scale, long mul_prev, long mul_cur,
                  long buckets, OptT prev_state, torch::Tensor state_slots,
                  torch::Tensor seq_lens, OptT query_starts, OptT query_lens);
void residual_update_norm(torch::Tensor x, OptT y, long update, OptT gate,
                          OptT gate_bias, OptT rms_w, double eps, OptT norm_w,
                          OptT norm_b, OptT h);
void xielu(torch::Tensor out, torch::Tensor z, torch::Tensor coef);
void gelu_gate_rows(torch::Tensor out, torch::Tensor t, torch::Tensor table,
                    torch::Tensor ids, long col0);
void sigmoid_gate_rows(torch::Tensor out, torch::Tensor a, torch::Tensor gate);
void grouped_sigmoid_route(torch::Tensor weight, torch::Tensor logits,
                           OptT correction, long n_experts, long top,
                           long n_groups, long keep_groups, long group_top);
void routed_silu_glu(torch::Tensor out, torch::Tensor gu, torch::Tensor weight,
                     long n_experts, long ff, long tail_ff);
void latent_rotary_append(torch::Tensor proj, long heads, long q_head,
                          long q_rot_off, long kv_off, long kv_rank,
                          long rot_dim, torch::Tensor w_kv, double eps,
                          torch::Tensor cos_sin, torch::Tensor cache,
                          torch::Tensor slot_mapping);
void head_kv_append(torch::Tensor k, torch::Tensor v, torch::Tensor k_cache,
               torch::Tensor v_cache, torch::Tensor slot_mapping);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "agentainer_amd CDNA4 (gfx950) gated-residual family kernels";
  m.def("bigram_embed", &bigram_embed,
        "scaled embedding + hashed bigram row; previous token kept as state");
  m.def("residual_update_norm", &residual_update_norm,
        "gated / unit-rms fp32 residual update fused with a layer norm");
  m.def("xielu", &xielu, "xIELU activation");
  m.def("gelu_gate_rows", &gelu_gate_rows,
        "gelu_tanh(t) * table[id] column slice");
  m.def("sigmoid_gate_rows", &sigmoid_gate_rows, "a * sigmoid(gate)");
  m.def("grouped_sigmoid_route", &grouped_sigmoid_route,
        "sigmoid scores, group-limited top-k, always-on gates");
  m.def("routed_silu_glu", &routed_silu_glu,
        "stacked SiLU-gated experts times routing weight, with a tail expert");
  m.def("latent_rotary_append", &latent_rotary_append,
        "rotate query parts, norm the latent, append latent | rotated key");
  m.def("head_kv_append", &head_kv_append, "copy K/V rows into the per-head pools");
}
