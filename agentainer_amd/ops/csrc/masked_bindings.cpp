// pybind11 bindings: scalar-gain norms, PolyNorm, rotary + q/k norm + K/V
// append, masked grouped-query attention.
#include <torch/extension.h>

void scalar_postnorm_residual(torch::Tensor x, torch::Tensor y,
                              torch::Tensor gain, double eps, torch::Tensor h);
void scalar_rmsnorm(torch::Tensor out, torch::Tensor x, torch::Tensor gain,
                    double eps);
void poly_norm(torch::Tensor out, torch::Tensor z, torch::Tensor coef,
               double eps);
torch::Tensor rotary_table(torch::Tensor positions, torch::Tensor freqs,
                           double amp);
void rotary_norm_append(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                        torch::Tensor k_cache, torch::Tensor v_cache,
                        torch::Tensor cos_sin, torch::Tensor slot_mapping,
                        double eps, c10::optional<torch::Tensor> q_w,
                        c10::optional<torch::Tensor> k_w, bool norm_first);
void masked_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                      torch::Tensor v_cache, torch::Tensor page_table,
                      torch::Tensor seq_lens,
                      c10::optional<torch::Tensor> query_starts,
                      c10::optional<torch::Tensor> query_lens, double scale,
                      long mask_kind, long mask_size, long keep_first,
                      bool sigmoid_weights, double softcap,
                      c10::optional<torch::Tensor> key_bias,
                      c10::optional<torch::Tensor> head_gate, long max_qlen,
                      bool force_simple, long splits,
                      c10::optional<torch::Tensor> dist_bias);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "agentainer_amd CDNA4 (gfx950) masked-attention family kernels";
  m.def("scalar_postnorm_residual", &scalar_postnorm_residual,
        "x += gain * y / rms(y); h = x in the compute dtype");
  m.def("scalar_rmsnorm", &scalar_rmsnorm, "gain * x / rms(x)");
  m.def("poly_norm", &poly_norm, "a U(z) + b U(z^2) + c U(z^3) + e");
  m.def("rotary_table", &rotary_table,
        "cos | sin of position * frequency for one step's tokens");
  m.def("rotary_norm_append", &rotary_norm_append,
        "rotary + q/k rms norm; append K/V to the paged pools");
  m.def("masked_attention", &masked_attention,
        "chunk / window masked GQA with softmax or sigmoid weights and an "
        "optional logarithmic distance bias");
}
