// Matrix-memory recurrences over per-sequence state (gfx950): gated linear
// attention, gated delta rule with per-key-channel decay, and the mLSTM
// memory with a running-maximum stabilizer — plus the per-head output norm
// and gate that follow them.
//
// Per head the memory S has `D` key rows and `Dv` value columns; every
// column evolves on its own given the token's k, q and decays:
//
//   S'   = g (.) S                      (g: per key row; mLSTM: one number)
//   a1_j = sum_r S'[r, j] k[r]          (delta rule only)
//   a2_j = sum_r S'[r, j] q[r]
//   u_j  = beta (v_j - a1_j)  |  v_j  |  e^(i - m') v_j
//   S    = S' + k u^T,   o_j = a2_j + u_j (k . q)     [= (S^T q)_j]
//
// so the work is cut over (sequence, head, block of value columns): a wave
// owns 64 / NSUB columns, NSUB adjacent lanes share a column and split its
// key rows (held in registers for the whole portion), the dot products are
// reduced over those lanes by DPP moves. The pool keeps S transposed
// ([slots, H, Dv, D]: a column's rows are contiguous) and the row -> lane
// mapping interleaves the sub-lanes by float4, so state loads and stores
// are 16-byte accesses that are contiguous across the NSUB lanes of a
// column, and the staged k / q / decay vectors are read from LDS as
// conflict-free float4. Four waves form a workgroup and share the staging:
// each wave loads and stages a quarter of a chunk's tokens for all four.
//
// Tokens are processed strictly in order, eight at a time: the raw inputs
// of the NEXT eight tokens are loaded into registers while the current
// eight are computed. The per-channel decays (sigmoid / softplus / exp) are
// evaluated beforehand by a fully parallel pass, the mLSTM gates and the
// running maximum by one wave per chunk (lane c: token c) — the serial
// loop holds multiply-adds only. Prompt portions and single decoded tokens
// run the same code, so a position's result does not depend on where the
// prompt was cut beyond the summation order of a launch's lane split. A
// sequence whose first row sits at position 0 starts from zero state; the
// final state is written back at the end; the mLSTM normalizer and maximum
// go through a per-row buffer (every column block reads them at its start).

#include "matrix_memory_kernel.h"

namespace mm {
void launch_gla(const ScanArgs& a, int B, int lanes, bool bf16, hipStream_t s);
void launch_delta(const ScanArgs& a, int B, int lanes, bool bf16,
                  hipStream_t s);
void launch_mlstm(const ScanArgs& a, int B, int lanes, bool bf16,
                  hipStream_t s);
}  // namespace mm

namespace {

using mm::KIND_GLA;
using mm::KIND_DELTA;
using mm::KIND_MLSTM;
using mm::ScanArgs;

// Per-key-channel decays, evaluated once per token and channel by a fully
// parallel pass (the recurrence kernel is latency-bound and must not spend
// its serial time on exp / log):
//   gla:   a = exp(logsigmoid(z + b) * inv_tau)
//   delta: g = exp(-exp(rate[h]) * softplus(z + b))
template <int KIND>
__global__ void decay_kernel(float* __restrict__ out,
                             const float* __restrict__ z, long z_rs,
                             const float* __restrict__ bias,
                             const float* __restrict__ head_rate, float param,
                             long n, int HD, int D) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long t = i / HD;
  const int c = (int)(i % HD);
  const float x = z[t * z_rs + c] + bias[c];
  float r;
  if constexpr (KIND == KIND_GLA) {
    r = expf(mm::log_sigmoid(x) * param);
  } else {
    r = expf(-expf(head_rate[c / D]) * mm::soft_plus(x));
  }
  out[i] = r;
}

__global__ void scatter_nm_kernel(float* __restrict__ n_state,
                                  float* __restrict__ m_state,
                                  const float* __restrict__ n_new,
                                  const float* __restrict__ m_new,
                                  const long* __restrict__ slots,
                                  const int* __restrict__ q_lens, int HD,
                                  int H) {
  const int b = blockIdx.y;
  if (q_lens && q_lens[b] <= 0) return;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  const long slot = slots[b];
  if (i < HD) n_state[slot * HD + i] = n_new[(long)b * HD + i];
  if (i < H) m_state[slot * H + i] = m_new[(long)b * H + i];
}

// ---- per-head RMS norm * weight * act(gate) ------------------------------

constexpr int MAXV = 8;   // value channels per lane: heads of up to 512

template <typename T, typename TG>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(
    T* __restrict__ out, const float* __restrict__ o,
    const float* __restrict__ w, int w_shared, const TG* __restrict__ gate,
    long gate_rs, float eps, bool silu_gate, long n_rows, int H, int Dv) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);  // (t, h)
  const int lane = threadIdx.x & 63;
  if (row >= n_rows) return;
  const long t = row / H;
  const int h = (int)(row % H);
  const float* orow = o + row * Dv;
  float v[MAXV];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < MAXV; ++e) {
    const int i = e * 64 + lane;
    v[e] = i < Dv ? orow[i] : 0.f;
    ss = fmaf(v[e], v[e], ss);
  }
  const float r = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
#pragma unroll
  for (int e = 0; e < MAXV; ++e) {
    const int i = e * 64 + lane;
    if (i < Dv) {
      const float gv = ldf(gate, t * gate_rs + (long)h * Dv + i);
      const float sg = 1.0f / (1.0f + expf(-gv));
      const float act = silu_gate ? gv * sg : sg;
      const float wv = w[w_shared ? i : h * Dv + i];
      stf(out, row * Dv + i, v[e] * r * wv * act);
    }
  }
}

}  // namespace

void matrix_memory_scan(long kind, torch::Tensor out, torch::Tensor q,
                        torch::Tensor k, torch::Tensor v, torch::Tensor gate,
                        c10::optional<torch::Tensor> gate_bias,
                        c10::optional<torch::Tensor> head_rate,
                        c10::optional<torch::Tensor> beta, double q_scale,
                        double gate_param, torch::Tensor S,
                        c10::optional<torch::Tensor> n_state,
                        c10::optional<torch::Tensor> m_state,
                        torch::Tensor state_slots, torch::Tensor seq_lens,
                        c10::optional<torch::Tensor> query_starts,
                        c10::optional<torch::Tensor> query_lens, long lanes) {
  TORCH_CHECK(kind >= 0 && kind <= 2, "unknown recurrence");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && out.dim() == 3);
  const int T_ = v.size(0), H = v.size(1), Dv = v.size(2);
  const int G = k.size(1), D = k.size(2);
  TORCH_CHECK(q.size(0) == T_ && k.size(0) == T_ && q.size(1) == G &&
              q.size(2) == D && G >= 1 && H % G == 0);
  TORCH_CHECK(D <= 512, "key size above 512 is not supported");
  TORCH_CHECK(q.stride(2) == 1 && k.stride(2) == 1 && v.stride(2) == 1 &&
              q.stride(1) == D && k.stride(1) == D && v.stride(1) == Dv);
  TORCH_CHECK(q.scalar_type() == k.scalar_type() &&
              q.scalar_type() == v.scalar_type());
  TORCH_CHECK(out.scalar_type() == at::kFloat && out.is_contiguous() &&
              out.size(0) == T_ && out.size(1) == H && out.size(2) == Dv);
  TORCH_CHECK(S.scalar_type() == at::kFloat && S.is_contiguous() &&
              S.dim() == 4 && S.size(1) == H && S.size(2) == Dv &&
              S.size(3) == D, "state must be fp32 [slots, H, Dv, D]");
  TORCH_CHECK(gate.scalar_type() == at::kFloat && gate.dim() == 2 &&
              gate.stride(1) == 1 && gate.size(0) == T_);
  TORCH_CHECK(gate_bias.has_value() &&
              gate_bias->scalar_type() == at::kFloat &&
              gate_bias->is_contiguous());
  ScanArgs a{};
  if (kind == KIND_MLSTM) {
    TORCH_CHECK(gate.size(1) == 2 * H && gate_bias->numel() == 2 * H);
    TORCH_CHECK(n_state.has_value() && m_state.has_value());
    TORCH_CHECK(n_state->scalar_type() == at::kFloat &&
                n_state->is_contiguous() && n_state->dim() == 3 &&
                n_state->size(0) == S.size(0) && n_state->size(1) == H &&
                n_state->size(2) == D);
    TORCH_CHECK(m_state->scalar_type() == at::kFloat &&
                m_state->is_contiguous() && m_state->dim() == 2 &&
                m_state->size(0) == S.size(0) && m_state->size(1) == H);
    TORCH_CHECK(G == H);
    a.n_state = n_state->data_ptr<float>();
    a.m_state = m_state->data_ptr<float>();
  } else {
    TORCH_CHECK(gate.size(1) == (long)H * D && gate_bias->numel() == (long)H * D);
  }
  if (kind == KIND_DELTA) {
    TORCH_CHECK(head_rate.has_value() && beta.has_value());
    TORCH_CHECK(head_rate->scalar_type() == at::kFloat &&
                head_rate->is_contiguous() && head_rate->numel() == H);
    TORCH_CHECK(beta->scalar_type() == at::kFloat && beta->dim() == 2 &&
                beta->size(0) == T_ && beta->size(1) == H &&
                beta->stride(1) == 1);
    a.beta = beta->data_ptr<float>();
    a.beta_rs = beta->stride(0);
  }
  TORCH_CHECK(state_slots.scalar_type() == at::kLong &&
              state_slots.is_contiguous());
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  const int B = seq_lens.numel();
  TORCH_CHECK(state_slots.numel() == B);
  TORCH_CHECK(query_starts.has_value() == query_lens.has_value());
  if (query_starts.has_value()) {
    TORCH_CHECK(query_starts->scalar_type() == at::kInt &&
                query_lens->scalar_type() == at::kInt &&
                query_starts->numel() == B && query_lens->numel() == B &&
                query_starts->is_contiguous() && query_lens->is_contiguous());
    a.q_starts = query_starts->data_ptr<int>();
    a.q_lens = query_lens->data_ptr<int>();
  } else {
    TORCH_CHECK(T_ == B, "one token per sequence expected");
  }
  if (T_ == 0 || B == 0) return;
  a.out = out.data_ptr<float>();
  a.q = q.data_ptr(); a.k = k.data_ptr(); a.v = v.data_ptr();
  a.gate = gate.data_ptr<float>();
  a.gate_rs = gate.stride(0);
  a.gate_bias = gate_bias->data_ptr<float>();
  auto stream = at::hip::getCurrentHIPStream();
  torch::Tensor decay;
  if (kind != KIND_MLSTM) {
    decay = torch::empty({T_, (long)H * D}, S.options());
    const long n = (long)T_ * H * D;
    if (kind == KIND_GLA) {
      hipLaunchKernelGGL((decay_kernel<KIND_GLA>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, decay.data_ptr<float>(), a.gate,
                         a.gate_rs, a.gate_bias, (const float*)nullptr,
                         (float)gate_param, n, H * D, D);
    } else {
      hipLaunchKernelGGL((decay_kernel<KIND_DELTA>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, decay.data_ptr<float>(), a.gate,
                         a.gate_rs, a.gate_bias, head_rate->data_ptr<float>(),
                         0.f, n, H * D, D);
    }
    a.gate = decay.data_ptr<float>();
    a.gate_rs = (long)H * D;
  }
  a.S = S.data_ptr<float>();
  a.slots = state_slots.data_ptr<long>();
  a.seq_lens = seq_lens.data_ptr<int>();
  a.q_rs = q.stride(0); a.k_rs = k.stride(0); a.v_rs = v.stride(0);
  a.H = H; a.G = G; a.D = D; a.Dv = Dv;
  a.q_scale = (float)q_scale;
  a.gate_param = (float)gate_param;
  torch::Tensor n_new, m_new;
  if (kind == KIND_MLSTM) {
    n_new = torch::empty({B, H, D}, S.options());
    m_new = torch::empty({B, H}, S.options());
    a.n_new = n_new.data_ptr<float>();
    a.m_new = m_new.data_ptr<float>();
  }
  const bool bf16 = q.scalar_type() == at::kBFloat16;
  TORCH_CHECK(bf16 || q.scalar_type() == at::kFloat,
              "expected bf16 or fp32 q, k, v");
  if (kind == KIND_GLA) mm::launch_gla(a, B, (int)lanes, bf16, stream);
  else if (kind == KIND_DELTA) mm::launch_delta(a, B, (int)lanes, bf16, stream);
  else mm::launch_mlstm(a, B, (int)lanes, bf16, stream);
  if (kind == KIND_MLSTM) {
    hipLaunchKernelGGL(scatter_nm_kernel, dim3((H * D + 255) / 256, B),
                       dim3(256), 0, stream, n_state->data_ptr<float>(),
                       m_state->data_ptr<float>(), a.n_new, a.m_new, a.slots,
                       a.q_lens, H * D, H);
  }
}

void head_rmsnorm_gate(torch::Tensor out, torch::Tensor o, torch::Tensor w,
                       torch::Tensor gate, double eps, bool silu_gate) {
  TORCH_CHECK(o.scalar_type() == at::kFloat && o.is_contiguous() &&
              o.dim() == 3);
  const int T_ = o.size(0), H = o.size(1), Dv = o.size(2);
  TORCH_CHECK(Dv <= 64 * MAXV, "value size above 512 is not supported");
  TORCH_CHECK(out.is_contiguous() && out.numel() == (long)T_ * H * Dv);
  TORCH_CHECK(w.scalar_type() == at::kFloat && w.is_contiguous() &&
              (w.numel() == Dv || w.numel() == (long)H * Dv));
  TORCH_CHECK(gate.dim() == 2 && gate.size(0) == T_ &&
              gate.size(1) == (long)H * Dv && gate.stride(1) == 1);
  const bool g_f32 = gate.scalar_type() == at::kFloat;
  TORCH_CHECK(g_f32 || gate.scalar_type() == out.scalar_type());
  const long n_rows = (long)T_ * H;
  if (n_rows == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
#define LAUNCH(TT, TG)                                                        \
  hipLaunchKernelGGL((head_norm_gate_kernel<TT, TG>),                         \
                     dim3((n_rows + 3) / 4), dim3(256), 0, stream,            \
                     (TT*)out.data_ptr(), o.data_ptr<float>(),                \
                     w.data_ptr<float>(), (int)(w.numel() == Dv),             \
                     (const TG*)gate.data_ptr(), (long)gate.stride(0),        \
                     (float)eps, silu_gate, n_rows, H, Dv)
  LATENT_DISPATCH_T(out, {
    if (g_f32) LAUNCH(T, float); else LAUNCH(T, T);
  });
#undef LAUNCH
}
