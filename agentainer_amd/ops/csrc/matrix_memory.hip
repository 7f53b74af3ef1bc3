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
// so the work is cut over (sequence, head, block of value columns): one
// wave owns 64 / NSUB columns, NSUB adjacent lanes share a column and split
// its key rows (32 per lane, held in registers for the whole portion), the
// two dot products are reduced over those lanes by shuffles. The pool keeps
// S transposed ([slots, H, Dv, D]: a column's rows are contiguous) and the
// row -> lane mapping interleaves the sub-lanes by float4, so state loads
// and stores are 16-byte accesses that are contiguous across the NSUB lanes
// of a column, and the staged k / q / g vectors are read from LDS as
// conflict-free float4.
//
// Tokens are processed strictly in order, eight at a time: the raw inputs
// of the NEXT eight tokens are loaded into registers while the current
// eight are computed; decays and gates (sigmoid, softplus, exp, tanh, the
// running maximum) are evaluated in fp32 when a chunk is staged. Prompt
// portions and single decoded tokens run the same code, so a position's
// result does not depend on where the prompt was cut. A sequence whose
// first row sits at position 0 starts from zero state; the final state is
// written back at the end.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

constexpr int KIND_GLA = 0, KIND_DELTA = 1, KIND_MLSTM = 2;
constexpr int RPT = 32;   // key rows per lane
constexpr int CH = 8;     // tokens staged together

struct ScanArgs {
  float* out;            // [T, H, Dv]
  const void* q;         // [T, G, D] (row stride q_rs)
  const void* k;
  const void* v;         // [T, H, Dv]
  const float* gate;     // kind-specific, row stride gate_rs
  const float* gate_bias;
  const float* head_rate;
  const float* beta;     // [T, H], row stride beta_rs
  float* S;              // [slots, H, Dv, D]
  const float* n_state;  // [slots, H, D]   (read at the start)
  const float* m_state;  // [slots, H]
  float* n_new;          // [B, H, D], [B, H]: the step's final normalizer
  float* m_new;          //   and maximum, scattered to the slots afterwards
  const long* slots;
  const int* seq_lens;
  const int* q_starts;
  const int* q_lens;
  long q_rs, k_rs, v_rs, gate_rs, beta_rs;
  int H, G, D, Dv;
  float q_scale, gate_param;
};

__device__ __forceinline__ float log_sigmoid(float x) {
  return fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
}
__device__ __forceinline__ float soft_plus(float x) {
  return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
}

template <int NSUB>
__device__ __forceinline__ float sub_sum(float v) {
#pragma unroll
  for (int off = 1; off < NSUB; off <<= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}

template <int KIND, typename TI, int NSUB>
__global__ __launch_bounds__(64) void scan_kernel(const ScanArgs a) {
  constexpr int COLS = 64 / NSUB;
  constexpr int ROWS = NSUB * RPT;               // key rows covered
  constexpr int EPL = ROWS / 64 > 0 ? ROWS / 64 : 1;  // staged elems per lane
  __shared__ __attribute__((aligned(16))) float kbuf[CH][ROWS];
  __shared__ __attribute__((aligned(16))) float qbuf[CH][ROWS];
  __shared__ __attribute__((aligned(16))) float gbuf[KIND == KIND_MLSTM ? 1 : CH][ROWS];

  const int lane = threadIdx.x;
  const int col = lane / NSUB, sub = lane % NSUB;
  const int h = blockIdx.y, b = blockIdx.z;
  const int j = blockIdx.x * COLS + col;
  const int H = a.H, D = a.D, Dv = a.Dv;
  const int g = h / (H / a.G);
  const bool col_ok = j < Dv;
  const int jc = col_ok ? j : Dv - 1;            // clamped: loads stay in bounds

  const int n_tok = a.q_lens ? a.q_lens[b] : 1;
  if (n_tok <= 0) return;
  const int s0 = a.q_starts ? a.q_starts[b] : b;
  const bool fresh = a.seq_lens[b] - n_tok <= 0;
  const long slot = a.slots[b];

  // ---- state into registers: row(i) = ((i / 4) * NSUB + sub) * 4 + i % 4
  float S[RPT];
  float nst[KIND == KIND_MLSTM ? RPT : 1];
  float m_run = 0.f;
  float* Sp = a.S + (((long)slot * H + h) * Dv + jc) * D;
  const bool vec4 = (D & 3) == 0;
#pragma unroll
  for (int i4 = 0; i4 < RPT / 4; ++i4) {
    const int r = (i4 * NSUB + sub) * 4;
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    if (!fresh) {
      if (vec4) {
        if (r < D) t = *reinterpret_cast<const float4*>(Sp + r);
      } else {
        if (r < D) t.x = Sp[r];
        if (r + 1 < D) t.y = Sp[r + 1];
        if (r + 2 < D) t.z = Sp[r + 2];
        if (r + 3 < D) t.w = Sp[r + 3];
      }
    }
    S[i4 * 4] = t.x; S[i4 * 4 + 1] = t.y; S[i4 * 4 + 2] = t.z; S[i4 * 4 + 3] = t.w;
  }
  if constexpr (KIND == KIND_MLSTM) {
    const float* np = a.n_state + ((long)slot * H + h) * D;
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int r = ((i >> 2) * NSUB + sub) * 4 + (i & 3);
      nst[i] = (!fresh && r < D) ? np[r] : 0.f;
    }
    if (!fresh) m_run = a.m_state[(long)slot * H + h];
  }

  // ---- raw inputs of the next chunk, in registers
  float rk[CH][EPL], rq[CH][EPL], rg[KIND == KIND_MLSTM ? 1 : CH][EPL];
  float rv[CH], rs1[CH], rs2[CH];   // v; beta | log-input gate; forget gate
  const TI* qp = (const TI*)a.q;
  const TI* kp = (const TI*)a.k;
  const TI* vp = (const TI*)a.v;

  auto load_chunk = [&](int t0) {
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const bool tok_ok = t0 + c < n_tok;
      const long row = s0 + (tok_ok ? t0 + c : n_tok - 1);
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int r = e * 64 + lane;
        const bool ok = r < D && r < ROWS;
        const int rc = ok ? r : 0;
        rk[c][e] = ok ? ldf(kp, row * a.k_rs + (long)g * D + rc) : 0.f;
        rq[c][e] = ok ? ldf(qp, row * a.q_rs + (long)g * D + rc) : 0.f;
        if constexpr (KIND != KIND_MLSTM)
          rg[c][e] = ok ? a.gate[row * a.gate_rs + (long)h * D + rc] : 0.f;
      }
      rv[c] = ldf(vp, row * a.v_rs + (long)h * Dv + jc);
      if constexpr (KIND == KIND_DELTA) rs1[c] = a.beta[row * a.beta_rs + h];
      if constexpr (KIND == KIND_MLSTM) {
        rs1[c] = a.gate[row * a.gate_rs + h];
        rs2[c] = a.gate[row * a.gate_rs + H + h];
      }
    }
  };

  // per-row constants of the staging transform
  float gb[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    const int r = e * 64 + lane;
    gb[e] = (KIND != KIND_MLSTM && r < D && r < ROWS)
                ? a.gate_bias[(long)h * D + r] : 0.f;
  }
  float rate = 0.f, bias_i = 0.f, bias_f = 0.f;
  if constexpr (KIND == KIND_DELTA) rate = expf(a.head_rate[h]);
  if constexpr (KIND == KIND_MLSTM) {
    bias_i = a.gate_bias[h];
    bias_f = a.gate_bias[H + h];
  }

  load_chunk(0);
  for (int t0 = 0; t0 < n_tok; t0 += CH) {
    // ---- stage this chunk: transforms in fp32, vectors to LDS
    float cv[CH], cu[CH], ckq[CH], cdf[CH], cei[CH];
    __syncthreads();                 // previous chunk's LDS reads are done
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      float kq = 0.f;
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const int r = e * 64 + lane;
        const float kk = rk[c][e];
        const float qq = rq[c][e] * a.q_scale;
        kq = fmaf(kk, qq, kq);
        if (r < ROWS) {
          kbuf[c][r] = kk;
          qbuf[c][r] = qq;
          if constexpr (KIND == KIND_GLA)
            gbuf[c][r] = r < D ? expf(log_sigmoid(rg[c][e] + gb[e]) *
                                      a.gate_param) : 1.f;
          if constexpr (KIND == KIND_DELTA)
            gbuf[c][r] = r < D ? expf(-rate * soft_plus(rg[c][e] + gb[e]))
                               : 1.f;
        }
      }
      ckq[c] = wave_sum(kq);
      cv[c] = rv[c];
      cu[c] = 1.f; cdf[c] = 1.f; cei[c] = 0.f;
      if constexpr (KIND == KIND_DELTA)
        cu[c] = 1.0f / (1.0f + expf(-rs1[c]));
      if constexpr (KIND == KIND_MLSTM) {
        if (t0 + c < n_tok) {
          const float cap = a.gate_param;
          const float ig = cap * tanhf((rs1[c] + bias_i) / cap);
          const float fg = log_sigmoid(cap * tanhf((rs2[c] + bias_f) / cap));
          const float mn = fmaxf(fg + m_run, ig);
          cdf[c] = expf(fg + m_run - mn);
          cu[c] = expf(ig - mn);
          cei[c] = expf(-mn);
          m_run = mn;
        }
      }
    }
    __syncthreads();
    if (t0 + CH < n_tok) load_chunk(t0 + CH);    // lands during the compute

    // ---- the recurrence, token by token
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      if (t0 + c < n_tok) {
        float a1 = 0.f, a2 = 0.f, nq = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < RPT / 4; ++i4) {
          const int r = (i4 * NSUB + sub) * 4;
          const float4 k4 = *reinterpret_cast<const float4*>(&kbuf[c][r]);
          const float4 q4 = *reinterpret_cast<const float4*>(&qbuf[c][r]);
          float4 g4;
          if constexpr (KIND == KIND_MLSTM) {
            g4 = make_float4(cdf[c], cdf[c], cdf[c], cdf[c]);
          } else {
            g4 = *reinterpret_cast<const float4*>(&gbuf[c][r]);
          }
          const float kk[4] = {k4.x, k4.y, k4.z, k4.w};
          const float qq[4] = {q4.x, q4.y, q4.z, q4.w};
          const float gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float s = S[i4 * 4 + e] * gg[e];
            S[i4 * 4 + e] = s;
            if constexpr (KIND == KIND_DELTA) a1 = fmaf(s, kk[e], a1);
            a2 = fmaf(s, qq[e], a2);
            if constexpr (KIND == KIND_MLSTM) {
              const float nn = fmaf(nst[i4 * 4 + e], cdf[c], cu[c] * kk[e]);
              nst[i4 * 4 + e] = nn;
              nq = fmaf(nn, qq[e], nq);
            }
          }
        }
        a2 = sub_sum<NSUB>(a2);
        float u;
        if constexpr (KIND == KIND_DELTA) {
          a1 = sub_sum<NSUB>(a1);
          u = cu[c] * (cv[c] - a1);
        } else if constexpr (KIND == KIND_MLSTM) {
          u = cu[c] * cv[c];
        } else {
          u = cv[c];
        }
#pragma unroll
        for (int i4 = 0; i4 < RPT / 4; ++i4) {
          const int r = (i4 * NSUB + sub) * 4;
          const float4 k4 = *reinterpret_cast<const float4*>(&kbuf[c][r]);
          S[i4 * 4] = fmaf(k4.x, u, S[i4 * 4]);
          S[i4 * 4 + 1] = fmaf(k4.y, u, S[i4 * 4 + 1]);
          S[i4 * 4 + 2] = fmaf(k4.z, u, S[i4 * 4 + 2]);
          S[i4 * 4 + 3] = fmaf(k4.w, u, S[i4 * 4 + 3]);
        }
        float o = fmaf(u, ckq[c], a2);
        if constexpr (KIND == KIND_MLSTM) {
          nq = sub_sum<NSUB>(nq);
          o = o / (fmaxf(fabsf(nq), cei[c]) + 1e-6f);
        }
        if (sub == 0 && col_ok)
          a.out[((long)(s0 + t0 + c) * H + h) * Dv + j] = o;
      }
    }
  }

  // ---- state back to the pool
  if (col_ok) {
#pragma unroll
    for (int i4 = 0; i4 < RPT / 4; ++i4) {
      const int r = (i4 * NSUB + sub) * 4;
      if (vec4) {
        if (r < D)
          *reinterpret_cast<float4*>(Sp + r) = make_float4(
              S[i4 * 4], S[i4 * 4 + 1], S[i4 * 4 + 2], S[i4 * 4 + 3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (r + e < D) Sp[r + e] = S[i4 * 4 + e];
      }
    }
  }
  if constexpr (KIND == KIND_MLSTM) {
    // every column block of this head read n and m at its start, and
    // blocks start at different times: the new values go to a per-row
    // buffer and reach the slot in a second launch
    if (blockIdx.x == 0 && col == 0) {
      float* np = a.n_new + ((long)b * H + h) * D;
#pragma unroll
      for (int i = 0; i < RPT; ++i) {
        const int r = ((i >> 2) * NSUB + sub) * 4 + (i & 3);
        if (r < D) np[r] = nst[i];
      }
      if (sub == 0) a.m_new[(long)b * H + h] = m_run;
    }
  }
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

template <int KIND, typename TI>
void launch_scan(const ScanArgs& a, int B, hipStream_t stream) {
  const int D = a.D;
#define SCAN_CASE(NS)                                                         \
  hipLaunchKernelGGL((scan_kernel<KIND, TI, NS>),                             \
                     dim3((a.Dv + 64 / NS - 1) / (64 / NS), a.H, B),          \
                     dim3(64), 0, stream, a)
  if (D <= 32) SCAN_CASE(1);
  else if (D <= 64) SCAN_CASE(2);
  else if (D <= 128) SCAN_CASE(4);
  else if (D <= 256) SCAN_CASE(8);
  else SCAN_CASE(16);
#undef SCAN_CASE
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
                        c10::optional<torch::Tensor> query_lens) {
  TORCH_CHECK(kind >= 0 && kind <= 2, "unknown recurrence");
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3 && out.dim() == 3);
  const int T_ = v.size(0), H = v.size(1), Dv = v.size(2);
  const int G = k.size(1), D = k.size(2);
  TORCH_CHECK(q.size(0) == T_ && k.size(0) == T_ && q.size(1) == G &&
              q.size(2) == D && G >= 1 && H % G == 0);
  TORCH_CHECK(D <= 16 * RPT, "key size above 512 is not supported");
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
    a.head_rate = head_rate->data_ptr<float>();
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
  a.gate_bias = gate_bias->data_ptr<float>();
  a.S = S.data_ptr<float>();
  a.slots = state_slots.data_ptr<long>();
  a.seq_lens = seq_lens.data_ptr<int>();
  a.q_rs = q.stride(0); a.k_rs = k.stride(0); a.v_rs = v.stride(0);
  a.gate_rs = gate.stride(0);
  a.H = H; a.G = G; a.D = D; a.Dv = Dv;
  a.q_scale = (float)q_scale;
  a.gate_param = (float)gate_param;
  auto stream = at::hip::getCurrentHIPStream();
  torch::Tensor n_new, m_new;
  if (kind == KIND_MLSTM) {
    n_new = torch::empty({B, H, D}, S.options());
    m_new = torch::empty({B, H}, S.options());
    a.n_new = n_new.data_ptr<float>();
    a.m_new = m_new.data_ptr<float>();
  }
  LATENT_DISPATCH_T(q, {
    if (kind == KIND_GLA) launch_scan<KIND_GLA, T>(a, B, stream);
    else if (kind == KIND_DELTA) launch_scan<KIND_DELTA, T>(a, B, stream);
    else launch_scan<KIND_MLSTM, T>(a, B, stream);
  });
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
