// Matrix-memory recurrence kernel (gfx950), shared by the per-recurrence
// translation units; see matrix_memory.hip for the algorithm.
#pragma once

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace mm {

constexpr int KIND_GLA = 0, KIND_DELTA = 1, KIND_MLSTM = 2;
constexpr int CH = 8;      // tokens staged together
constexpr int WAVES = 4;   // waves of a workgroup; they share the staging
constexpr int TPW = CH / WAVES;

struct ScanArgs {
  float* out;            // [T, H, Dv]
  const void* q;         // [T, G, D] (row stride q_rs)
  const void* k;
  const void* v;         // [T, H, Dv]
  const float* gate;     // gla / delta: decays [T, H*D], already evaluated;
                         // mLSTM: gate pre-activations [T, 2H]
  const float* gate_bias;
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

template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(
      0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}

// sum over the NSUB adjacent lanes that share a column (data-parallel
// primitives inside a row of 16 lanes; no LDS round trip)
template <int NSUB>
__device__ __forceinline__ float sub_sum(float v) {
  if constexpr (NSUB >= 2) v += dpp_mov<0xB1>(v);    // quad_perm [1,0,3,2]
  if constexpr (NSUB >= 4) v += dpp_mov<0x4E>(v);    // quad_perm [2,3,0,1]
  if constexpr (NSUB >= 8) v += dpp_mov<0x141>(v);   // row_half_mirror
  if constexpr (NSUB >= 16) v += dpp_mov<0x140>(v);  // row_mirror
  return v;
}

// sum over the wave: rows of 16 lanes by DPP, the four rows by lane reads
__device__ __forceinline__ float wave_total(float v) {
  v = sub_sum<16>(v);
  const int i = __float_as_int(v);
  return __int_as_float(__builtin_amdgcn_readlane(i, 0)) +
         __int_as_float(__builtin_amdgcn_readlane(i, 16)) +
         __int_as_float(__builtin_amdgcn_readlane(i, 32)) +
         __int_as_float(__builtin_amdgcn_readlane(i, 48));
}

template <int KIND, typename TI, int NSUB, int RPT>
__global__ __launch_bounds__(256) void scan_kernel(const ScanArgs a) {
  constexpr int COLS = 64 / NSUB;                // columns per wave
  constexpr int ROWS = NSUB * RPT;               // key rows covered
  constexpr int EPL = ROWS / 64 > 0 ? ROWS / 64 : 1;  // staged elems per lane
  constexpr int R4 = RPT / 4;
  __shared__ __attribute__((aligned(16))) float kbuf[CH][ROWS];
  __shared__ __attribute__((aligned(16))) float qbuf[CH][ROWS];
  __shared__ __attribute__((aligned(16))) float gbuf[KIND == KIND_MLSTM ? 1 : CH][ROWS];
  __shared__ float sc[CH][4];   // k.q | write scale (beta, e^(i-m)) | e^(f+m-m') | e^(-m')

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane / NSUB, sub = lane % NSUB;
  const int h = blockIdx.y, b = blockIdx.z;
  const int j = (blockIdx.x * WAVES + wave) * COLS + col;
  const int H = a.H, D = a.D, Dv = a.Dv;
  const int g = h / (H / a.G);
  const bool col_ok = j < Dv;
  const int jc = col_ok ? j : Dv - 1;            // clamped: loads stay in bounds

  const int n_tok = a.q_lens ? a.q_lens[b] : 1;
  if (n_tok <= 0) return;                        // the whole workgroup
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
  for (int i4 = 0; i4 < R4; ++i4) {
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

  // ---- raw inputs of the next chunk, in registers. Wave w stages the
  // tokens c = w, w + WAVES, ... of a chunk for the whole workgroup; every
  // lane keeps its own column's v; wave 0 evaluates the mLSTM gates, lane
  // c those of token c.
  float rk[TPW][EPL], rq[TPW][EPL], rg[KIND == KIND_MLSTM ? 1 : TPW][EPL];
  float rb[TPW];
  float rv[CH];
  float rgi = 0.f, rgf = 0.f;
  const TI* qp = (const TI*)a.q;
  const TI* kp = (const TI*)a.k;
  const TI* vp = (const TI*)a.v;

  auto load_chunk = [&](int t0) {
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
      const int c = i * WAVES + wave;
      if (t0 + c < n_tok) {                      // wave-uniform
        const long row = s0 + t0 + c;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          const int r = e * 64 + lane;
          const bool ok = r < D && r < ROWS;
          const int rc = ok ? r : 0;
          rk[i][e] = ok ? ldf(kp, row * a.k_rs + (long)g * D + rc) : 0.f;
          rq[i][e] = ok ? ldf(qp, row * a.q_rs + (long)g * D + rc) : 0.f;
          if constexpr (KIND != KIND_MLSTM)
            rg[i][e] = ok ? a.gate[row * a.gate_rs + (long)h * D + rc] : 1.f;
        }
        if constexpr (KIND == KIND_DELTA) rb[i] = a.beta[row * a.beta_rs + h];
      }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c)
      if (t0 + c < n_tok)
        rv[c] = ldf(vp, (long)(s0 + t0 + c) * a.v_rs + (long)h * Dv + jc);
    if constexpr (KIND == KIND_MLSTM) {
      if (wave == 0 && lane < CH && t0 + lane < n_tok) {
        const long row = s0 + t0 + lane;
        rgi = a.gate[row * a.gate_rs + h];
        rgf = a.gate[row * a.gate_rs + H + h];
      }
    }
  };

  float bias_i = 0.f, bias_f = 0.f;
  if constexpr (KIND == KIND_MLSTM) {
    bias_i = a.gate_bias[h];
    bias_f = a.gate_bias[H + h];
  }

  load_chunk(0);
  for (int t0 = 0; t0 < n_tok; t0 += CH) {
    __syncthreads();                 // previous chunk's LDS reads are done
    // ---- stage this chunk: vectors and per-token numbers to LDS
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
      const int c = i * WAVES + wave;
      if (t0 + c < n_tok) {
        float kq = 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
          const int r = e * 64 + lane;
          const float kk = rk[i][e];
          const float qq = rq[i][e] * a.q_scale;
          kq = fmaf(kk, qq, kq);
          if (r < ROWS) {
            kbuf[c][r] = kk;
            qbuf[c][r] = qq;
            if constexpr (KIND != KIND_MLSTM) gbuf[c][r] = rg[i][e];
          }
        }
        kq = wave_total(kq);
        if (lane == 0) {
          sc[c][0] = kq;
          if constexpr (KIND == KIND_DELTA)
            sc[c][1] = 1.0f / (1.0f + expf(-rb[i]));
        }
      }
    }
    if constexpr (KIND == KIND_MLSTM) {
      if (wave == 0) {
        const float cap = a.gate_param;
        const float ig = cap * tanhf((rgi + bias_i) / cap);
        const float fg = log_sigmoid(cap * tanhf((rgf + bias_f) / cap));
        float m_before = 0.f, m_after = 0.f;     // of this lane's token
#pragma unroll
        for (int c = 0; c < CH; ++c) {
          if (t0 + c < n_tok) {
            const float fc = __shfl(fg, c, WAVE), ic = __shfl(ig, c, WAVE);
            const float mn = fmaxf(fc + m_run, ic);
            if (lane == c) { m_before = m_run; m_after = mn; }
            m_run = mn;
          }
        }
        if (lane < CH && t0 + lane < n_tok) {
          sc[lane][1] = expf(ig - m_after);
          sc[lane][2] = expf(fg + m_before - m_after);
          sc[lane][3] = expf(-m_after);
        }
      }
    }
    __syncthreads();
    float cv[CH], cu[CH], ckq[CH], cdf[CH], cei[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      cv[c] = rv[c];
      ckq[c] = sc[c][0];
      cu[c] = KIND == KIND_GLA ? 1.f : sc[c][1];
      cdf[c] = KIND == KIND_MLSTM ? sc[c][2] : 1.f;
      cei[c] = KIND == KIND_MLSTM ? sc[c][3] : 0.f;
    }
    if (t0 + CH < n_tok) load_chunk(t0 + CH);    // lands during the compute

    // ---- the recurrence, token by token
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      if (t0 + c < n_tok) {
        // four independent partial sums per dot product: the chains of
        // dependent multiply-adds are RPT / 4 long
        float a1[4] = {0.f, 0.f, 0.f, 0.f}, a2[4] = {0.f, 0.f, 0.f, 0.f};
        float nq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i4 = 0; i4 < R4; ++i4) {
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
            if constexpr (KIND == KIND_DELTA) a1[e] = fmaf(s, kk[e], a1[e]);
            a2[e] = fmaf(s, qq[e], a2[e]);
            if constexpr (KIND == KIND_MLSTM) {
              const float nn = fmaf(nst[i4 * 4 + e], cdf[c], cu[c] * kk[e]);
              nst[i4 * 4 + e] = nn;
              nq[e] = fmaf(nn, qq[e], nq[e]);
            }
          }
        }
        const float a2s = sub_sum<NSUB>((a2[0] + a2[1]) + (a2[2] + a2[3]));
        float u;
        if constexpr (KIND == KIND_DELTA) {
          const float a1s = sub_sum<NSUB>((a1[0] + a1[1]) + (a1[2] + a1[3]));
          u = cu[c] * (cv[c] - a1s);
        } else if constexpr (KIND == KIND_MLSTM) {
          u = cu[c] * cv[c];
        } else {
          u = cv[c];
        }
#pragma unroll
        for (int i4 = 0; i4 < R4; ++i4) {
          const int r = (i4 * NSUB + sub) * 4;
          const float4 k4 = *reinterpret_cast<const float4*>(&kbuf[c][r]);
          S[i4 * 4] = fmaf(k4.x, u, S[i4 * 4]);
          S[i4 * 4 + 1] = fmaf(k4.y, u, S[i4 * 4 + 1]);
          S[i4 * 4 + 2] = fmaf(k4.z, u, S[i4 * 4 + 2]);
          S[i4 * 4 + 3] = fmaf(k4.w, u, S[i4 * 4 + 3]);
        }
        float o = fmaf(u, ckq[c], a2s);
        if constexpr (KIND == KIND_MLSTM) {
          const float nqs = sub_sum<NSUB>((nq[0] + nq[1]) + (nq[2] + nq[3]));
          o = o / (fmaxf(fabsf(nqs), cei[c]) + 1e-6f);
        }
        if (sub == 0 && col_ok)
          a.out[((long)(s0 + t0 + c) * H + h) * Dv + j] = o;
      }
    }
  }

  // ---- state back to the pool
  if (col_ok) {
#pragma unroll
    for (int i4 = 0; i4 < R4; ++i4) {
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
    if (blockIdx.x == 0 && wave == 0 && col == 0) {
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

// The lanes that share a column (NSUB) and the rows per lane (RPT) are
// chosen per launch: at least enough lanes to hold D rows at 32 per lane,
// and more (fewer rows per lane, more waves) while the launch would leave
// the chip's SIMDs short of waves. `lanes` > 0 forces NSUB (A/B runs).
template <int KIND, typename TI>
void launch_scan(const ScanArgs& a, int B, int lanes, hipStream_t stream) {
  const int D = a.D;
  int lo = 1;
  while (lo * 32 < D) lo <<= 1;                  // fewest lanes per column
  int ns = lo;
  if (lanes > 0) {
    ns = lanes < lo ? lo : (lanes > 16 ? 16 : lanes);
  } else {
    const long cols = (long)B * a.H * a.Dv;
    while (ns < 16 && ns < lo * 4 && cols * ns / 64 < 4096) ns <<= 1;
  }
#define SCAN_CASE(NS, RP)                                                     \
  hipLaunchKernelGGL((scan_kernel<KIND, TI, NS, RP>),                         \
                     dim3((a.Dv + WAVES * (64 / NS) - 1) / (WAVES * (64 / NS)),\
                          a.H, B),                                            \
                     dim3(64 * WAVES), 0, stream, a)
  if (D <= 32) {
    if (ns >= 4) SCAN_CASE(4, 8); else if (ns == 2) SCAN_CASE(2, 16);
    else SCAN_CASE(1, 32);
  } else if (D <= 64) {
    if (ns >= 8) SCAN_CASE(8, 8); else if (ns == 4) SCAN_CASE(4, 16);
    else SCAN_CASE(2, 32);
  } else if (D <= 128) {
    if (ns >= 16) SCAN_CASE(16, 8); else if (ns == 8) SCAN_CASE(8, 16);
    else SCAN_CASE(4, 32);
  } else if (D <= 256) {
    if (ns >= 16) SCAN_CASE(16, 16); else SCAN_CASE(8, 32);
  } else {
    SCAN_CASE(16, 32);
  }
#undef SCAN_CASE
}

}  // namespace mm
