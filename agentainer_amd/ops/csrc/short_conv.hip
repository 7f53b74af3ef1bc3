// Depthwise short causal convolution over time with a per-sequence tail
// (gfx950).
//
//   y[t, c] = sum_j w[j, c] * u[t - taps + 1 + j, c]      (w is [taps, C])
//
// over a step's token rows (variable-length portions of several sequences,
// or one new token per sequence). Inputs before the step's first row come
// from tail[slot] (the last taps-1 inputs of the sequence, fp32), inputs
// before position 0 are zero. Fused behind it, per option: SiLU, and for
// the first `norm_channels` channels (cut into heads of `head_dim`) the
// unit-vector scaling y / sqrt(sum(y^2) + eps) with an extra factor on the
// first `lead_channels`.
//
// Kernel 1: a wave (or an aligned group of 8..64 of its lanes) per (token,
// chunk of channels) — a chunk is one head where heads are normalized —
// four consecutive channels per lane where sizes and alignment allow, so
// loads and stores are 8- or 16-byte accesses that are coalesced along the
// channel axis and the head's sum is a reduction over the group's lanes.
// It only READS the tail. Kernel 2 (one thread per (sequence,
// channel)) then rewrites the tail from the step's last inputs, shifting
// the old tail when the portion is shorter than taps-1.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

constexpr int MAX_TAPS = 8;
constexpr int MAXV = 8;   // channels per lane: chunks of up to 512 channels

// sequence of token row t: the last b with starts[b] <= t
__device__ __forceinline__ int find_seq(const int* starts, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (starts[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_kernel(
    TO* __restrict__ out, long out_rs, const TI* __restrict__ u, long u_rs,
    const float* __restrict__ w, const float* __restrict__ tail,
    const long* __restrict__ slots, const int* __restrict__ seq_lens,
    const int* __restrict__ q_starts, const int* __restrict__ q_lens, int B,
    int C, int taps, int cs, int n_chunks, int nyb, bool silu,
    int norm_channels, int lead_channels, float lead_scale, float l2_eps) {
  // consecutive workgroups walk along a token's channels (contiguous
  // memory), not along tokens at one channel offset (a power-of-two row
  // stride would send them all to the same memory channels)
  const int t = blockIdx.x / nyb;
  const int chunk = (blockIdx.x % nyb) * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (chunk >= n_chunks) return;
  int b, off, n;
  if (q_starts) {
    b = find_seq(q_starts, B, t);
    off = t - q_starts[b];
    n = q_lens[b];
  } else {
    b = t; off = 0; n = 1;
  }
  const int pos0 = seq_lens[b] - n;          // position of the portion's row 0
  const long slot = slots[b];
  const float* tl = tail + slot * (long)(taps - 1) * C;
  const int c0 = chunk * cs;
  float yv[MAXV];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < MAXV; ++e) {
    const int c = c0 + e * 64 + lane;
    yv[e] = 0.f;
    if (e * 64 + lane < cs && c < C) {
      float acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int src = off - (taps - 1) + j;   // row within the portion
        float uv = 0.f;
        if (src >= 0) {
          uv = ldf(u, (long)(t - off + src) * u_rs + c);
        } else if (pos0 + src >= 0) {
          uv = tl[(long)(taps - 1 + src) * C + c];
        }
        acc = fmaf(w[(long)j * C + c], uv, acc);
      }
      if (silu) acc = acc / (1.0f + expf(-acc));
      yv[e] = acc;
      ss = fmaf(acc, acc, ss);
    }
  }
  float mul = 1.f;
  if (c0 < norm_channels) {
    ss = wave_sum(ss);
    mul = 1.0f / sqrtf(ss + l2_eps);
    if (c0 < lead_channels) mul *= lead_scale;
  }
#pragma unroll
  for (int e = 0; e < MAXV; ++e) {
    const int c = c0 + e * 64 + lane;
    if (e * 64 + lane < cs && c < C) stf(out, (long)t * out_rs + c, yv[e] * mul);
  }
}

// Four consecutive channels per lane (8- or 16-byte loads and stores);
// LPH lanes cover one chunk, 64 / LPH chunks share a wave, and a head's sum
// is reduced over its LPH lanes only. Needs cs, C and the row strides to be
// multiples of 4 and cs <= 256.
template <typename TI, typename TO, int LPH>
__global__ __launch_bounds__(256) void short_conv_vec_kernel(
    TO* __restrict__ out, long out_rs, const TI* __restrict__ u, long u_rs,
    const float* __restrict__ w, const float* __restrict__ tail,
    const long* __restrict__ slots, const int* __restrict__ seq_lens,
    const int* __restrict__ q_starts, const int* __restrict__ q_lens, int B,
    int C, int taps, int cs, int n_chunks, int nyb, bool silu,
    int norm_channels, int lead_channels, float lead_scale, float l2_eps) {
  constexpr int CPW = 64 / LPH;
  const int t = blockIdx.x / nyb;
  const int lane = threadIdx.x & 63;
  const int chunk = ((blockIdx.x % nyb) * 4 + (threadIdx.x >> 6)) * CPW +
                    lane / LPH;
  const int li = lane % LPH;
  int b, off, n;
  if (q_starts) {
    b = find_seq(q_starts, B, t);
    off = t - q_starts[b];
    n = q_lens[b];
  } else {
    b = t; off = 0; n = 1;
  }
  const int pos0 = seq_lens[b] - n;
  const float* tl = tail + slots[b] * (long)(taps - 1) * C;
  const int c0 = chunk * cs;
  const int c = c0 + li * 4;
  const bool active = chunk < n_chunks && li * 4 < cs && c < C;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (active) {
    for (int j = 0; j < taps; ++j) {
      const int src = off - (taps - 1) + j;
      float uv[4] = {0.f, 0.f, 0.f, 0.f};
      if (src >= 0) {
        ld4(u, (long)(t - off + src) * u_rs + c, uv);
      } else if (pos0 + src >= 0) {
        ld4(tl, (long)(taps - 1 + src) * C + c, uv);
      }
      float wv[4];
      ld4(w, (long)j * C + c, wv);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = fmaf(wv[e], uv[e], acc[e]);
    }
    if (silu) {
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
    }
  }
  float mul = 1.f;
  if (norm_channels > 0) {           // uniform: the shuffles need every lane
    float ss = acc[0] * acc[0] + acc[1] * acc[1] + acc[2] * acc[2] +
               acc[3] * acc[3];
#pragma unroll
    for (int o = 1; o < LPH; o <<= 1) ss += __shfl_xor(ss, o, WAVE);
    if (c0 < norm_channels) {
      mul = 1.0f / sqrtf(ss + l2_eps);
      if (c0 < lead_channels) mul *= lead_scale;
    }
  }
  if (active) {
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] *= mul;
    st4(out, (long)t * out_rs + c, acc);
  }
}

template <typename TI>
__global__ __launch_bounds__(256) void conv_tail_kernel(
    float* __restrict__ tail, const TI* __restrict__ u, long u_rs,
    const long* __restrict__ slots, const int* __restrict__ seq_lens,
    const int* __restrict__ q_starts, const int* __restrict__ q_lens, int C,
    int taps) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int n = q_lens ? q_lens[b] : 1;
  if (n <= 0) return;
  const int s0 = q_starts ? q_starts[b] : b;
  const int pos0 = seq_lens[b] - n;
  float* tl = tail + slots[b] * (long)(taps - 1) * C;
  // ascending i: an old entry is read (at i + n > i) before it is rewritten
  for (int i = 0; i < taps - 1; ++i) {
    const int src = n - (taps - 1) + i;
    float v = 0.f;
    if (src >= 0) {
      v = ldf(u, (long)(s0 + src) * u_rs + c);
    } else if (pos0 + src >= 0) {
      v = tl[(long)(i + n) * C + c];
    }
    tl[(long)i * C + c] = v;
  }
}

}  // namespace

void short_conv_state(torch::Tensor out, torch::Tensor u, torch::Tensor w,
                      torch::Tensor tail, torch::Tensor state_slots,
                      torch::Tensor seq_lens,
                      c10::optional<torch::Tensor> query_starts,
                      c10::optional<torch::Tensor> query_lens, bool silu,
                      long norm_channels, long head_dim, long lead_channels,
                      double lead_scale, double l2_eps) {
  TORCH_CHECK(u.dim() == 2 && u.stride(1) == 1 && out.dim() == 2 &&
              out.stride(1) == 1);
  const int T_ = u.size(0), C = u.size(1);
  TORCH_CHECK(out.size(0) == T_ && out.size(1) == C);
  TORCH_CHECK(w.scalar_type() == at::kFloat && w.is_contiguous() &&
              w.dim() == 2 && w.size(1) == C, "weights must be [taps, C]");
  const int taps = w.size(0);
  TORCH_CHECK(taps >= 1 && taps <= MAX_TAPS, "unsupported tap count");
  TORCH_CHECK(tail.scalar_type() == at::kFloat && tail.is_contiguous() &&
              tail.dim() == 3 && tail.size(1) == taps - 1 && tail.size(2) == C,
              "tail must be fp32 [slots, taps-1, channels]");
  TORCH_CHECK(state_slots.scalar_type() == at::kLong &&
              state_slots.is_contiguous());
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  const int B = seq_lens.numel();
  TORCH_CHECK(state_slots.numel() == B);
  TORCH_CHECK(query_starts.has_value() == query_lens.has_value());
  const int* qs = nullptr;
  const int* ql = nullptr;
  if (query_starts.has_value()) {
    TORCH_CHECK(query_starts->scalar_type() == at::kInt &&
                query_lens->scalar_type() == at::kInt &&
                query_starts->numel() == B && query_lens->numel() == B &&
                query_starts->is_contiguous() && query_lens->is_contiguous());
    qs = query_starts->data_ptr<int>();
    ql = query_lens->data_ptr<int>();
  } else {
    TORCH_CHECK(T_ == B, "one token per sequence expected");
  }
  TORCH_CHECK(norm_channels >= 0 && norm_channels <= C &&
              lead_channels <= norm_channels);
  int cs = 256;
  if (norm_channels > 0) {
    TORCH_CHECK(head_dim >= 1 && head_dim <= 64 * MAXV &&
                norm_channels % head_dim == 0 &&
                lead_channels % head_dim == 0, "bad head size");
    cs = head_dim;
  }
  if (T_ == 0 || B == 0) return;
  const int n_chunks = (C + cs - 1) / cs;
  const bool out_f32 = out.scalar_type() == at::kFloat;
  TORCH_CHECK(out_f32 || out.scalar_type() == at::kBFloat16);
  auto stream = at::hip::getCurrentHIPStream();
#define LAUNCH(TI, TO)                                                        \
  hipLaunchKernelGGL((short_conv_kernel<TI, TO>),                             \
                     dim3((unsigned)((long)T_ * ((n_chunks + 3) / 4))),       \
                     dim3(256), 0, stream,                                    \
                     (TO*)out.data_ptr(), (long)out.stride(0),                \
                     (const TI*)u.data_ptr(), (long)u.stride(0),              \
                     w.data_ptr<float>(), tail.data_ptr<float>(),             \
                     state_slots.data_ptr<long>(), seq_lens.data_ptr<int>(),  \
                     qs, ql, B, C, taps, cs, n_chunks, (n_chunks + 3) / 4,    \
                     silu, (int)norm_channels, (int)lead_channels,            \
                     (float)lead_scale, (float)l2_eps)
  const bool vec = cs % 4 == 0 && cs <= 256 && C % 4 == 0 &&
                   u.stride(0) % 4 == 0 && out.stride(0) % 4 == 0 &&
                   u.storage_offset() % 4 == 0 && out.storage_offset() % 4 == 0;
  int lph = 1;
  while (lph * 4 < cs) lph <<= 1;
#define LAUNCH_VEC(TI, TO, L)                                                 \
  hipLaunchKernelGGL((short_conv_vec_kernel<TI, TO, L>),                      \
                     dim3((unsigned)((long)T_ * ((n_chunks + 4 * (64 / L) - 1) / \
                                                 (4 * (64 / L))))),           \
                     dim3(256), 0, stream, (TO*)out.data_ptr(),               \
                     (long)out.stride(0), (const TI*)u.data_ptr(),            \
                     (long)u.stride(0), w.data_ptr<float>(),                  \
                     tail.data_ptr<float>(), state_slots.data_ptr<long>(),    \
                     seq_lens.data_ptr<int>(), qs, ql, B, C, taps, cs,        \
                     n_chunks, (n_chunks + 4 * (64 / L) - 1) / (4 * (64 / L)), \
                     silu, (int)norm_channels, (int)lead_channels,            \
                     (float)lead_scale, (float)l2_eps)
#define LAUNCH_VEC_L(TI, TO)                                                  \
  do {                                                                        \
    if (lph <= 8) LAUNCH_VEC(TI, TO, 8);                                      \
    else if (lph == 16) LAUNCH_VEC(TI, TO, 16);                               \
    else if (lph == 32) LAUNCH_VEC(TI, TO, 32);                               \
    else LAUNCH_VEC(TI, TO, 64);                                              \
  } while (0)
  LATENT_DISPATCH_T(u, {
    if (vec) {
      if (out_f32) LAUNCH_VEC_L(T, float); else LAUNCH_VEC_L(T, short);
    } else {
      if (out_f32) LAUNCH(T, float); else LAUNCH(T, short);
    }
    if (taps > 1) {
      hipLaunchKernelGGL((conv_tail_kernel<T>), dim3((C + 255) / 256, B),
                         dim3(256), 0, stream, tail.data_ptr<float>(),
                         (const T*)u.data_ptr(), (long)u.stride(0),
                         state_slots.data_ptr<long>(),
                         seq_lens.data_ptr<int>(), qs, ql, C, taps);
    }
  });
#undef LAUNCH
#undef LAUNCH_VEC
#undef LAUNCH_VEC_L
}
