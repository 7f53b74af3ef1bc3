// Group-limited softmax routing and the clamped gated expert activation
// (gfx950).
//
//   grouped_softmax_route: per token row (one wave), in fp32:
//     s = softmax(z);  c = s + correction          (c only decides the CHOICE)
//     experts form n_groups equal consecutive groups; a group scores
//     max(c) over its members; the keep_groups best groups stay eligible;
//     the `top` eligible experts with the largest c are chosen and weigh
//     s / (sum of chosen s + 1e-20) * scale.   weight[t, e] = 0 elsewhere.
//   routed_clamped_glu: stacked-expert activation with the routing weight
//     on the expert OUTPUT (the down projection is linear, so scaling its
//     input row scales its output): g = min(gate, limit),
//     u = clamp(up, -limit, limit),
//     out[t, e, f] = w[t, e] * g * sigmoid(slope * g) * (u + 1); experts
//     with w == 0 write 0 without reading their columns.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

constexpr int ROUTE_PER_LANE = 16;  // experts <= 64 * 16
constexpr int MAX_GROUPS = 64;

__global__ __launch_bounds__(64) void grouped_route_kernel(
    float* __restrict__ weight, const float* __restrict__ logits,
    const float* __restrict__ correction, int E, int top, int n_groups,
    int keep_groups, float scale) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const int gsz = E / n_groups;
  float s[ROUTE_PER_LANE], c[ROUTE_PER_LANE];
  bool taken[ROUTE_PER_LANE];
  float mx = -INFINITY;
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    taken[k] = false;
    s[k] = e < E ? logits[t * E + e] : -INFINITY;
    mx = fmaxf(mx, s[k]);
  }
  mx = wave_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    s[k] = e < E ? expf(s[k] - mx) : 0.f;
    sum += s[k];
  }
  sum = wave_sum(sum);
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    s[k] = s[k] / sum;
    c[k] = e < E ? s[k] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  // eligible groups: lane g holds the score of group g
  unsigned long long eligible = ~0ull;
  if (n_groups > 1 && keep_groups < n_groups) {
    float gscore = -INFINITY;
    for (int g = 0; g < n_groups; ++g) {
      float m = -INFINITY;
#pragma unroll
      for (int k = 0; k < ROUTE_PER_LANE; ++k) {
        const int e = k * WAVE + lane;
        if (e < E && e / gsz == g) m = fmaxf(m, c[k]);
      }
      m = wave_max(m);
      if (lane == g) gscore = m;
    }
    eligible = 0ull;
    bool mine = false;
    for (int r = 0; r < keep_groups; ++r) {
      float bv = (lane < n_groups && !mine) ? gscore : -INFINITY;
      int bg = (lane < n_groups && !mine) ? lane : 0x7fffffff;
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, WAVE);
        const int og = __shfl_xor(bg, off, WAVE);
        if (ov > bv || (ov == bv && og < bg)) { bv = ov; bg = og; }
      }
      if (bg < n_groups) {
        eligible |= 1ull << bg;
        if (lane == bg) mine = true;
      }
    }
  }
  float chosen = 0.f;
  for (int r = 0; r < top; ++r) {
    float bv = -INFINITY;
    int be = 0x7fffffff;
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k) {
      const int e = k * WAVE + lane;
      if (e < E && !taken[k] && ((eligible >> (e / gsz)) & 1ull) &&
          (c[k] > bv || be == 0x7fffffff)) {
        bv = c[k]; be = e;
      }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, WAVE);
      const int oe = __shfl_xor(be, off, WAVE);
      if (oe != 0x7fffffff &&
          (be == 0x7fffffff || ov > bv || (ov == bv && oe < be))) {
        bv = ov; be = oe;
      }
    }
#pragma unroll
    for (int k = 0; k < ROUTE_PER_LANE; ++k)
      if (k * WAVE + lane == be) { taken[k] = true; chosen += s[k]; }
  }
  chosen = wave_sum(chosen);
  const float mul = scale / (chosen + 1e-20f);
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    if (e < E) weight[t * E + e] = taken[k] ? s[k] * mul : 0.f;
  }
}

template <typename T, int VEC>
__global__ void clamped_glu_kernel(T* __restrict__ out,
                                   const T* __restrict__ gu,
                                   const float* __restrict__ weight, long w_rs,
                                   long n, int E, int F, long gu_rs,
                                   float limit, float slope) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const long t = i / ((long)E * F);
  const int rem = (int)(i % ((long)E * F));
  const int e = rem / F, f = rem % F;
  const float w = weight[t * w_rs + e];
  float o[VEC];
  if (w == 0.f) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = 0.f;
  } else {
    float g[VEC], u[VEC];
    const long base = t * gu_rs + (long)e * 2 * F + f;
    if constexpr (VEC == 4) {
      ld4(gu, base, g);
      ld4(gu, base + F, u);
    } else {
      g[0] = ldf(gu, base);
      u[0] = ldf(gu, base + F);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float gc = fminf(g[j], limit);
      const float uc = fminf(fmaxf(u[j], -limit), limit);
      o[j] = w * (gc / (1.0f + expf(-slope * gc))) * (uc + 1.0f);
    }
  }
  if constexpr (VEC == 4) {
    st4(out, i, o);
  } else {
    stf(out, i, o[0]);
  }
}

}  // namespace

void grouped_softmax_route(torch::Tensor weight, torch::Tensor logits,
                           c10::optional<torch::Tensor> correction, long top,
                           long n_groups, long keep_groups, double scale) {
  TORCH_CHECK(weight.scalar_type() == at::kFloat && weight.is_contiguous());
  TORCH_CHECK(logits.scalar_type() == at::kFloat && logits.is_contiguous() &&
              logits.dim() == 2);
  const int T_ = logits.size(0), E = logits.size(1);
  TORCH_CHECK(weight.numel() == (long)T_ * E);
  TORCH_CHECK(E <= WAVE * ROUTE_PER_LANE, "too many experts");
  TORCH_CHECK(n_groups >= 1 && n_groups <= MAX_GROUPS && E % n_groups == 0 &&
              keep_groups >= 1 && keep_groups <= n_groups, "bad groups");
  TORCH_CHECK(top >= 1 && top <= keep_groups * (E / n_groups),
              "top out of range");
  const float* corr = nullptr;
  if (correction.has_value()) {
    TORCH_CHECK(correction->scalar_type() == at::kFloat &&
                correction->is_contiguous() && correction->numel() == E);
    corr = correction->data_ptr<float>();
  }
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  hipLaunchKernelGGL(grouped_route_kernel, dim3(T_), dim3(64), 0, stream,
                     weight.data_ptr<float>(), logits.data_ptr<float>(), corr,
                     E, (int)top, (int)n_groups, (int)keep_groups,
                     (float)scale);
}

void routed_clamped_glu(torch::Tensor out, torch::Tensor gu,
                        torch::Tensor weight, long n_experts, double limit,
                        double slope) {
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && gu.dim() == 2 &&
              gu.stride(1) == 1 && gu.scalar_type() == out.scalar_type());
  TORCH_CHECK(weight.scalar_type() == at::kFloat && weight.dim() == 2 &&
              weight.stride(1) == 1);
  const int T_ = out.size(0), E = n_experts;
  TORCH_CHECK(E >= 1 && weight.size(1) >= E && weight.size(0) == T_ &&
              gu.size(0) == T_);
  TORCH_CHECK(out.size(1) % E == 0);
  const int F = out.size(1) / E;
  TORCH_CHECK(gu.size(1) == (long)2 * E * F, "gate|up width mismatch");
  const long n = (long)T_ * E * F;
  if (n == 0) return;
  const bool vec = F % 4 == 0 && gu.stride(0) % 4 == 0 &&
                   gu.storage_offset() % 4 == 0;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((clamped_glu_kernel<T, 4>), dim3((n / 4 + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gu.data_ptr(), weight.data_ptr<float>(),
                         (long)weight.stride(0), n, E, F, (long)gu.stride(0),
                         (float)limit, (float)slope);
    } else {
      hipLaunchKernelGGL((clamped_glu_kernel<T, 1>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gu.data_ptr(), weight.data_ptr<float>(),
                         (long)weight.stride(0), n, E, F, (long)gu.stride(0),
                         (float)limit, (float)slope);
    }
  });
}
