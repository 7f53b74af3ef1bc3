// Sigmoid group-limited routing with always-on gates, and the gated expert
// activation with the routing weight on the output side (gfx950).
//
//   grouped_sigmoid_route: per token row (one wave), in fp32:
//     s = sigmoid(z);  c = s + correction          (c only decides the CHOICE)
//     the E experts form n_groups equal consecutive groups; a group scores
//     the sum of its group_top largest c; the keep_groups best groups stay
//     eligible (the others count as -inf: c may be negative); the `top`
//     eligible experts with the largest c are chosen and weigh s — not
//     renormalized. weight[t, e] = 0 elsewhere. Columns E.. of the logits
//     are always-on gates: weight = sigmoid(z).
//   routed_silu_glu: stacked experts, out[t, e*F + f] = w[t, e] *
//     silu(gate) * up; experts with w == 0 write 0 without reading their
//     columns. A tail expert of another inner size Ft follows the E equal
//     ones (gate | up at column E*2F of gu, output at column E*F) and is
//     weighed by w[t, E].

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

constexpr int ROUTE_PER_LANE = 16;  // experts <= 64 * 16
constexpr int MAX_GROUPS = 64;

__global__ __launch_bounds__(64) void sigmoid_route_kernel(
    float* __restrict__ weight, const float* __restrict__ logits,
    const float* __restrict__ correction, int E, int A, int top, int n_groups,
    int keep_groups, int group_top) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x;
  const int gsz = E / n_groups;
  const long rs = E + A;
  float s[ROUTE_PER_LANE], c[ROUTE_PER_LANE];
  bool taken[ROUTE_PER_LANE];
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    taken[k] = false;
    s[k] = e < E ? 1.0f / (1.0f + expf(-logits[t * rs + e])) : 0.f;
    c[k] = e < E ? s[k] + (correction ? correction[e] : 0.f) : -INFINITY;
  }
  for (int a = lane; a < A; a += WAVE)
    weight[t * rs + E + a] = 1.0f / (1.0f + expf(-logits[t * rs + E + a]));

  // eligible groups: lane g holds the score of group g
  unsigned long long eligible = ~0ull;
  if (n_groups > 1 && keep_groups < n_groups) {
    float gscore = -INFINITY;
    for (int g = 0; g < n_groups; ++g) {
      // sum of the group's group_top largest c: pick them one at a time
      bool used[ROUTE_PER_LANE];
#pragma unroll
      for (int k = 0; k < ROUTE_PER_LANE; ++k) used[k] = false;
      float acc = 0.f;
      const int picks = min(group_top, gsz);
      for (int r = 0; r < picks; ++r) {
        float bv = -INFINITY;
        int be = 0x7fffffff;
#pragma unroll
        for (int k = 0; k < ROUTE_PER_LANE; ++k) {
          const int e = k * WAVE + lane;
          if (e < E && e / gsz == g && !used[k] &&
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
          if (k * WAVE + lane == be) used[k] = true;
        acc += bv;
      }
      if (lane == g) gscore = acc;
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
        if (og != 0x7fffffff &&
            (bg == 0x7fffffff || ov > bv || (ov == bv && og < bg))) {
          bv = ov; bg = og;
        }
      }
      if (bg < n_groups) {
        eligible |= 1ull << bg;
        if (lane == bg) mine = true;
      }
    }
  }
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
      if (k * WAVE + lane == be) taken[k] = true;
  }
#pragma unroll
  for (int k = 0; k < ROUTE_PER_LANE; ++k) {
    const int e = k * WAVE + lane;
    if (e < E) weight[t * rs + e] = taken[k] ? s[k] : 0.f;
  }
}

// one thread per VEC consecutive outputs of a row; VEC divides F and Ft
template <typename T, int VEC>
__global__ void silu_glu_kernel(T* __restrict__ out, const T* __restrict__ gu,
                                const float* __restrict__ weight, long w_rs,
                                long n, int E, int F, int Ft, long gu_rs) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const int C = E * F + Ft;
  const long t = i / C;
  const int rem = (int)(i % C);
  int e, f, fe;
  long base;
  if (rem < E * F) {
    e = rem / F; f = rem % F; fe = F;
    base = t * gu_rs + (long)e * 2 * F + f;
  } else {
    e = E; f = rem - E * F; fe = Ft;
    base = t * gu_rs + (long)E * 2 * F + f;
  }
  const float w = weight[t * w_rs + e];
  float o[VEC];
  if (w == 0.f) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[j] = 0.f;
  } else {
    float g[VEC], u[VEC];
    if constexpr (VEC == 4) {
      ld4(gu, base, g);
      ld4(gu, base + fe, u);
    } else {
      g[0] = ldf(gu, base);
      u[0] = ldf(gu, base + fe);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      o[j] = w * (g[j] / (1.0f + expf(-g[j]))) * u[j];
  }
  if constexpr (VEC == 4) {
    st4(out, i, o);
  } else {
    stf(out, i, o[0]);
  }
}

}  // namespace

void grouped_sigmoid_route(torch::Tensor weight, torch::Tensor logits,
                           c10::optional<torch::Tensor> correction,
                           long n_experts, long top, long n_groups,
                           long keep_groups, long group_top) {
  TORCH_CHECK(weight.scalar_type() == at::kFloat && weight.is_contiguous());
  TORCH_CHECK(logits.scalar_type() == at::kFloat && logits.is_contiguous() &&
              logits.dim() == 2);
  const int T_ = logits.size(0), E = n_experts;
  const int A = logits.size(1) - E;
  TORCH_CHECK(E >= 1 && A >= 0 && weight.numel() == (long)T_ * (E + A));
  TORCH_CHECK(E <= WAVE * ROUTE_PER_LANE, "too many experts");
  TORCH_CHECK(n_groups >= 1 && n_groups <= MAX_GROUPS && E % n_groups == 0 &&
              keep_groups >= 1 && keep_groups <= n_groups, "bad groups");
  TORCH_CHECK(top >= 1 && top <= keep_groups * (E / n_groups),
              "top out of range");
  TORCH_CHECK(group_top >= 1);
  const float* corr = nullptr;
  if (correction.has_value()) {
    TORCH_CHECK(correction->scalar_type() == at::kFloat &&
                correction->is_contiguous() && correction->numel() == E);
    corr = correction->data_ptr<float>();
  }
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  hipLaunchKernelGGL(sigmoid_route_kernel, dim3(T_), dim3(64), 0, stream,
                     weight.data_ptr<float>(), logits.data_ptr<float>(), corr,
                     E, A, (int)top, (int)n_groups, (int)keep_groups,
                     (int)group_top);
}

void routed_silu_glu(torch::Tensor out, torch::Tensor gu, torch::Tensor weight,
                     long n_experts, long ff, long tail_ff) {
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && gu.dim() == 2 &&
              gu.stride(1) == 1 && gu.scalar_type() == out.scalar_type());
  TORCH_CHECK(weight.scalar_type() == at::kFloat && weight.dim() == 2 &&
              weight.stride(1) == 1);
  const int T_ = out.size(0), E = n_experts, F = ff, Ft = tail_ff;
  TORCH_CHECK(E >= 0 && F >= 1 && Ft >= 0 && (E > 0 || Ft > 0));
  TORCH_CHECK(weight.size(0) == T_ && gu.size(0) == T_ &&
              weight.size(1) >= E + (Ft > 0 ? 1 : 0));
  TORCH_CHECK(out.size(1) == (long)E * F + Ft, "output width mismatch");
  TORCH_CHECK(gu.size(1) == (long)2 * E * F + 2 * Ft, "gate|up width mismatch");
  const long n = (long)T_ * out.size(1);
  if (n == 0) return;
  const bool vec = F % 4 == 0 && Ft % 4 == 0 && gu.stride(0) % 4 == 0 &&
                   gu.storage_offset() % 4 == 0;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((silu_glu_kernel<T, 4>), dim3((n / 4 + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gu.data_ptr(), weight.data_ptr<float>(),
                         (long)weight.stride(0), n, E, F, Ft,
                         (long)gu.stride(0));
    } else {
      hipLaunchKernelGGL((silu_glu_kernel<T, 1>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)gu.data_ptr(), weight.data_ptr<float>(),
                         (long)weight.stride(0), n, E, F, Ft,
                         (long)gu.stride(0));
    }
  });
}
