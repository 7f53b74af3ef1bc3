// Post-norm residual step with a (1 + w) RMS norm (gfx950).
//
//   s = (alpha + row_add[t]) * x + s1 * y + s2 * y2
//   x <- s / sqrt(mean(s^2) + eps) * w1p          (fp32 residual, in place)
//   h  = T(x)                                     (feeds the next GEMM)
//
// y, y2 and row_add are optional; w1p holds 1 + w. The weighted sum of up
// to two sublayer outputs, the per-row addition to the residual's
// coefficient (the share of experts whose output is the input itself), the
// norm and the cast are one kernel: one read of each input, one
// read+write of x. One 256-thread workgroup per row; the second pass
// re-reads what the same threads just read (L1/L2 hits). y may be fp32
// while h is bf16 (outputs accumulated in fp32).

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

template <typename T, int VEC>
__device__ __forceinline__ void ldv(const T* p, long i, float* v) {
  if constexpr (VEC == 4) {
    ld4(p, i, v);
  } else {
    v[0] = ldf(p, i);
  }
}
template <typename T, int VEC>
__device__ __forceinline__ void stv(T* p, long i, const float* v) {
  if constexpr (VEC == 4) {
    st4(p, i, v);
  } else {
    stf(p, i, v[0]);
  }
}

template <typename T, typename TY, int VEC>
__global__ __launch_bounds__(256) void postln_kernel(
    float* __restrict__ x, const TY* __restrict__ y, long y_rs, float s1,
    const T* __restrict__ y2, long y2_rs, float s2, float alpha,
    const float* __restrict__ row_add, const float* __restrict__ w1p,
    float eps, T* __restrict__ h, int W) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const float a = alpha + (row_add ? row_add[row] : 0.f);
  float* xr = x + row * W;
  const TY* yr = y ? y + row * y_rs : nullptr;
  const T* y2r = y2 ? y2 + row * y2_rs : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x * VEC; i < W; i += 256 * VEC) {
    float xv[VEC], v[VEC];
    ldv<float, VEC>(xr, i, xv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) xv[j] *= a;
    if (yr) {
      ldv<TY, VEC>(yr, i, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) xv[j] = fmaf(v[j], s1, xv[j]);
    }
    if (y2r) {
      ldv<T, VEC>(y2r, i, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) xv[j] = fmaf(v[j], s2, xv[j]);
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) ss = fmaf(xv[j], xv[j], ss);
  }
  const float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)W + eps);
  T* hr = h + row * W;
  for (int i = threadIdx.x * VEC; i < W; i += 256 * VEC) {
    float xv[VEC], v[VEC], wv[VEC];
    ldv<float, VEC>(xr, i, xv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) xv[j] *= a;
    if (yr) {
      ldv<TY, VEC>(yr, i, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) xv[j] = fmaf(v[j], s1, xv[j]);
    }
    if (y2r) {
      ldv<T, VEC>(y2r, i, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) xv[j] = fmaf(v[j], s2, xv[j]);
    }
    ldv<float, VEC>(w1p, i, wv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) xv[j] = xv[j] * r * wv[j];
    stv<float, VEC>(xr, i, xv);
    stv<T, VEC>(hr, i, xv);
  }
}

}  // namespace

void postln_rmsnorm_residual(torch::Tensor x, c10::optional<torch::Tensor> y,
                             double y_scale, c10::optional<torch::Tensor> y2,
                             double y2_scale, double alpha,
                             c10::optional<torch::Tensor> row_add,
                             torch::Tensor w1p, double eps, torch::Tensor h) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() &&
              x.dim() == 2);
  TORCH_CHECK(h.is_contiguous() && h.dim() == 2 && h.sizes() == x.sizes());
  const int rows = x.size(0), W = x.size(1);
  TORCH_CHECK(w1p.scalar_type() == at::kFloat && w1p.is_contiguous() &&
              w1p.numel() == W);
  bool y_f32 = false;
  long y_rs = 0, y2_rs = 0;
  if (y.has_value()) {
    TORCH_CHECK(y->dim() == 2 && y->size(0) == rows && y->size(1) == W &&
                y->stride(1) == 1);
    y_f32 = y->scalar_type() == at::kFloat;
    TORCH_CHECK(y_f32 || y->scalar_type() == h.scalar_type());
    y_rs = y->stride(0);
  }
  if (y2.has_value()) {
    TORCH_CHECK(y2->dim() == 2 && y2->size(0) == rows && y2->size(1) == W &&
                y2->stride(1) == 1 && y2->scalar_type() == h.scalar_type());
    y2_rs = y2->stride(0);
  }
  if (row_add.has_value())
    TORCH_CHECK(row_add->scalar_type() == at::kFloat &&
                row_add->is_contiguous() && row_add->numel() == rows);
  if (rows == 0) return;
  bool vec = W % 4 == 0 && y_rs % 4 == 0 && y2_rs % 4 == 0;
  if (y.has_value()) vec = vec && y->storage_offset() % 4 == 0;
  if (y2.has_value()) vec = vec && y2->storage_offset() % 4 == 0;
  const float* ra = row_add.has_value() ? row_add->data_ptr<float>() : nullptr;
  const void* yp = y.has_value() ? y->data_ptr() : nullptr;
  const void* y2p = y2.has_value() ? y2->data_ptr() : nullptr;
  auto stream = at::hip::getCurrentHIPStream();
#define LAUNCH(TT, TY, V)                                                     \
  hipLaunchKernelGGL((postln_kernel<TT, TY, V>), dim3(rows), dim3(256), 0,    \
                     stream, x.data_ptr<float>(), (const TY*)yp, y_rs,        \
                     (float)y_scale, (const TT*)y2p, y2_rs, (float)y2_scale,  \
                     (float)alpha, ra, w1p.data_ptr<float>(), (float)eps,     \
                     (TT*)h.data_ptr(), W)
  LATENT_DISPATCH_T(h, {
    if (y_f32) {
      if (vec) LAUNCH(T, float, 4); else LAUNCH(T, float, 1);
    } else {
      if (vec) LAUNCH(T, T, 4); else LAUNCH(T, T, 1);
    }
  });
#undef LAUNCH
}
