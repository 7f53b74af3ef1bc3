// Gated residual update fused with a layer norm, and the elementwise
// activations of the gated family (gfx950).
//
//   residual_update_norm   x (fp32, in place) gets one of
//                            nothing
//                            x += sigmoid(gate + gate_bias) * y
//                            x += y / sqrt(mean(y^2) + eps) * rms_w
//                          and then h = ((x - mean) / sqrt(var + eps)) * w + b
//                          in the compute dtype (the next GEMM's input), or
//                          h = x cast (no norm weights), or nothing.
//                          One 256-thread workgroup per row; the updated row
//                          stays in registers between the passes (rows up to
//                          256 * 4 * ROW_REGS values), so x is read and
//                          written once. The variance is the mean of squared
//                          deviations (second pass over registers), not
//                          E[x^2] - mean^2.
//   xielu                  z > 0: a_p z^2 + z/2; z <= 0: a_n (e^z - 1 - z) + z/2
//   gelu_gate_rows         out[r, d] = gelu_tanh(t[r, d]) * table[ids[r], c0 + d]
//   sigmoid_gate_rows      out[r, c] = a[r, c] * sigmoid(gate[r, c])
//
// All math is fp32; T is the compute dtype (short = bf16 bits, float).

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

constexpr int UPD_NONE = 0, UPD_GATE = 1, UPD_RMS = 2;
constexpr int ROW_REGS = 8;   // float4 groups per thread: rows <= 8192 values

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

__device__ __forceinline__ float sigmoid_(float v) {
  return 1.0f / (1.0f + expf(-v));
}

// NREG groups of VEC values per thread hold the row; W <= 256 * VEC * NREG
template <typename T, int VEC, int NREG>
__global__ __launch_bounds__(256) void residual_update_norm_kernel(
    float* __restrict__ x, const T* __restrict__ y, long y_rs, int update,
    const T* __restrict__ gate, long g_rs, const float* __restrict__ gate_bias,
    const float* __restrict__ rms_w, float eps,
    const float* __restrict__ norm_w, const float* __restrict__ norm_b,
    T* __restrict__ h, int W) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* xr = x + row * W;
  const float inv_w = 1.0f / (float)W;
  float xv[NREG][VEC];

  float scale_y = 1.0f;
  if (update == UPD_RMS) {
    const T* yr = y + row * y_rs;
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < NREG; ++k) {
      const int i = (k * 256 + threadIdx.x) * VEC;
      if (i < W) {
        float v[VEC];
        ldv<T, VEC>(yr, i, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) ss = fmaf(v[j], v[j], ss);
      }
    }
    scale_y = 1.0f / sqrtf(block_sum_256(ss, red) * inv_w + eps);
  }

  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < NREG; ++k) {
    const int i = (k * 256 + threadIdx.x) * VEC;
#pragma unroll
    for (int j = 0; j < VEC; ++j) xv[k][j] = 0.f;
    if (i < W) {
      ldv<float, VEC>(xr, i, xv[k]);
      if (update == UPD_GATE) {
        float v[VEC], g[VEC], gb[VEC];
        ldv<T, VEC>(y + row * y_rs, i, v);
        ldv<T, VEC>(gate + row * g_rs, i, g);
#pragma unroll
        for (int j = 0; j < VEC; ++j) gb[j] = 0.f;
        if (gate_bias) ldv<float, VEC>(gate_bias, i, gb);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          xv[k][j] = fmaf(sigmoid_(g[j] + gb[j]), v[j], xv[k][j]);
      } else if (update == UPD_RMS) {
        float v[VEC], w[VEC];
        ldv<T, VEC>(y + row * y_rs, i, v);
        ldv<float, VEC>(rms_w, i, w);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          xv[k][j] = fmaf(v[j] * scale_y, w[j], xv[k][j]);
      }
      if (update != UPD_NONE) stv<float, VEC>(xr, i, xv[k]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) sum += xv[k][j];
    }
  }
  if (h == nullptr) return;
  T* hr = h + row * W;
  if (norm_w == nullptr) {
#pragma unroll
    for (int k = 0; k < NREG; ++k) {
      const int i = (k * 256 + threadIdx.x) * VEC;
      if (i < W) stv<T, VEC>(hr, i, xv[k]);
    }
    return;
  }
  const float mean = block_sum_256(sum, red) * inv_w;
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < NREG; ++k) {
    const int i = (k * 256 + threadIdx.x) * VEC;
    if (i < W) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        xv[k][j] -= mean;
        sq = fmaf(xv[k][j], xv[k][j], sq);
      }
    }
  }
  const float r = 1.0f / sqrtf(block_sum_256(sq, red) * inv_w + eps);
#pragma unroll
  for (int k = 0; k < NREG; ++k) {
    const int i = (k * 256 + threadIdx.x) * VEC;
    if (i < W) {
      float w[VEC], b[VEC], o[VEC];
      ldv<float, VEC>(norm_w, i, w);
#pragma unroll
      for (int j = 0; j < VEC; ++j) b[j] = 0.f;
      if (norm_b) ldv<float, VEC>(norm_b, i, b);
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = fmaf(xv[k][j] * r, w[j], b[j]);
      stv<T, VEC>(hr, i, o);
    }
  }
}

// bf16, 8 values (16 bytes) per thread
__global__ void xielu_bf16x8_kernel(short* __restrict__ out,
                                    const short* __restrict__ z, long z_rs,
                                    const float* __restrict__ coef, long n,
                                    int C) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (i >= n) return;
  const long r = i / C;
  const int c = (int)(i % C);
  const float ap = coef[0], an = coef[1];
  const bf16x8 v = *reinterpret_cast<const bf16x8*>(z + r * z_rs + c);
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float a = bits2f(v[j]);
    o[j] = f2bits(a > 0.f ? fmaf(ap * a, a, 0.5f * a)
                          : fmaf(an, expm1f(a) - a, 0.5f * a));
  }
  *reinterpret_cast<bf16x8*>(out + i) = o;
}

template <typename T, int VEC>
__global__ void xielu_kernel(T* __restrict__ out, const T* __restrict__ z,
                             long z_rs, const float* __restrict__ coef, long n,
                             int C) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const long r = i / C;
  const int c = (int)(i % C);
  const float ap = coef[0], an = coef[1];
  float v[VEC], o[VEC];
  ldv<T, VEC>(z, r * z_rs + c, v);
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    const float a = v[j];
    o[j] = a > 0.f ? fmaf(ap * a, a, 0.5f * a)
                   : fmaf(an, expm1f(a) - a, 0.5f * a);
  }
  stv<T, VEC>(out, i, o);
}

template <typename T>
__global__ void gelu_gate_rows_kernel(T* __restrict__ out,
                                      const T* __restrict__ t, long t_rs,
                                      const T* __restrict__ table, long tab_rs,
                                      const long* __restrict__ ids, int col0,
                                      long n, int C) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const long r = i / C;
  const int c = (int)(i % C);
  const float z = ldf(t, r * t_rs + c);
  const float g =
      0.5f * z * (1.0f + tanhf(0.7978845608028654f *
                               (z + 0.044715f * z * z * z)));
  stf(out, i, g * ldf(table, ids[r] * tab_rs + col0 + c));
}

template <typename T, int VEC>
__global__ void sigmoid_gate_rows_kernel(T* __restrict__ out, long o_rs,
                                         const T* __restrict__ a, long a_rs,
                                         const T* __restrict__ g, long g_rs,
                                         long n, int C) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (i >= n) return;
  const long r = i / C;
  const int c = (int)(i % C);
  float av[VEC], gv[VEC], o[VEC];
  ldv<T, VEC>(a, r * a_rs + c, av);
  ldv<T, VEC>(g, r * g_rs + c, gv);
#pragma unroll
  for (int j = 0; j < VEC; ++j) o[j] = av[j] * sigmoid_(gv[j]);
  stv<T, VEC>(out, r * o_rs + c, o);
}

bool aligned_rows(const torch::Tensor& t, int elems) {
  return t.stride(0) % elems == 0 && t.storage_offset() % elems == 0;
}

}  // namespace

void residual_update_norm(torch::Tensor x, c10::optional<torch::Tensor> y,
                          long update, c10::optional<torch::Tensor> gate,
                          c10::optional<torch::Tensor> gate_bias,
                          c10::optional<torch::Tensor> rms_w, double eps,
                          c10::optional<torch::Tensor> norm_w,
                          c10::optional<torch::Tensor> norm_b,
                          c10::optional<torch::Tensor> h) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() &&
              x.dim() == 2);
  const int rows = x.size(0), W = x.size(1);
  TORCH_CHECK(update >= UPD_NONE && update <= UPD_RMS);
  TORCH_CHECK(W <= 256 * 4 * ROW_REGS, "row wider than ", 256 * 4 * ROW_REGS);
  auto check_vec = [&](const c10::optional<torch::Tensor>& t) {
    if (t.has_value())
      TORCH_CHECK(t->scalar_type() == at::kFloat && t->is_contiguous() &&
                  t->numel() == W);
  };
  check_vec(gate_bias);
  check_vec(rms_w);
  check_vec(norm_w);
  check_vec(norm_b);
  bool vec = W % 4 == 0;
  long y_rs = 0, g_rs = 0;
  at::ScalarType ct = at::kFloat;
  bool have_ct = false;
  auto check_rows = [&](const torch::Tensor& t) {
    TORCH_CHECK(t.dim() == 2 && t.size(0) == rows && t.size(1) == W &&
                t.stride(1) == 1);
    TORCH_CHECK(!have_ct || t.scalar_type() == ct,
                "y, gate and h share one element type");
    ct = t.scalar_type();
    have_ct = true;
    vec = vec && aligned_rows(t, 4);
  };
  if (update != UPD_NONE) {
    TORCH_CHECK(y.has_value(), "an update needs y");
    check_rows(*y);
    y_rs = y->stride(0);
  }
  if (update == UPD_GATE) {
    TORCH_CHECK(gate.has_value(), "gated update needs the gate logits");
    check_rows(*gate);
    g_rs = gate->stride(0);
  }
  if (update == UPD_RMS) TORCH_CHECK(rms_w.has_value());
  if (h.has_value()) {
    check_rows(*h);
    TORCH_CHECK(h->is_contiguous());
  } else {
    TORCH_CHECK(!norm_w.has_value());
  }
  if (rows == 0 || (update == UPD_NONE && !h.has_value())) return;
  if (!have_ct) return;
  const void* yp = update != UPD_NONE ? y->data_ptr() : nullptr;
  const void* gp = update == UPD_GATE ? gate->data_ptr() : nullptr;
  const float* gb = gate_bias.has_value() ? gate_bias->data_ptr<float>() : nullptr;
  const float* rw = rms_w.has_value() ? rms_w->data_ptr<float>() : nullptr;
  const float* nw = norm_w.has_value() ? norm_w->data_ptr<float>() : nullptr;
  const float* nb = norm_b.has_value() ? norm_b->data_ptr<float>() : nullptr;
  void* hp = h.has_value() ? h->data_ptr() : nullptr;
  auto stream = at::hip::getCurrentHIPStream();
#define LAUNCH(TT, V, N)                                                      \
  hipLaunchKernelGGL((residual_update_norm_kernel<TT, V, N>), dim3(rows),     \
                     dim3(256), 0, stream, x.data_ptr<float>(),               \
                     (const TT*)yp, y_rs, (int)update, (const TT*)gp, g_rs,   \
                     gb, rw, (float)eps, nw, nb, (TT*)hp, W)
  const bool bf = ct == at::kBFloat16;
  TORCH_CHECK(bf || ct == at::kFloat, "expected bf16 or fp32 rows");
  if (vec) {
    const int groups = (W / 4 + 255) / 256;
    if (groups <= 2) {
      if (bf) LAUNCH(short, 4, 2); else LAUNCH(float, 4, 2);
    } else {
      if (bf) LAUNCH(short, 4, ROW_REGS); else LAUNCH(float, 4, ROW_REGS);
    }
  } else {
    TORCH_CHECK(W <= 256 * 32, "unaligned row wider than 8192");
    if (bf) LAUNCH(short, 1, 32); else LAUNCH(float, 1, 32);
  }
#undef LAUNCH
}

void xielu(torch::Tensor out, torch::Tensor z, torch::Tensor coef) {
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && z.dim() == 2 &&
              z.sizes() == out.sizes() && z.stride(1) == 1 &&
              z.scalar_type() == out.scalar_type());
  TORCH_CHECK(coef.scalar_type() == at::kFloat && coef.numel() == 2 &&
              coef.is_contiguous());
  const long n = out.numel();
  const int C = out.size(1);
  if (n == 0) return;
  const bool vec = C % 4 == 0 && aligned_rows(z, 4);
  auto stream = at::hip::getCurrentHIPStream();
  if (out.scalar_type() == at::kBFloat16 && C % 8 == 0 && aligned_rows(z, 8) &&
      reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(z.data_ptr()) % 16 == 0) {
    hipLaunchKernelGGL(xielu_bf16x8_kernel, dim3((n / 8 + 255) / 256),
                       dim3(256), 0, stream, (short*)out.data_ptr(),
                       (const short*)z.data_ptr(), (long)z.stride(0),
                       coef.data_ptr<float>(), n, C);
    return;
  }
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((xielu_kernel<T, 4>), dim3((n / 4 + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)z.data_ptr(), (long)z.stride(0),
                         coef.data_ptr<float>(), n, C);
    } else {
      hipLaunchKernelGGL((xielu_kernel<T, 1>), dim3((n + 255) / 256),
                         dim3(256), 0, stream, (T*)out.data_ptr(),
                         (const T*)z.data_ptr(), (long)z.stride(0),
                         coef.data_ptr<float>(), n, C);
    }
  });
}

void gelu_gate_rows(torch::Tensor out, torch::Tensor t, torch::Tensor table,
                    torch::Tensor ids, long col0) {
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && t.dim() == 2 &&
              t.sizes() == out.sizes() && t.stride(1) == 1 &&
              t.scalar_type() == out.scalar_type() &&
              table.scalar_type() == out.scalar_type());
  TORCH_CHECK(table.dim() == 2 && table.stride(1) == 1 && col0 >= 0 &&
              col0 + out.size(1) <= table.size(1), "table slice out of range");
  TORCH_CHECK(ids.scalar_type() == at::kLong && ids.is_contiguous() &&
              ids.numel() == out.size(0));
  const long n = out.numel();
  if (n == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    hipLaunchKernelGGL((gelu_gate_rows_kernel<T>), dim3((n + 255) / 256),
                       dim3(256), 0, stream, (T*)out.data_ptr(),
                       (const T*)t.data_ptr(), (long)t.stride(0),
                       (const T*)table.data_ptr(), (long)table.stride(0),
                       ids.data_ptr<long>(), (int)col0, n, (int)out.size(1));
  });
}

void sigmoid_gate_rows(torch::Tensor out, torch::Tensor a, torch::Tensor gate) {
  TORCH_CHECK(out.dim() == 2 && a.dim() == 2 && gate.dim() == 2 &&
              a.sizes() == out.sizes() && gate.sizes() == out.sizes() &&
              out.stride(1) == 1 && a.stride(1) == 1 && gate.stride(1) == 1);
  TORCH_CHECK(a.scalar_type() == out.scalar_type() &&
              gate.scalar_type() == out.scalar_type());
  const long n = out.numel();
  const int C = out.size(1);
  if (n == 0) return;
  const bool vec = C % 4 == 0 && aligned_rows(out, 4) && aligned_rows(a, 4) &&
                   aligned_rows(gate, 4);
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(out, {
    if (vec) {
      hipLaunchKernelGGL((sigmoid_gate_rows_kernel<T, 4>),
                         dim3((n / 4 + 255) / 256), dim3(256), 0, stream,
                         (T*)out.data_ptr(), (long)out.stride(0),
                         (const T*)a.data_ptr(), (long)a.stride(0),
                         (const T*)gate.data_ptr(), (long)gate.stride(0), n, C);
    } else {
      hipLaunchKernelGGL((sigmoid_gate_rows_kernel<T, 1>),
                         dim3((n + 255) / 256), dim3(256), 0, stream,
                         (T*)out.data_ptr(), (long)out.stride(0),
                         (const T*)a.data_ptr(), (long)a.stride(0),
                         (const T*)gate.data_ptr(), (long)gate.stride(0), n, C);
    }
  });
}
