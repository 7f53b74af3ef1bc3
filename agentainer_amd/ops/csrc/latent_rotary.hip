// Rotary + latent norm + append for latent attention with a shared rotated
// key part, and the plain K/V append (gfx950).
//
//   latent_rotary_append: one workgroup per token row of the input
//   projection proj [T, n]:
//     * every query head's rotated part proj[h*q_head + q_rot_off .. +rot_dim]
//       is rotated IN PLACE,
//     * c = proj[kv_off .. +R] / sqrt(mean(c^2) + eps) * w goes to
//       cache[slot, 0..R),
//     * the shared key part proj[kv_off+R .. +rot_dim] is rotated into
//       cache[slot, R .. R+rot_dim),
//     * the pool row's remaining columns are zeroed.
//   Rotation pairs coordinate i with i + half, half = cos_sin.size(1) / 2,
//   coordinates from 2*half on pass unchanged; cos_sin [T, 2*half] fp32 is
//   the step's cos | sin table. All math fp32. slot < 0 skips the append.
//
//   head_kv_append: k [T, G, D], v [T, G, Dv] copied to the per-head pools
//   [P, G, PS, D] / [P, G, PS, Dv] at slot = page*PS + offset.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void latent_rotary_append_kernel(
    T* __restrict__ proj, long p_rs, int H, int q_head, int q_rot_off,
    int kv_off, int R, int rot_dim, int half, const float* __restrict__ w_kv,
    float eps, const float* __restrict__ cos_sin, T* __restrict__ cache, int Rp,
    const long* __restrict__ slots) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  T* pr = proj + t * p_rs;
  const float* cs = cos_sin + t * 2 * half;
  // queries: H * half pairs
  for (int i = threadIdx.x; i < H * half; i += 256) {
    const int h = i / half, j = i % half;
    T* qr = pr + h * q_head + q_rot_off;
    const float a = ldf(qr, j), b = ldf(qr, j + half);
    const float c = cs[j], s = cs[half + j];
    stf(qr, j, a * c - b * s);
    stf(qr, j + half, b * c + a * s);
  }
  const long slot = slots[t];
  // latent norm (every thread takes part in the reduction)
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) {
    const float v = ldf(pr, kv_off + i);
    ss = fmaf(v, v, ss);
  }
  const float r = 1.0f / sqrtf(block_sum_256(ss, red) / (float)R + eps);
  if (slot < 0) return;
  T* row = cache + slot * Rp;
  for (int i = threadIdx.x; i < R; i += 256)
    stf(row, i, ldf(pr, kv_off + i) * r * w_kv[i]);
  const T* kr = pr + kv_off + R;
  for (int j = threadIdx.x; j < half; j += 256) {
    const float a = ldf(kr, j), b = ldf(kr, j + half);
    const float c = cs[j], s = cs[half + j];
    stf(row, R + j, a * c - b * s);
    stf(row, R + j + half, b * c + a * s);
  }
  for (int j = 2 * half + threadIdx.x; j < rot_dim; j += 256)
    stf(row, R + j, ldf(kr, j));
  for (int j = R + rot_dim + threadIdx.x; j < Rp; j += 256) stf(row, j, 0.f);
}

template <typename T>
__global__ void kv_append_kernel(const T* __restrict__ k, long k_ts, long k_hs,
                                 const T* __restrict__ v, long v_ts, long v_hs,
                                 T* __restrict__ kc, T* __restrict__ vc,
                                 const long* __restrict__ slots, int G, int D,
                                 int Dv, int PS) {
  const long t = blockIdx.x;
  const long slot = slots[t];
  if (slot < 0) return;
  const long page = slot / PS, off = slot % PS;
  for (int i = threadIdx.x; i < G * (D + Dv); i += blockDim.x) {
    const int g = i / (D + Dv), e = i % (D + Dv);
    if (e < D)
      kc[((page * G + g) * PS + off) * D + e] = k[t * k_ts + g * k_hs + e];
    else
      vc[((page * G + g) * PS + off) * Dv + (e - D)] =
          v[t * v_ts + g * v_hs + (e - D)];
  }
}

}  // namespace

void latent_rotary_append(torch::Tensor proj, long heads, long q_head,
                          long q_rot_off, long kv_off, long kv_rank,
                          long rot_dim, torch::Tensor w_kv, double eps,
                          torch::Tensor cos_sin, torch::Tensor cache,
                          torch::Tensor slot_mapping) {
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1);
  const int T_ = proj.size(0);
  TORCH_CHECK(heads >= 1 && q_rot_off >= 0 && rot_dim >= 0 &&
              q_rot_off + rot_dim <= q_head && heads * q_head <= kv_off &&
              kv_off + kv_rank + rot_dim <= proj.size(1) && kv_rank >= 1,
              "projection layout out of range");
  TORCH_CHECK(cos_sin.scalar_type() == at::kFloat && cos_sin.is_contiguous() &&
              cos_sin.dim() == 2 && cos_sin.size(0) == T_ &&
              cos_sin.size(1) % 2 == 0);
  const int half = cos_sin.size(1) / 2;
  TORCH_CHECK(2 * half <= rot_dim, "rotary dims exceed the rotated part");
  TORCH_CHECK(w_kv.scalar_type() == at::kFloat && w_kv.is_contiguous() &&
              w_kv.numel() == kv_rank);
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() &&
              cache.scalar_type() == proj.scalar_type() &&
              cache.size(2) >= kv_rank + rot_dim, "pool row too narrow");
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong &&
              slot_mapping.is_contiguous() && slot_mapping.numel() == T_);
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(proj, {
    hipLaunchKernelGGL((latent_rotary_append_kernel<T>), dim3(T_), dim3(256), 0,
                       stream, (T*)proj.data_ptr(), (long)proj.stride(0),
                       (int)heads, (int)q_head, (int)q_rot_off, (int)kv_off,
                       (int)kv_rank, (int)rot_dim, half,
                       w_kv.data_ptr<float>(), (float)eps,
                       cos_sin.data_ptr<float>(), (T*)cache.data_ptr(),
                       (int)cache.size(2), slot_mapping.data_ptr<long>());
  });
}

void head_kv_append(torch::Tensor k, torch::Tensor v, torch::Tensor k_cache,
               torch::Tensor v_cache, torch::Tensor slot_mapping) {
  TORCH_CHECK(k.dim() == 3 && v.dim() == 3 && k.stride(2) == 1 &&
              v.stride(2) == 1 && k.size(0) == v.size(0) &&
              k.size(1) == v.size(1));
  const int T_ = k.size(0), G = k.size(1), D = k.size(2), Dv = v.size(2);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.dim() == 4 && v_cache.is_contiguous() &&
              k_cache.size(1) == G && v_cache.size(1) == G &&
              k_cache.size(3) == D && v_cache.size(3) == Dv &&
              k_cache.size(2) == v_cache.size(2) &&
              k_cache.size(0) == v_cache.size(0), "pool shapes disagree");
  TORCH_CHECK(k_cache.scalar_type() == k.scalar_type() &&
              v_cache.scalar_type() == k.scalar_type() &&
              v.scalar_type() == k.scalar_type());
  TORCH_CHECK(slot_mapping.scalar_type() == at::kLong &&
              slot_mapping.is_contiguous() && slot_mapping.numel() == T_);
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(k, {
    hipLaunchKernelGGL((kv_append_kernel<T>), dim3(T_), dim3(256), 0, stream,
                       (const T*)k.data_ptr(), (long)k.stride(0),
                       (long)k.stride(1), (const T*)v.data_ptr(),
                       (long)v.stride(0), (long)v.stride(1),
                       (T*)k_cache.data_ptr(), (T*)v_cache.data_ptr(),
                       slot_mapping.data_ptr<long>(), G, D, Dv,
                       (int)k_cache.size(2));
  });
}
