// Scaled token embedding plus a hashed bigram embedding (gfx950).
//
//   x[r] = scale * embed[id_r] + bigram[row_r]            (fp32 out)
//   row_r = (mul_prev * id_(r-1) + mul_cur * id_r) mod buckets,
//   row_r = buckets (the table's last row) for a sequence's first token.
//
// The previous id of a step's first row of a sequence is per-sequence state
// (prev_state[slot], int32); a sequence whose first row sits at position 0
// ignores it. Kernel 1 (one workgroup per token row) only READS the state;
// kernel 2 (one thread per sequence) then stores the portion's last id, so
// rows of one sequence that run in different workgroups never race with
// the update.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include "latent_common.h"

namespace {

__device__ __forceinline__ int find_seq(const int* starts, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (starts[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename T>
__global__ __launch_bounds__(256) void bigram_embed_kernel(
    float* __restrict__ x, const long* __restrict__ ids,
    const T* __restrict__ embed, const T* __restrict__ bigram, float scale,
    long mul_prev, long mul_cur, long buckets,
    const int* __restrict__ prev_state, const long* __restrict__ slots,
    const int* __restrict__ seq_lens, const int* __restrict__ q_starts,
    const int* __restrict__ q_lens, int B, int W, long vocab) {
  const int r = blockIdx.x;
  long id = ids[r];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  const T* er = embed + id * W;
  const T* br = nullptr;
  if (bigram != nullptr) {
    int b, off, n;
    if (q_starts) {
      b = find_seq(q_starts, B, r);
      off = r - q_starts[b];
      n = q_lens[b];
    } else {
      b = r; off = 0; n = 1;
    }
    const int pos = seq_lens[b] - n + off;
    long row = buckets;
    if (pos > 0) {
      const long prev = off > 0 ? ids[r - 1] : (long)prev_state[slots[b]];
      row = (prev * mul_prev + id * mul_cur) % buckets;
      if (row < 0) row += buckets;
    }
    br = bigram + row * W;
  }
  float* xr = x + (long)r * W;
  if (W % 4 == 0) {   // table rows then start 4-element aligned
    for (int i = threadIdx.x * 4; i < W; i += 256 * 4) {
      float v[4], b[4] = {0.f, 0.f, 0.f, 0.f};
      ld4(er, i, v);
      if (br) ld4(br, i, b);
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = fmaf(v[j], scale, b[j]);
      st4(xr, i, v);
    }
    return;
  }
  for (int i = threadIdx.x; i < W; i += 256) {
    float v = ldf(er, i) * scale;
    if (br) v += ldf(br, i);
    xr[i] = v;
  }
}

__global__ void bigram_state_kernel(int* __restrict__ prev_state,
                                    const long* __restrict__ ids,
                                    const long* __restrict__ slots,
                                    const int* __restrict__ q_starts,
                                    const int* __restrict__ q_lens, int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  const int n = q_lens ? q_lens[b] : 1;
  if (n <= 0) return;
  const int last = (q_starts ? q_starts[b] : b) + n - 1;
  prev_state[slots[b]] = (int)ids[last];
}

}  // namespace

void bigram_embed(torch::Tensor x, torch::Tensor ids, torch::Tensor embed,
                  c10::optional<torch::Tensor> bigram, double scale,
                  long mul_prev, long mul_cur, long buckets,
                  c10::optional<torch::Tensor> prev_state,
                  torch::Tensor state_slots, torch::Tensor seq_lens,
                  c10::optional<torch::Tensor> query_starts,
                  c10::optional<torch::Tensor> query_lens) {
  TORCH_CHECK(x.scalar_type() == at::kFloat && x.is_contiguous() &&
              x.dim() == 2);
  const int T_ = x.size(0), W = x.size(1);
  TORCH_CHECK(ids.scalar_type() == at::kLong && ids.is_contiguous() &&
              ids.numel() == T_);
  TORCH_CHECK(embed.dim() == 2 && embed.is_contiguous() && embed.size(1) == W);
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  const int B = seq_lens.numel();
  TORCH_CHECK(state_slots.scalar_type() == at::kLong &&
              state_slots.is_contiguous() && state_slots.numel() == B);
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
    TORCH_CHECK(T_ == B, "decode: one row per sequence");
  }
  const void* bp = nullptr;
  int* ps = nullptr;
  if (bigram.has_value()) {
    TORCH_CHECK(bigram->dim() == 2 && bigram->is_contiguous() &&
                bigram->size(1) == W && bigram->size(0) == buckets + 1 &&
                bigram->scalar_type() == embed.scalar_type() && buckets >= 1,
                "bigram table must hold buckets + 1 rows");
    TORCH_CHECK(prev_state.has_value() &&
                prev_state->scalar_type() == at::kInt &&
                prev_state->is_contiguous(),
                "a bigram table needs the int32 previous-token state");
    bp = bigram->data_ptr();
    ps = prev_state->data_ptr<int>();
  }
  if (T_ == 0) return;
  auto stream = at::hip::getCurrentHIPStream();
  LATENT_DISPATCH_T(embed, {
    hipLaunchKernelGGL((bigram_embed_kernel<T>), dim3(T_), dim3(256), 0,
                       stream, x.data_ptr<float>(), ids.data_ptr<long>(),
                       (const T*)embed.data_ptr(), (const T*)bp, (float)scale,
                       mul_prev, mul_cur, buckets, ps,
                       state_slots.data_ptr<long>(), seq_lens.data_ptr<int>(),
                       qs, ql, B, W, (long)embed.size(0));
  });
  if (ps != nullptr)
    hipLaunchKernelGGL(bigram_state_kernel, dim3((B + 63) / 64), dim3(64), 0,
                       stream, ps, ids.data_ptr<long>(),
                       state_slots.data_ptr<long>(), qs, ql, B);
}
