// Masked grouped-query attention over paged per-head K/V pools (gfx950).
//
//   k_cache [P, G, PS, D]   v_cache [P, G, PS, Dv]   (a page holds, per kv
//   head, PS consecutive token rows: one (page, head) block is contiguous)
//   q [T, H, D], out [T, H, Dv]; query head h reads kv head h / (H/G).
//
//   score  = <q, k> * scale;  score <- cap * tanh(score / cap)   (cap > 0)
//            score <- score - r1[h] * ln(1 + r2[h] * (p - j))    (dist given)
//   mask   : causal   j <= p
//            window   j <= p and (p - j < size  or  j < keep)
//            chunk    j <= p and floor(p/size) == floor(j/size)
//   weight : softmax over the visible keys, or sigmoid(score + bias[h])
//            per visible key with no normalization
//   out    = sum_j weight_j v_j  (* sigmoid(gate[t, h]) when a gate is given;
//            a gate of heads * Dv columns gates every output coordinate:
//            * sigmoid(gate[t, h * Dv + e]))
//
// Every query therefore sees at most two key ranges: a kept prefix [0, ns)
// and a main range [lo, p]. Scores, masks, weights and accumulation are
// fp32. The same kernels serve prompt portions (query_starts / query_lens)
// and single decoded tokens (one query per sequence, seq_len <= 0 = pad
// row -> zeros).
//
//   masked_attn_mfma      bf16 MFMA tile kernel. Columns are flattened
//                         (token, head-in-group) pairs of one sequence and
//                         one kv head, 16 per wave, 64 per workgroup, so
//                         the heads of a group share every staged key tile
//                         and a decode step still fills MFMA columns with
//                         heads. It computes S^T = K Q^T and O^T = V^T P^T:
//                         the C layout of S^T (lane = one query column,
//                         4 consecutive keys) IS the B-operand layout of
//                         P^T, so weights go from registers straight into
//                         the second MFMA, softmax statistics are per lane
//                         and only V needs a transposed LDS tile.
//   masked_attn_rowwave   one wave per (query token, head), any element
//                         type: the fp32 path and the fallback for head
//                         sizes the tile kernel does not take.
//
// MFMA fragment maps (v_mfma_f32_16x16x32_bf16): A lane l holds
// A[l%16][(l/16)*8 + j]; B lane l holds B[(l/16)*8 + j][l%16]; C/D lane l
// holds rows (l/16)*4 + r, column l%16.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <algorithm>
#include <cfloat>
#include "latent_common.h"

namespace {

typedef __bf16 bf16v8 __attribute__((ext_vector_type(8)));

constexpr int MK_CAUSAL = 0, MK_WINDOW = 1, MK_CHUNK = 2;

// first key of the main visible range of a query at position p
__device__ __forceinline__ int mask_lo(int p, int kind, int size) {
  if (kind == MK_WINDOW) return max(0, p - size + 1);
  if (kind == MK_CHUNK) return p - p % size;
  return 0;
}

__device__ __forceinline__ float sigmoidf_(float x) {
  return 1.0f / (1.0f + expf(-x));
}

// bf16 tile kernels: hardware exp2 / rcp forms (relative error ~1e-6, far
// below the bf16 rounding of the weights they produce)
__device__ __forceinline__ float fast_exp(float x) { return __expf(x); }
__device__ __forceinline__ float fast_sigmoid(float x) {
  return __fdividef(1.0f, 1.0f + __expf(-x));
}
__device__ __forceinline__ float fast_tanh(float x) {
  return 2.0f * fast_sigmoid(2.0f * x) - 1.0f;
}

// distance bias: r1 * ln(1 + r2 * d), d >= 0
__device__ __forceinline__ float dist_penalty(float r1, float r2, int d) {
  return r1 * log1pf(r2 * (float)max(d, 0));
}
// tile kernels: hardware log2 (the argument is >= 1)
__device__ __forceinline__ float fast_dist_penalty(float r1, float r2, int d) {
  return r1 * 0.6931471805599453f * __log2f(fmaf(r2, (float)max(d, 0), 1.0f));
}

// token position -> (page index in the sequence's table, row in the page);
// page sizes that are powers of two (ps_shift >= 0) avoid the division
__device__ __forceinline__ void page_of(int j, int PS, int ps_shift, int& pg,
                                        int& off) {
  if (ps_shift >= 0) {
    pg = j >> ps_shift;
    off = j & (PS - 1);
  } else {
    pg = j / PS;
    off = j % PS;
  }
}

__device__ __forceinline__ bf16v8 pack_bf16(const float* v) {
  bf16v8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (__bf16)v[e];
  return r;
}

// ------------------------------------------------------------------
// masked_attn_rowwave: one wave per (query token, head)
// ------------------------------------------------------------------
constexpr int RW_MAX_ACC = 8;  // Dv <= 64 * 8

template <typename T>
__global__ __launch_bounds__(64) void masked_attn_rowwave_kernel(
    T* __restrict__ out, long o_ts, long o_hs, const T* __restrict__ q,
    long q_ts, long q_hs, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ page_table, const int* __restrict__ seq_lens,
    const int* __restrict__ q_starts, const int* __restrict__ q_lens,
    float scale, int kind, int size, int keep, int sigmoid_w, float softcap,
    const float* __restrict__ key_bias, const T* __restrict__ gate, long g_ts,
    int gate_elem, const float* __restrict__ dist, int H, int G, int D, int Dv,
    int PS, int max_pages, int vec) {
  extern __shared__ float smem[];
  float* q_s = smem;       // [D]
  float* p_s = smem + D;   // [64]
  const int qi = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
  const int lane = threadIdx.x;
  const int qlen = q_lens ? q_lens[b] : 1;
  if (qi >= qlen) return;
  const int total = seq_lens[b];
  const long rowi = (q_starts ? q_starts[b] : b) + qi;
  T* op = out + rowi * o_ts + h * o_hs;
  if (total <= 0) {  // pad row of a captured decode batch
    for (int i = lane; i < Dv; i += WAVE) stf(op, i, 0.f);
    return;
  }
  const int qpos = total - qlen + qi;
  const int lo = mask_lo(qpos, kind, size);
  const int ns = min(keep, lo);            // kept prefix not in the main range
  const int nvis = ns + qpos - lo + 1;
  const int g = h / (H / G);
  const T* qp = q + rowi * q_ts + h * q_hs;
  for (int i = lane; i < D; i += WAVE) q_s[i] = ldf(qp, i);
  __syncthreads();
  const int* pt = page_table + (long)b * max_pages;
  const float bias = (sigmoid_w && key_bias != nullptr) ? key_bias[h] : 0.f;
  const float r1 = dist ? dist[2 * h] : 0.f, r2 = dist ? dist[2 * h + 1] : 0.f;

  float m = -FLT_MAX, l = 0.f;
  float acc[RW_MAX_ACC];
#pragma unroll
  for (int k = 0; k < RW_MAX_ACC; ++k) acc[k] = 0.f;

  for (int u0 = 0; u0 < nvis; u0 += WAVE) {
    const int u = u0 + lane;
    const bool valid = u < nvis;
    float s = -FLT_MAX;
    if (valid) {
      const int j = u < ns ? u : lo + (u - ns);
      const T* kr = kc + ((((long)pt[j / PS] * G + g) * PS) + j % PS) * D;
      float d = 0.f;
      if (vec) {
        for (int i = 0; i < D; i += 4) {
          float c4[4];
          ld4(kr, i, c4);
          d = fmaf(q_s[i], c4[0], d);
          d = fmaf(q_s[i + 1], c4[1], d);
          d = fmaf(q_s[i + 2], c4[2], d);
          d = fmaf(q_s[i + 3], c4[3], d);
        }
      } else {
        for (int i = 0; i < D; ++i) d = fmaf(q_s[i], ldf(kr, i), d);
      }
      s = d * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      if (dist) s -= dist_penalty(r1, r2, qpos - j);
    }
    float p, alpha = 1.0f;
    if (sigmoid_w) {
      p = valid ? sigmoidf_(s + bias) : 0.f;
    } else {
      const float mn = fmaxf(m, wave_max(s));
      alpha = (m == -FLT_MAX) ? 0.f : expf(m - mn);
      p = valid ? expf(s - mn) : 0.f;
      l = l * alpha + wave_sum(p);
      m = mn;
    }
    p_s[lane] = p;
    __syncthreads();
#pragma unroll
    for (int k = 0; k < RW_MAX_ACC; ++k) acc[k] *= alpha;
    const int n = min(WAVE, nvis - u0);
    for (int jj = 0; jj < n; ++jj) {
      const int ug = u0 + jj;
      const int jg = ug < ns ? ug : lo + (ug - ns);
      const T* vr = vc + ((((long)pt[jg / PS] * G + g) * PS) + jg % PS) * Dv;
      const float pj = p_s[jj];
#pragma unroll
      for (int k = 0; k < RW_MAX_ACC; ++k) {
        const int d = k * WAVE + lane;
        if (d < Dv) acc[k] = fmaf(pj, ldf(vr, d), acc[k]);
      }
    }
    __syncthreads();
  }
  float mul = sigmoid_w ? 1.0f : 1.0f / l;
  if (gate != nullptr && !gate_elem)
    mul *= sigmoidf_(ldf(gate, rowi * g_ts + h));
#pragma unroll
  for (int k = 0; k < RW_MAX_ACC; ++k) {
    const int d = k * WAVE + lane;
    if (d < Dv) {
      float o = acc[k] * mul;
      if (gate != nullptr && gate_elem)
        o *= sigmoidf_(ldf(gate, rowi * g_ts + (long)h * Dv + d));
      stf(op, d, o);
    }
  }
}

// ------------------------------------------------------------------
// masked_attn_mfma: bf16 tile kernel
// ------------------------------------------------------------------
constexpr int KVT = 32;             // keys per staged tile
constexpr int COLS_PER_WAVE = 16;
constexpr int COLS_PER_BLOCK = 64;
constexpr int VT_STRIDE = KVT + 8;  // shorts; one value coordinate's keys

// where key kk of a tile sits in a transposed V row: the 8 keys one lane
// feeds to the second MFMA (4 from each 16-key score block) are contiguous
__device__ __forceinline__ int vt_slot(int kk) {
  return ((kk & 15) >> 2) * 8 + (kk >> 4) * 4 + (kk & 3);
}

// NDB / NVB bound the key size in 32-wide chunks and the value size in
// 16-wide chunks (registers are sized by them); nd <= NDB and nv <= NVB are
// runtime arguments.
template <int NDB, int NVB>
__global__ __launch_bounds__(256) void masked_attn_mfma_kernel(
    short* __restrict__ out, long o_ts, long o_hs, const short* __restrict__ q,
    long q_ts, long q_hs, const short* __restrict__ kc,
    const short* __restrict__ vc, const int* __restrict__ page_table,
    const int* __restrict__ seq_lens, const int* __restrict__ q_starts,
    const int* __restrict__ q_lens, float scale, int kind, int size, int keep,
    int sigmoid_w, float softcap, const float* __restrict__ key_bias,
    const short* __restrict__ gate, long g_ts, int gate_elem,
    const float* __restrict__ dist, int H, int G, int nd, int nv, int PS,
    int max_pages, int ps_shift) {
  extern __shared__ __attribute__((aligned(16))) short lds[];
  constexpr int KL = NDB / 2;              // 16-byte K loads per thread
  const int D = nd * 32, Dv = nv * 16;
  const int KS = D + 8;                    // padded key row stride
  short* k_lds = lds;                      // [KVT][KS]
  short* vt_lds = lds + KVT * KS;          // [Dv][VT_STRIDE]

  const int b = blockIdx.y, g = blockIdx.z;
  const int R = H / G;
  const int qlen = q_lens ? q_lens[b] : 1;
  const int ncols = qlen * R;
  const int c0 = blockIdx.x * COLS_PER_BLOCK;
  if (c0 >= ncols) return;
  const int total = seq_lens[b];
  const long row_base = q_starts ? q_starts[b] : b;
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wid = tid / WAVE;
  const int l16 = lane % 16, lg = lane / 16;

  if (total <= 0) {  // pad row of a captured decode batch: zeros
    const int c1 = min(c0 + COLS_PER_BLOCK, ncols);
    for (int i = tid; i < (c1 - c0) * Dv; i += 256) {
      const int c = c0 + i / Dv, e = i % Dv;
      out[(row_base + c / R) * o_ts + (g * R + c % R) * o_hs + e] = 0;
    }
    return;
  }
  const int ctx = total - qlen;
  const int* pt = page_table + (long)b * max_pages;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;

  // ---- key tiles of this block: kept prefix + main range of its columns
  const int c_last = min(c0 + COLS_PER_BLOCK, ncols) - 1;
  const int bq_first = ctx + c0 / R, bq_last = ctx + c_last / R;
  const int kt_end = bq_last / KVT + 1;
  const int sink_tiles = (keep + KVT - 1) / KVT;
  const int main_first = mask_lo(bq_first, kind, size) / KVT;
  auto next_tile = [&](int kt) {
    ++kt;
    return (kt >= sink_tiles && kt < main_first) ? main_first : kt;
  };

  // ---- this wave's columns
  const int cw0 = c0 + wid * COLS_PER_WAVE;
  const bool wave_live = cw0 < ncols;
  const int col = cw0 + l16;
  const bool col_ok = col < ncols;
  const int qi = col_ok ? col / R : 0;
  const int h = g * R + (col_ok ? col % R : 0);
  const int qpos = col_ok ? ctx + qi : -1;     // -1: nothing visible
  const int lo = col_ok ? mask_lo(qpos, kind, size) : 0;
  const int wq_first = ctx + min(cw0, ncols - 1) / R;
  const int wq_last = ctx + min(cw0 + COLS_PER_WAVE - 1, ncols - 1) / R;
  const int w_lo = mask_lo(wq_first, kind, size);
  const float bias = (sigmoid_w && key_bias != nullptr) ? key_bias[h] : 0.f;
  const float r1 = dist ? dist[2 * h] : 0.f, r2 = dist ? dist[2 * h + 1] : 0.f;

  // Q^T as the first MFMA's B operand: lane -> column l16, dims c*32+lg*8..
  bf16v8 qf[NDB];
  {
    const short* qp = q + (row_base + qi) * q_ts + (long)h * q_hs;
#pragma unroll
    for (int c = 0; c < NDB; ++c) {
      if (c < nd && col_ok)
        qf[c] = *reinterpret_cast<const bf16v8*>(qp + c * 32 + lg * 8);
      else
        qf[c] = bf16v8{};
    }
  }

  f32x4 o[NVB];
#pragma unroll
  for (int i = 0; i < NVB; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -FLT_MAX, l = 0.f;

  // ---- staging: global -> registers -> LDS
  const int kchunks = D / 8, vchunks = Dv / 8;     // 16-byte chunks per row
  // V: one unit = 4 consecutive keys x one 8-value chunk, so that the
  // transposed tile is written 4 keys (8 bytes) at a time; <= 256 units
  bf16x8 kreg[KL], vreg[4];
  const bool v_unit = tid < 8 * vchunks;
  const int v_kq = tid / vchunks, v_ch = tid % vchunks;
  auto load_tile = [&](int kt) {
    const int t0 = kt * KVT;
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const int idx = tid + i * 256;
      kreg[i] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      if (idx < KVT * kchunks) {
        const int kk = idx / kchunks, ch = idx % kchunks;
        const int j = t0 + kk;
        if (j < total) {
          int pg, off;
          page_of(j, PS, ps_shift, pg, off);
          const long row = ((long)pt[pg] * G + g) * PS + off;
          kreg[i] = *reinterpret_cast<const bf16x8*>(kc + row * D + ch * 8);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      vreg[r] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      const int j = t0 + v_kq * 4 + r;
      if (v_unit && j < total) {
        int pg, off;
        page_of(j, PS, ps_shift, pg, off);
        const long row = ((long)pt[pg] * G + g) * PS + off;
        vreg[r] = *reinterpret_cast<const bf16x8*>(vc + row * Dv + v_ch * 8);
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const int idx = tid + i * 256;
      if (idx < KVT * kchunks) {
        const int kk = idx / kchunks, ch = idx % kchunks;
        *reinterpret_cast<bf16x8*>(k_lds + kk * KS + ch * 8) = kreg[i];
      }
    }
    if (v_unit) {
      const int slot = vt_slot(v_kq * 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const bf16x4 w4 = {vreg[0][e], vreg[1][e], vreg[2][e], vreg[3][e]};
        *reinterpret_cast<bf16x4*>(vt_lds + (v_ch * 8 + e) * VT_STRIDE + slot) =
            w4;
      }
    }
  };

  int kt = next_tile(-1);
  load_tile(kt);
  while (true) {
    __syncthreads();          // every wave is done with the previous tile
    store_tile();
    __syncthreads();
    const int nkt = next_tile(kt);
    const bool more = nkt < kt_end;
    if (more) load_tile(nkt);  // in flight while this tile is computed
    const int t0 = kt * KVT;
    if (wave_live && t0 <= wq_last && (t0 + KVT > w_lo || t0 < keep)) {
      // ---- S^T = K Q^T for two 16-key blocks
      f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
      for (int c = 0; c < NDB; ++c) {
        if (c < nd) {
          const bf16v8 a0 = *reinterpret_cast<const bf16v8*>(
              k_lds + l16 * KS + c * 32 + lg * 8);
          const bf16v8 a1 = *reinterpret_cast<const bf16v8*>(
              k_lds + (16 + l16) * KS + c * 32 + lg * 8);
          s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[c], s0, 0, 0, 0);
          s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qf[c], s1, 0, 0, 0);
        }
      }
      // lane holds, for its column, keys t0 + lg*4 + r and t0 + 16 + lg*4 + r
      float sv[8];
      bool vis[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sv[r] = s0[r];
        sv[4 + r] = s1[r];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = t0 + (e >> 2) * 16 + lg * 4 + (e & 3);
        vis[e] = j <= qpos && (j >= lo || j < keep);
        float s = sv[e] * scale;
        if (softcap > 0.f) s = softcap * fast_tanh(s * inv_cap);
        if (dist) s -= fast_dist_penalty(r1, r2, qpos - j);
        sv[e] = s;
      }
      float pv[8];
      if (sigmoid_w) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          pv[e] = vis[e] ? fast_sigmoid(sv[e] + bias) : 0.f;
      } else {
        float tm = -FLT_MAX;
#pragma unroll
        for (int e = 0; e < 8; ++e) tm = fmaxf(tm, vis[e] ? sv[e] : -FLT_MAX);
        tm = fmaxf(tm, __shfl_xor(tm, 16, WAVE));
        tm = fmaxf(tm, __shfl_xor(tm, 32, WAVE));
        const float mn = fmaxf(m, tm);
        const float alpha = (m == -FLT_MAX) ? 0.f : fast_exp(m - mn);
        float ts = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pv[e] = vis[e] ? fast_exp(sv[e] - mn) : 0.f;
          ts += pv[e];
        }
        ts += __shfl_xor(ts, 16, WAVE);
        ts += __shfl_xor(ts, 32, WAVE);
        l = l * alpha + ts;
        m = mn;
#pragma unroll
        for (int i = 0; i < NVB; ++i)
          if (i < nv) o[i] *= alpha;
      }
      // P^T as the second MFMA's B operand, straight from registers
      const bf16v8 pf = pack_bf16(pv);
      // ---- O^T += V^T P^T
#pragma unroll
      for (int i = 0; i < NVB; ++i) {
        if (i < nv) {
          const bf16v8 af = *reinterpret_cast<const bf16v8*>(
              vt_lds + (i * 16 + l16) * VT_STRIDE + lg * 8);
          o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, pf, o[i], 0, 0, 0);
        }
      }
    }
    if (!more) break;
    kt = nkt;
  }

  // ---- epilogue: lane holds O^T[i*16 + lg*4 + r][column]
  if (!col_ok) return;
  float mul = sigmoid_w ? 1.0f : 1.0f / l;
  if (gate != nullptr && !gate_elem)
    mul *= sigmoidf_(bits2f(gate[(row_base + qi) * g_ts + h]));
  const short* ge = (gate != nullptr && gate_elem)
                        ? gate + (row_base + qi) * g_ts + (long)h * (nv * 16)
                        : nullptr;
  short* op = out + (row_base + qi) * o_ts + (long)h * o_hs;
#pragma unroll
  for (int i = 0; i < NVB; ++i) {
    if (i < nv) {
      bf16x4 t;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float v = o[i][r] * mul;
        if (ge) v *= sigmoidf_(bits2f(ge[i * 16 + lg * 4 + r]));
        t[r] = f2bits(v);
      }
      *reinterpret_cast<bf16x4*>(op + i * 16 + lg * 4) = t;
    }
  }
}

// ------------------------------------------------------------------
// masked_attn_decode: one new token per sequence, bf16, H/G <= 16
// ------------------------------------------------------------------
// A decode step has one query position per sequence: nothing amortizes a
// block-wide staged tile and barriers would idle three waves of four. Here
// every WAVE owns whole 32-key tiles: it loads the K fragments of its tile
// straight from HBM into MFMA A operands, transposes V through a private
// LDS patch (wave-local synchronization only) and keeps its own (m, l, O)
// for the group's heads (columns of the MFMA). The visible tiles of the
// sequence — kept prefix first, then the main range — are dealt round-robin
// to the 4 waves of n_splits workgroups (grid.x), so a long window spreads
// over the chip. Waves are merged through LDS; with n_splits > 1 each
// workgroup writes an un-normalized partial and masked_attn_combine
// finishes. Latency is hidden by occupancy (several workgroups per CU, each
// wave with a 32-key tile in flight), not by software pipelining.

__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int NDB, int NVB>
__global__ __launch_bounds__(256) void masked_attn_decode_kernel(
    short* __restrict__ out, long o_ts, long o_hs, const short* __restrict__ q,
    long q_ts, long q_hs, const short* __restrict__ kc,
    const short* __restrict__ vc, const int* __restrict__ page_table,
    const int* __restrict__ seq_lens, float scale, int kind, int size, int keep,
    int sigmoid_w, float softcap, const float* __restrict__ key_bias,
    const short* __restrict__ gate, long g_ts, int gate_elem,
    const float* __restrict__ dist, int H, int G, int nd, int nv, int PS,
    int max_pages, int ps_shift, float* __restrict__ part_o,
    float* __restrict__ part_ml, int n_splits) {
  extern __shared__ __attribute__((aligned(16))) short lds[];
  const int D = nd * 32, Dv = nv * 16;
  const int split = blockIdx.x, b = blockIdx.y, g = blockIdx.z;
  const int R = H / G;
  const int tid = threadIdx.x;
  const int lane = tid % WAVE, wid = tid / WAVE;
  const int l16 = lane % 16, lg = lane / 16;
  const int total = seq_lens[b];
  const long part_base = ((long)(b * G + g) * n_splits + split) * R;

  if (total <= 0) {  // pad row of a captured batch
    for (int i = tid; i < R * Dv; i += 256) {
      const int c = i / Dv, e = i % Dv;
      if (n_splits == 1) {
        out[(long)b * o_ts + (long)(g * R + c) * o_hs + e] = 0;
      } else {
        part_o[(part_base + c) * Dv + e] = 0.f;
        if (e == 0) {
          part_ml[(part_base + c) * 2] = -FLT_MAX;
          part_ml[(part_base + c) * 2 + 1] = 0.f;
        }
      }
    }
    return;
  }
  const int qpos = total - 1;
  const int lo = mask_lo(qpos, kind, size);
  const int* pt = page_table + (long)b * max_pages;
  const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
  const int kt_end = qpos / KVT + 1;
  const int main_first = lo / KVT;
  const int n_sink = min((keep + KVT - 1) / KVT, main_first);
  const int n_vt = n_sink + kt_end - main_first;

  const bool col_ok = l16 < R;
  const int h = g * R + (col_ok ? l16 : 0);
  const float bias = (sigmoid_w && key_bias != nullptr) ? key_bias[h] : 0.f;
  const float r1 = dist ? dist[2 * h] : 0.f, r2 = dist ? dist[2 * h + 1] : 0.f;
  const int cq = col_ok ? qpos : -1;

  bf16v8 qf[NDB];
  {
    const short* qp = q + (long)b * q_ts + (long)h * q_hs;
#pragma unroll
    for (int c = 0; c < NDB; ++c) {
      if (c < nd && col_ok)
        qf[c] = *reinterpret_cast<const bf16v8*>(qp + c * 32 + lg * 8);
      else
        qf[c] = bf16v8{};
    }
  }
  f32x4 o[NVB];
#pragma unroll
  for (int i = 0; i < NVB; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -FLT_MAX, l = 0.f;

  // this wave's V^T patch: [Dv][32 keys] with no padding (4 workgroups of
  // 4 waves fit a CU's LDS); the 16-byte unit inside a row is XOR-ed with
  // bits of the row so the A-fragment reads of 16 rows spread over all banks
  short* vt = lds + (size_t)wid * Dv * KVT;
  const int vchunks = Dv / 8;                       // = 2 * nv
  // this lane's (key quad, chunk) units of a tile's V rows
  constexpr int VU = (NVB + 3) / 4;
  int u_kq[VU], u_ch[VU];
  bool u_ok[VU];
#pragma unroll
  for (int it = 0; it < VU; ++it) {
    const int u = lane + it * WAVE;
    u_ok[it] = u < 8 * vchunks;
    u_kq[it] = u / vchunks;
    u_ch[it] = u % vchunks;
  }

  for (int v = split * 4 + wid; v < n_vt; v += 4 * n_splits) {
    const int kt = v < n_sink ? v : main_first + (v - n_sink);
    const int t0 = kt * KVT;
    // K fragments: lane -> key l16 (+16), dims c*32 + lg*8 ..
    bf16v8 ka[2][NDB];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int j = t0 + kb * 16 + l16;
      const bool ok = j < total;
      int pg, off;
      page_of(ok ? j : 0, PS, ps_shift, pg, off);
      const long row = ((long)pt[pg] * G + g) * PS + off;
      const short* kr = kc + row * D + lg * 8;
#pragma unroll
      for (int c = 0; c < NDB; ++c) {
        if (c < nd && ok)
          ka[kb][c] = *reinterpret_cast<const bf16v8*>(kr + c * 32);
        else
          ka[kb][c] = bf16v8{};
      }
    }
    // V: unit = 4 consecutive keys x one 8-value chunk (16 bytes per load)
    bf16x8 vr[VU][4];
#pragma unroll
    for (int it = 0; it < VU; ++it) {
      const int jq = t0 + u_kq[it] * 4;
      if ((PS & 3) == 0) {       // the four keys of a unit share a page
        int pg, off;
        page_of(jq < total ? jq : 0, PS, ps_shift, pg, off);
        const short* vrow =
            vc + (((long)pt[pg] * G + g) * PS + off) * Dv + u_ch[it] * 8;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          vr[it][r] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
          if (u_ok[it] && jq + r < total)
            vr[it][r] = *reinterpret_cast<const bf16x8*>(vrow + r * Dv);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          vr[it][r] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
          const int j = jq + r;
          if (u_ok[it] && j < total) {
            int pg, off;
            page_of(j, PS, ps_shift, pg, off);
            const long row = ((long)pt[pg] * G + g) * PS + off;
            vr[it][r] = *reinterpret_cast<const bf16x8*>(
                vc + row * Dv + u_ch[it] * 8);
          }
        }
      }
    }
    wave_lds_sync();   // the previous tile's reads of the patch are done
#pragma unroll
    for (int it = 0; it < VU; ++it) {
      if (u_ok[it]) {
        const int slot = vt_slot(u_kq[it] * 4);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const bf16x4 w4 = {vr[it][0][e], vr[it][1][e], vr[it][2][e],
                             vr[it][3][e]};
          const int row = u_ch[it] * 8 + e;
          *reinterpret_cast<bf16x4*>(
              vt + row * KVT + (((slot >> 3) ^ ((row >> 2) & 3)) << 3) +
              (slot & 7)) = w4;
        }
      }
    }
    wave_lds_sync();
    f32x4 s0 = f32x4{0.f, 0.f, 0.f, 0.f}, s1 = s0;
#pragma unroll
    for (int c = 0; c < NDB; ++c) {
      if (c < nd) {
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[0][c], qf[c], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[1][c], qf[c], s1, 0, 0, 0);
      }
    }
    float sv[8], pv[8];
    bool vis[8];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      sv[r] = s0[r];
      sv[4 + r] = s1[r];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int j = t0 + (e >> 2) * 16 + lg * 4 + (e & 3);
      vis[e] = j <= cq && (j >= lo || j < keep);
      float s = sv[e] * scale;
      if (softcap > 0.f) s = softcap * fast_tanh(s * inv_cap);
      if (dist) s -= fast_dist_penalty(r1, r2, qpos - j);
      sv[e] = s;
    }
    if (sigmoid_w) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        pv[e] = vis[e] ? fast_sigmoid(sv[e] + bias) : 0.f;
    } else {
      float tm = -FLT_MAX;
#pragma unroll
      for (int e = 0; e < 8; ++e) tm = fmaxf(tm, vis[e] ? sv[e] : -FLT_MAX);
      tm = fmaxf(tm, __shfl_xor(tm, 16, WAVE));
      tm = fmaxf(tm, __shfl_xor(tm, 32, WAVE));
      const float mn = fmaxf(m, tm);
      const float alpha = (m == -FLT_MAX) ? 0.f : fast_exp(m - mn);
      float ts = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pv[e] = vis[e] ? fast_exp(sv[e] - mn) : 0.f;
        ts += pv[e];
      }
      ts += __shfl_xor(ts, 16, WAVE);
      ts += __shfl_xor(ts, 32, WAVE);
      l = l * alpha + ts;
      m = mn;
#pragma unroll
      for (int i = 0; i < NVB; ++i)
        if (i < nv) o[i] *= alpha;
    }
    const bf16v8 pf = pack_bf16(pv);
#pragma unroll
    for (int i = 0; i < NVB; ++i) {
      if (i < nv) {
        const int row = i * 16 + l16;
        const bf16v8 af = *reinterpret_cast<const bf16v8*>(
            vt + row * KVT + ((lg ^ ((row >> 2) & 3)) << 3));
        o[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, pf, o[i], 0, 0, 0);
      }
    }
  }

  // ---- merge the 4 waves through LDS: fo[wave][e][col], fml[wave][col][2]
  __syncthreads();
  float* fo = reinterpret_cast<float*>(lds);
  float* fml = fo + 4 * Dv * 16;
#pragma unroll
  for (int i = 0; i < NVB; ++i) {
    if (i < nv) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        fo[(wid * Dv + i * 16 + lg * 4 + r) * 16 + l16] = o[i][r];
    }
  }
  if (lg == 0) {
    fml[(wid * 16 + l16) * 2] = m;
    fml[(wid * 16 + l16) * 2 + 1] = l;
  }
  __syncthreads();
  for (int i = tid; i < R * Dv; i += 256) {
    const int c = i / Dv, e = i % Dv;
    float M = -FLT_MAX;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, fml[(w * 16 + c) * 2]);
    float L = 0.f, O = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f =
          sigmoid_w ? 1.0f : expf(fml[(w * 16 + c) * 2] - M);
      L = fmaf(fml[(w * 16 + c) * 2 + 1], f, L);
      O = fmaf(fo[(w * Dv + e) * 16 + c], f, O);
    }
    if (n_splits == 1) {
      float mul = sigmoid_w ? 1.0f : 1.0f / L;
      if (gate != nullptr)
        mul *= sigmoidf_(bits2f(
            gate[(long)b * g_ts +
                 (gate_elem ? (long)(g * R + c) * Dv + e : (long)(g * R + c))]));
      out[(long)b * o_ts + (long)(g * R + c) * o_hs + e] = f2bits(O * mul);
    } else {
      part_o[(part_base + c) * Dv + e] = O;
      if (e == 0) {
        part_ml[(part_base + c) * 2] = M;
        part_ml[(part_base + c) * 2 + 1] = L;
      }
    }
  }
}

// merge the n_splits partials of every (sequence, head): grid (B, H)
__global__ __launch_bounds__(64) void masked_attn_combine_kernel(
    short* __restrict__ out, long o_ts, long o_hs,
    const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const short* __restrict__ gate, long g_ts, int gate_elem, int sigmoid_w,
    int H, int G, int Dv, int n_splits) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int R = H / G, g = h / R, c = h % R;
  const long base = (long)(b * G + g) * n_splits;
  float M = -FLT_MAX;
  for (int s = 0; s < n_splits; ++s)
    M = fmaxf(M, part_ml[((base + s) * R + c) * 2]);
  float L = 0.f;
  for (int s = 0; s < n_splits; ++s) {
    const float f =
        sigmoid_w ? 1.0f : expf(part_ml[((base + s) * R + c) * 2] - M);
    L = fmaf(part_ml[((base + s) * R + c) * 2 + 1], f, L);
  }
  float mul = sigmoid_w ? 1.0f : (L > 0.f ? 1.0f / L : 0.f);
  if (gate != nullptr && !gate_elem)
    mul *= sigmoidf_(bits2f(gate[(long)b * g_ts + h]));
  for (int e = threadIdx.x; e < Dv; e += WAVE) {
    float O = 0.f;
    for (int s = 0; s < n_splits; ++s) {
      const float f =
          sigmoid_w ? 1.0f : expf(part_ml[((base + s) * R + c) * 2] - M);
      O = fmaf(part_o[((base + s) * R + c) * Dv + e], f, O);
    }
    if (gate != nullptr && gate_elem)
      O *= sigmoidf_(bits2f(gate[(long)b * g_ts + (long)h * Dv + e]));
    out[(long)b * o_ts + (long)h * o_hs + e] = f2bits(O * mul);
  }
}

bool aligned16(const void* p) {
  return reinterpret_cast<uintptr_t>(p) % 16 == 0;
}

}  // namespace

void masked_attention(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
                      torch::Tensor v_cache, torch::Tensor page_table,
                      torch::Tensor seq_lens,
                      c10::optional<torch::Tensor> query_starts,
                      c10::optional<torch::Tensor> query_lens, double scale,
                      long mask_kind, long mask_size, long keep_first,
                      bool sigmoid_weights, double softcap,
                      c10::optional<torch::Tensor> key_bias,
                      c10::optional<torch::Tensor> head_gate, long max_qlen,
                      bool force_simple, long splits,
                      c10::optional<torch::Tensor> dist_bias) {
  TORCH_CHECK(q.dim() == 3 && out.dim() == 3 && q.stride(2) == 1 &&
              out.stride(2) == 1);
  const int T_ = q.size(0), H = q.size(1), D = q.size(2), Dv = out.size(2);
  TORCH_CHECK(out.size(0) == T_ && out.size(1) == H);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() &&
              v_cache.dim() == 4 && v_cache.is_contiguous());
  const int G = k_cache.size(1), PS = k_cache.size(2);
  TORCH_CHECK(k_cache.size(3) == D && v_cache.size(3) == Dv &&
              v_cache.size(1) == G && v_cache.size(2) == PS &&
              v_cache.size(0) == k_cache.size(0), "pool shapes disagree");
  TORCH_CHECK(G >= 1 && H % G == 0, "heads % kv_heads != 0");
  TORCH_CHECK(q.scalar_type() == out.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type(),
              "q, out and the pools share one element type");
  TORCH_CHECK(page_table.scalar_type() == at::kInt && page_table.dim() == 2 &&
              page_table.is_contiguous());
  TORCH_CHECK(seq_lens.scalar_type() == at::kInt && seq_lens.is_contiguous());
  const int B = seq_lens.numel(), max_pages = page_table.size(1);
  TORCH_CHECK(page_table.size(0) >= B);
  TORCH_CHECK(mask_kind >= MK_CAUSAL && mask_kind <= MK_CHUNK);
  TORCH_CHECK(mask_kind == MK_CAUSAL || mask_size >= 1, "mask size < 1");
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
    TORCH_CHECK(max_qlen >= 1, "max_qlen must be given for prompt portions");
  } else {
    TORCH_CHECK(T_ == B, "decode: one query per sequence");
    max_qlen = 1;
  }
  const float* kb = nullptr;
  if (key_bias.has_value()) {
    TORCH_CHECK(key_bias->scalar_type() == at::kFloat &&
                key_bias->numel() == H && key_bias->is_contiguous());
    kb = key_bias->data_ptr<float>();
  }
  long g_ts = 0;
  int gate_elem = 0;   // 1: the gate has one column per output coordinate
  if (head_gate.has_value()) {
    TORCH_CHECK(head_gate->dim() == 2 && head_gate->size(0) == T_ &&
                (head_gate->size(1) == H ||
                 head_gate->size(1) == (long)H * Dv) &&
                head_gate->stride(1) == 1 &&
                head_gate->scalar_type() == q.scalar_type(),
                "gate is [tokens, heads] or [tokens, heads * value size]");
    g_ts = head_gate->stride(0);
    gate_elem = head_gate->size(1) != H ? 1 : 0;
  }
  const float* db = nullptr;
  if (dist_bias.has_value()) {
    TORCH_CHECK(dist_bias->scalar_type() == at::kFloat &&
                dist_bias->numel() == 2 * H && dist_bias->is_contiguous(),
                "dist_bias is fp32 [heads, 2]");
    db = dist_bias->data_ptr<float>();
  }
  if (T_ == 0 || B == 0) return;
  const int keep = mask_kind == MK_WINDOW ? (int)keep_first : 0;
  auto stream = at::hip::getCurrentHIPStream();
  const int R = H / G;

  const bool mfma_ok =
      q.scalar_type() == at::kBFloat16 && !force_simple && D % 32 == 0 &&
      D <= 256 && Dv % 16 == 0 && Dv <= 256 && q.stride(0) % 8 == 0 &&
      q.stride(1) % 8 == 0 && out.stride(0) % 4 == 0 && out.stride(1) % 4 == 0 &&
      aligned16(q.data_ptr()) && aligned16(out.data_ptr()) &&
      aligned16(k_cache.data_ptr()) && aligned16(v_cache.data_ptr());
  if (mfma_ok) {
    const int nd = D / 32, nv = Dv / 16;
    int ps_shift = -1;
    if ((PS & (PS - 1)) == 0)
      for (ps_shift = 0; (1 << ps_shift) < PS; ++ps_shift) {}
    const short* gp =
        head_gate.has_value() ? (const short*)head_gate->data_ptr() : nullptr;
    if (!query_starts.has_value() && R <= 16) {
      // decode: tiles dealt to waves; split long key ranges over workgroups
      long bound = (long)max_pages * PS;           // keys a query can see
      if (mask_kind != MK_CAUSAL) bound = std::min(bound, mask_size + keep + 31L);
      const long tiles = (bound + KVT - 1) / KVT + 1;
      long n_splits = splits > 0 ? splits : (1024 + (long)B * G - 1) / ((long)B * G);
      n_splits = std::max(1L, std::min(n_splits, std::max(1L, tiles / 4)));
      n_splits = std::min(n_splits, 64L);
      torch::Tensor po, pml;
      float* pop = nullptr;
      float* pmlp = nullptr;
      if (n_splits > 1) {
        auto opts = torch::TensorOptions().dtype(torch::kFloat).device(q.device());
        po = torch::empty({(long)B * G * n_splits * R * Dv}, opts);
        pml = torch::empty({(long)B * G * n_splits * R * 2}, opts);
        pop = po.data_ptr<float>();
        pmlp = pml.data_ptr<float>();
      }
      const dim3 dgrid((unsigned)n_splits, B, G);
      const size_t dlds = (size_t)4 * Dv * KVT * 2 + 512;
#define LAUNCH_DECODE(NDB_, NVB_)                                             \
  hipLaunchKernelGGL((masked_attn_decode_kernel<NDB_, NVB_>), dgrid,          \
                     dim3(256), dlds, stream, (short*)out.data_ptr(),         \
                     (long)out.stride(0), (long)out.stride(1),                \
                     (const short*)q.data_ptr(), (long)q.stride(0),           \
                     (long)q.stride(1), (const short*)k_cache.data_ptr(),     \
                     (const short*)v_cache.data_ptr(),                        \
                     page_table.data_ptr<int>(), seq_lens.data_ptr<int>(),    \
                     (float)scale, (int)mask_kind, (int)mask_size, keep,      \
                     sigmoid_weights ? 1 : 0, (float)softcap, kb, gp, g_ts,   \
                     gate_elem, db, H, G, nd, nv, PS, max_pages, ps_shift,    \
                     pop, pmlp, (int)n_splits)
      if (nd <= 4 && nv <= 4) {
        LAUNCH_DECODE(4, 4);
      } else if (nd <= 4 && nv <= 8) {
        LAUNCH_DECODE(4, 8);
      } else {
        LAUNCH_DECODE(8, 16);
      }
#undef LAUNCH_DECODE
      if (n_splits > 1) {
        hipLaunchKernelGGL(masked_attn_combine_kernel, dim3(B, H), dim3(64), 0,
                           stream, (short*)out.data_ptr(), (long)out.stride(0),
                           (long)out.stride(1), pop, pmlp, gp, g_ts, gate_elem,
                           sigmoid_weights ? 1 : 0, H, G, Dv, (int)n_splits);
      }
      return;
    }
    const dim3 grid((unsigned)(((long)max_qlen * R + COLS_PER_BLOCK - 1) /
                               COLS_PER_BLOCK), B, G);
    const size_t lds = ((size_t)KVT * (D + 8) + (size_t)Dv * VT_STRIDE) * 2;
#define LAUNCH_MFMA(NDB_, NVB_)                                               \
  hipLaunchKernelGGL((masked_attn_mfma_kernel<NDB_, NVB_>), grid, dim3(256),  \
                     lds, stream, (short*)out.data_ptr(),                     \
                     (long)out.stride(0), (long)out.stride(1),                \
                     (const short*)q.data_ptr(), (long)q.stride(0),           \
                     (long)q.stride(1), (const short*)k_cache.data_ptr(),     \
                     (const short*)v_cache.data_ptr(),                        \
                     page_table.data_ptr<int>(), seq_lens.data_ptr<int>(), qs, \
                     ql, (float)scale, (int)mask_kind, (int)mask_size, keep,  \
                     sigmoid_weights ? 1 : 0, (float)softcap, kb, gp, g_ts,   \
                     gate_elem, db, H, G, nd, nv, PS, max_pages, ps_shift)
    if (nd <= 4 && nv <= 4) {
      LAUNCH_MFMA(4, 4);
    } else if (nd <= 4 && nv <= 8) {
      LAUNCH_MFMA(4, 8);
    } else {
      LAUNCH_MFMA(8, 16);
    }
#undef LAUNCH_MFMA
    return;
  }

  TORCH_CHECK(Dv <= WAVE * RW_MAX_ACC, "value size above ", WAVE * RW_MAX_ACC);
  const size_t smem = (size_t)(D + WAVE) * sizeof(float);
  TORCH_CHECK(smem <= 64 * 1024, "head size too large");
  const dim3 grid((unsigned)max_qlen, B, H);
  LATENT_DISPATCH_T(q, {
    const int vec = (D % 4 == 0) && aligned16(k_cache.data_ptr());
    const T* gp =
        head_gate.has_value() ? (const T*)head_gate->data_ptr() : nullptr;
    hipLaunchKernelGGL(
        masked_attn_rowwave_kernel<T>, grid, dim3(64), smem, stream,
        (T*)out.data_ptr(), (long)out.stride(0), (long)out.stride(1),
        (const T*)q.data_ptr(), (long)q.stride(0), (long)q.stride(1),
        (const T*)k_cache.data_ptr(), (const T*)v_cache.data_ptr(),
        page_table.data_ptr<int>(), seq_lens.data_ptr<int>(), qs, ql,
        (float)scale, (int)mask_kind, (int)mask_size, keep,
        sigmoid_weights ? 1 : 0, (float)softcap, kb, gp, g_ts, gate_elem, db, H,
        G, D, Dv, PS, max_pages, vec);
  });
}
