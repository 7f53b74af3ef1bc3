"""ops — dispatch layer over the gfx950 HIP kernels.

Policy (the driver's "native code not loaded" check depends on this):
  * On a CUDA/ROCm device: the in-tree HIP extension (_hip_ops.so) is
    REQUIRED. If it is missing or fails to import, GPU ops raise
    RuntimeError — there is no silent eager fallback on a GPU box.
  * On CPU: the fp32 torch references (ops.reference) run, so the engine
    and control plane are testable without a GPU.

Build the extension with `python -m agentainer_amd.ops.build` (or via
__graft_entry__.build()).
"""

from __future__ import annotations

import os
from typing import Optional

import torch

from . import reference

_hip = None
_hip_err: Optional[str] = None


def _load_hip():
    global _hip, _hip_err
    if _hip is not None or _hip_err is not None:
        return _hip
    so = os.path.join(os.path.dirname(__file__), "_hip_ops.so")
    if not os.path.exists(so):
        _hip_err = f"HIP extension not built ({so} missing); run python -m agentainer_amd.ops.build"
        return None
    try:
        import importlib.util

        spec = importlib.util.spec_from_file_location("agentainer_amd.ops._hip_ops", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _hip = mod
    except Exception as exc:  # noqa: BLE001
        _hip_err = f"HIP extension failed to load: {exc}"
    return _hip


def hip_available() -> bool:
    return _load_hip() is not None


def _dispatch(name: str, *tensors: torch.Tensor):
    """Return the HIP module if the leading tensor is on GPU, else None.
    On GPU with no extension: fail loudly (never a silent fallback)."""
    if tensors[0].is_cuda:
        mod = _load_hip()
        if mod is None:
            raise RuntimeError(
                f"op {name!r} on GPU requires the gfx950 HIP extension: {_hip_err}")
        return mod
    return None


def rmsnorm(out, x, w, eps: float = 1e-5):
    mod = _dispatch("rmsnorm", x)
    if mod:
        mod.rmsnorm(out, x, w, float(eps))
    else:
        reference.rmsnorm(out, x, w, eps)
    return out


def fused_add_rmsnorm(out, x, residual, w, eps: float = 1e-5):
    mod = _dispatch("fused_add_rmsnorm", x)
    if mod:
        mod.fused_add_rmsnorm(out, x, residual, w, float(eps))
    else:
        reference.fused_add_rmsnorm(out, x, residual, w, eps)
    return out


def silu_mul(out, gate, up):
    mod = _dispatch("silu_mul", gate)
    if mod:
        mod.silu_mul(out, gate, up)
    else:
        reference.silu_mul(out, gate, up)
    return out


make_cos_sin_table = reference.make_cos_sin_table


def rope_inplace(q, k, cos_sin, positions):
    mod = _dispatch("rope_inplace", q)
    if mod:
        mod.rope_inplace(q, k, cos_sin, positions)
    else:
        reference.rope_inplace(q, k, cos_sin, positions)


def rope_append(q, k, v, k_cache, v_cache, cos_sin, positions, slot_mapping):
    """Fused rope_inplace(q,k) + kv_append(k,v). CPU falls back to the two
    reference ops."""
    mod = _dispatch("rope_append", q)
    if mod:
        mod.rope_append(q, k, v, k_cache, v_cache, cos_sin, positions,
                        slot_mapping)
    else:
        reference.rope_inplace(q, k, cos_sin, positions)
        reference.kv_append(k_cache, v_cache, k, v, slot_mapping)


def kv_append(k_cache, v_cache, k, v, slot_mapping):
    mod = _dispatch("kv_append", k)
    if mod:
        mod.kv_append(k_cache, v_cache, k, v, slot_mapping)
    else:
        reference.kv_append(k_cache, v_cache, k, v, slot_mapping)


def paged_decode_attention(out, q, k_cache, v_cache, page_table, seq_lens,
                           scale: float):
    mod = _dispatch("paged_decode_attention", q)
    if mod:
        mod.paged_decode_attention(out, q, k_cache, v_cache, page_table,
                                   seq_lens, float(scale))
    else:
        reference.paged_decode_attention(out, q, k_cache, v_cache, page_table,
                                         seq_lens, scale)
    return out


def paged_prefill_attention(out, q, k_cache, v_cache, page_table, seq_lens,
                            query_starts, query_lens, scale: float,
                            max_qlen: int = 0):
    mod = _dispatch("paged_prefill_attention", q)
    if mod:
        mod.paged_prefill_attention(out, q, k_cache, v_cache, page_table,
                                    seq_lens, query_starts, query_lens,
                                    float(scale), int(max_qlen))
    else:
        reference.paged_prefill_attention(out, q, k_cache, v_cache, page_table,
                                          seq_lens, query_starts, query_lens,
                                          scale)
    return out


def greedy_sample(out, logits):
    mod = _dispatch("greedy_sample", logits)
    if mod:
        mod.greedy_sample(out, logits)
    else:
        reference.greedy_sample(out, logits)
    return out


def topp_sample(out, logits, temps, top_ps, seeds):
    mod = _dispatch("topp_sample", logits)
    if mod:
        mod.topp_sample(out, logits, temps, top_ps, seeds)
    else:
        reference.topp_sample(out, logits, temps, top_ps, seeds)
    return out


_ws_cache = {}
_EMPTY_WS = {}
SKINNY_DISABLED = os.environ.get("AGENTAINER_DISABLE_SKINNY", "0") == "1"
SKINNY_FORCED = os.environ.get("AGENTAINER_FORCE_SKINNY", "0") == "1"
# shapes where the hand-written skinny GEMM beat hipBLASLt on MI355X,
# with the (split_k, k_chunk) that won the tools/sg_sweep.py grid
# (M=64; see profiles/README.md). Library keeps qkv/gate_up: at
# N>=6144 its MT256 tiles already stream near the roofline.
_SKINNY_SHAPES = {
    (4096, 4096): (4, 128),    # o-proj: 14.2 us vs lib 18.6
    (4096, 14336): (8, 128),   # down-proj: 30.3 us vs lib 34.4
}
SKINNY_NT = os.environ.get("AGENTAINER_SKINNY_NT", "0") == "1"
SKINNY_KC = int(os.environ.get("AGENTAINER_SKINNY_KC", "0"))  # 0 = tuned
# A/B hook: extra tuned shapes as "N:K:split:kc,..." (perf experiments)
for _spec in os.environ.get("AGENTAINER_SKINNY_SHAPES", "").split(","):
    if _spec.strip():
        _n, _k, _s, _c = (int(v) for v in _spec.split(":"))
        _SKINNY_SHAPES[(_n, _k)] = (_s, _c)


def _skinny_split(ntiles: int, K: int) -> int:
    # target ~256 blocks (1 per CU — measured optimum: 2 blocks/CU halve
    # the per-block LDS and contend on the chunk barriers)
    split = 1
    while split < 16 and ntiles * split < 256 and K % (256 * split * 2) == 0:
        split *= 2
    return split


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """Shuffle a static [N, K] weight into MFMA-fragment-linear layout
    packed[n_tile][k_chunk][lane][8] so the skinny GEMM's weight stream is
    contiguous per wave. Done once at model load; flat [N*K] result."""
    N, K = w.shape
    assert N % 16 == 0 and K % 32 == 0
    p = w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()
    return p.view(-1)


def _skinny_ws(device, N: int, split: int) -> torch.Tensor:
    if split > 1:
        key = (device, N, split)
        ws = _ws_cache.get(key)
        if ws is None or ws.numel() < split * 64 * N:
            ws = torch.empty(split * 64 * N, dtype=torch.float32, device=device)
            _ws_cache[key] = ws
        return ws
    ws = _EMPTY_WS.get(device)
    if ws is None:
        ws = torch.empty(1, dtype=torch.float32, device=device)
        _EMPTY_WS[device] = ws
    return ws


def linear(x: torch.Tensor, w: torch.Tensor,
           w_packed: Optional[torch.Tensor] = None,
           bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[M,K] @ w[N,K]^T (+ bias, added in the library GEMM's epilogue).
    Decode-shaped (M<=64) GPU GEMMs go to the
    hand-written skinny MFMA kernel — packed-weight variant when the
    caller pre-packed W (streams at the HBM roofline); everything else to
    hipBLASLt via F.linear."""
    M, K = x.shape
    N = w.size(0)
    tuned = _SKINNY_SHAPES.get((N, K))
    if (x.is_cuda and M <= 64 and N % 64 == 0 and K % 256 == 0
            and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and (tuned is not None or SKINNY_FORCED) and not SKINNY_DISABLED
            and bias is None and hip_available()):
        mod = _dispatch("skinny_gemm", x)
        split, kc = tuned if tuned else (_skinny_split(N // 64, K), 128)
        if SKINNY_KC:
            kc = SKINNY_KC
        if K % (kc * split):
            split = _skinny_split(N // 64, K)
        out = torch.empty(M, N, dtype=x.dtype, device=x.device)
        ws = _skinny_ws(x.device, N, split)
        if w_packed is not None:
            mod.skinny_gemm_packed(out, x.contiguous(), w_packed, N, K, ws,
                                   split, SKINNY_NT, kc)
        else:
            mod.skinny_gemm(out, x.contiguous(), w, ws, split)
        return out
    return torch.nn.functional.linear(x, w, bias)


def quantize_weight_fp8(w: torch.Tensor):
    """Offline per-output-channel OCP e4m3 quantization of a [N, K] weight:
    returns (fragment-linear packed bytes, f32 scales[N]). Serves the fp8
    MFMA expert decode GEMM (BASELINE config 5)."""
    N, K = w.shape
    sw = w.float().abs().amax(dim=1).clamp(min=1e-8) / 448.0
    scaled = (w.float() / sw[:, None]).clamp(-448.0, 448.0)
    try:
        w8 = scaled.to(torch.float8_e4m3fn).view(torch.uint8)
    except (RuntimeError, TypeError):
        w8 = scaled.cpu().to(torch.float8_e4m3fn).view(torch.uint8).to(w.device)
    packed = (w8.view(N // 16, 16, K // 32, 4, 8)
              .permute(0, 2, 3, 1, 4).contiguous().view(-1))
    return packed, sw.float().contiguous()


def linear_fp8(x: torch.Tensor, w_packed: torch.Tensor, sw: torch.Tensor,
               N: int) -> torch.Tensor:
    """x[M,K] bf16 @ fp8-quantized W^T: dynamic per-token activation quant
    then the fp8 MFMA skinny GEMM (half the weight bytes of bf16)."""
    M, K = x.shape
    mod = _dispatch("skinny_gemm_fp8", x)
    assert mod is not None, "linear_fp8 is GPU-only"
    xc = x.contiguous()
    x8 = torch.empty(M, K, dtype=torch.uint8, device=x.device)
    sx = torch.empty(M, dtype=torch.float32, device=x.device)
    mod.quant_fp8_rows(x8, sx, xc)
    split = _skinny_split(N // 64, K)
    ws = _skinny_ws(x.device, N, split)
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    mod.skinny_gemm_fp8(out, x8, sx, w_packed, sw, N, K, ws, split)
    return out


# e2m1 (fp4) code values, index = code (bit 3 = sign)
_FP4_GRID = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
# operand-role combo for the scaled MFMA (validated on hardware via
# tests/test_gpu_ops.py::test_mxfp4_gemm; override for probing only)
MXFP4_COMBO = int(os.environ.get("AGENTAINER_MXFP4_COMBO", "0"))


def quantize_weight_mxfp4(w: torch.Tensor):
    """Offline MXFP4 quantization of a [N, K] weight for the block-scaled
    MFMA expert GEMM (gfx950 v_mfma_scale_f32_16x16x128_f8f6f4): e2m1
    codes, 2 per byte, with one e8m0 scale per (row, 64-element k-block)
    — the scale granularity the instruction's scale lanes expose
    (tools/mx_probe.py). Returns (packed codes [N*K/2] u8 fragment-linear,
    scales [N/16 * K/128 * 32] u8 e8m0, kernel-ordered)."""
    N, K = w.shape
    assert N % 16 == 0 and K % 128 == 0, "MXFP4: N%16==0, K%128==0"
    wf = w.float().view(N, K // 32, 32)          # true MX block-32
    amax = wf.abs().amax(dim=-1).clamp(min=1e-8)
    # e8m0 scale 2^e with amax/2^e <= 6 (e2m1 max)
    e = torch.ceil(torch.log2(amax / 6.0)).clamp(-127, 127)
    scale = torch.pow(2.0, e)
    q = wf / scale.unsqueeze(-1)
    # nearest e2m1 via bucketize on the midpoints (device-native: this
    # runs at model load for up to 512 Mixtral expert matrices)
    mids = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0],
                        device=wf.device)
    idx = torch.bucketize(q.abs().contiguous(), mids)
    codes = (idx + torch.where(q < 0, 8, 0)).to(torch.uint8).view(N, K)
    # pack 2 codes/byte along k (lo nibble = even k)
    by = (codes[:, 0::2] | (codes[:, 1::2] << 4))  # [N, K/2]
    # fragment-linear: B lane map (probed):
    # B[(l/16)*32 + j][l%16] -> W[tile*16 + l%16][kc*128 + (l/16)*32 + j],
    # 32 codes = 16 bytes per lane
    byv = by.view(N // 16, 16, K // 128, 4, 16)     # [T][col][kc][q][16B]
    packed = byv.permute(0, 2, 3, 1, 4).contiguous().view(-1)
    # scales: one e8m0 per (col, 32-block); scale lane l covers
    # (kb = l/16, col = l%16) -> scv[T][kc][kb][col], 64 B per fragment
    e8 = (e + 127).clamp(0, 254).to(torch.uint8).view(N, K // 32)
    scv = e8.view(N // 16, 16, K // 128, 4).permute(0, 2, 3, 1).contiguous()
    return packed.to(w.device), scv.view(-1).to(w.device)


def dequantize_mxfp4(packed: torch.Tensor, scales: torch.Tensor,
                     N: int, K: int) -> torch.Tensor:
    """CPU reference inverse of quantize_weight_mxfp4 (tests/oracles)."""
    p = packed.cpu().view(N // 16, K // 128, 4, 16, 16)
    by = p.permute(0, 3, 1, 2, 4).contiguous().view(N, K // 2)
    lo = (by & 0xF).long()
    hi = (by >> 4).long()
    codes = torch.stack([lo, hi], dim=-1).view(N, K)
    vals = _FP4_GRID[codes & 7] * torch.where(codes >= 8, -1.0, 1.0)
    sc = scales.cpu().view(N // 16, K // 128, 4, 16).permute(0, 3, 1, 2)
    sc = sc.contiguous().view(N, K // 32).float()
    sc = torch.pow(2.0, sc - 127)
    return (vals.view(N, K // 32, 32) * sc.unsqueeze(-1)).view(N, K)


def linear_mxfp4(x: torch.Tensor, w_packed: torch.Tensor,
                 w_scales: torch.Tensor, N: int) -> torch.Tensor:
    """x[M,K] bf16 @ MXFP4 W^T: per-row e2m1 activation quant + the
    block-scaled 16x16x128 fp4 MFMA — quarter the weight bytes of bf16.
    (Mixed fp8-activation x fp4-weight through the scaled MFMA NaNs on
    this silicon/compiler — tools/mx_probe.py — so both operands run
    e2m1; activations carry a per-row f32 scale applied in the
    epilogue.)"""
    M, K = x.shape
    mod = _dispatch("skinny_gemm_mxfp4", x)
    assert mod is not None, "linear_mxfp4 is GPU-only"
    xc = x.contiguous()
    x8 = torch.empty(M, K // 2, dtype=torch.uint8, device=x.device)
    sx = torch.empty(M, dtype=torch.float32, device=x.device)
    mod.quant_fp4_rows(x8, sx, xc)
    split = _skinny_split(N // 64, K)
    ws = _skinny_ws(x.device, N, split)
    out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    mod.skinny_gemm_mxfp4(out, x8, sx, w_packed, w_scales, N, K, ws, split,
                          MXFP4_COMBO)
    return out


def linear_quant(x: torch.Tensor, qt) -> torch.Tensor:
    """Dispatch a quantized decode GEMM: qt = (kind, packed, scales, N)
    with kind "mxfp4" or "fp8" (engine.dense_quant / expert paths)."""
    kind, packed, scales, N = qt
    if kind == "mxfp4":
        return linear_mxfp4(x, packed, scales, N)
    return linear_fp8(x, packed, scales, N)


def gather_kv_pages(dst, k_cache, v_cache, page_ids):
    mod = _dispatch("gather_kv_pages", k_cache)
    if mod:
        mod.gather_kv_pages(dst, k_cache, v_cache, page_ids)
    else:
        reference.gather_kv_pages(dst, k_cache, v_cache, page_ids)


def scatter_kv_pages(k_cache, v_cache, src, page_ids):
    mod = _dispatch("scatter_kv_pages", k_cache)
    if mod:
        mod.scatter_kv_pages(k_cache, v_cache, src, page_ids)
    else:
        reference.scatter_kv_pages(k_cache, v_cache, src, page_ids)


# ---------------------------------------------------------------------
# Grouped norm / latent window attention / sigmoid-routed experts.
# These kernels live in their own extension (_hip_latent.so) so a model
# that needs only them compiles only them. Same policy as above: on a GPU
# the extension is required, on CPU the fp32 references run.
# ---------------------------------------------------------------------

_latent = None
_latent_err: Optional[str] = None


def _load_latent():
    global _latent, _latent_err
    if _latent is not None or _latent_err is not None:
        return _latent
    so = os.path.join(os.path.dirname(__file__), "_hip_latent.so")
    if not os.path.exists(so):
        _latent_err = (f"HIP extension not built ({so} missing); run "
                       "python -m agentainer_amd.ops.build latent")
        return None
    try:
        import importlib.util

        spec = importlib.util.spec_from_file_location(
            "agentainer_amd.ops._hip_latent", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _latent = mod
    except Exception as exc:  # noqa: BLE001
        _latent_err = f"HIP extension failed to load: {exc}"
    return _latent


def latent_available() -> bool:
    return _load_latent() is not None


def _dispatch_latent(name: str, t: torch.Tensor):
    if t.is_cuda:
        mod = _load_latent()
        if mod is None:
            raise RuntimeError(
                f"op {name!r} on GPU requires the gfx950 HIP extension: "
                f"{_latent_err}")
        return mod
    return None


def residual_grouped_rmsnorm(x_res, add_a, add_b, mult: float, weights, outs,
                             groups: int, eps: float):
    """fp32 residual update fused with up to two grouped RMS norms of the
    updated stream (see reference.residual_grouped_rmsnorm)."""
    mod = _dispatch_latent("residual_grouped_rmsnorm", x_res)
    if mod:
        mod.residual_grouped_rmsnorm(
            x_res, add_a, add_b, float(mult), weights[0], outs[0],
            weights[1] if len(weights) > 1 else None,
            outs[1] if len(outs) > 1 else None, int(groups), float(eps))
    else:
        reference.residual_grouped_rmsnorm(x_res, add_a, add_b, mult, weights,
                                           outs, groups, eps)
    return outs


def latent_norm_append(proj, q_off, q_rank, kv_off, kv_rank, wq, wkv, eps,
                       cq_out, cache, slot_mapping):
    mod = _dispatch_latent("latent_norm_append", proj)
    if mod:
        mod.latent_norm_append(proj, int(q_off), int(q_rank), int(kv_off),
                               int(kv_rank), wq, wkv, float(eps), cq_out,
                               cache, slot_mapping)
    else:
        reference.latent_norm_append(proj, q_off, q_rank, kv_off, kv_rank, wq,
                                     wkv, eps, cq_out, cache, slot_mapping)


# AGENTAINER_LATENT_SIMPLE=1 forces the one-wave-per-row kernel (A/B and
# numerics cross-checks against the MFMA tile kernel)
LATENT_SIMPLE = os.environ.get("AGENTAINER_LATENT_SIMPLE", "0") == "1"
# decode key-span slices per sequence; 0 = sized to fill the chip
LATENT_SPLITS = int(os.environ.get("AGENTAINER_LATENT_SPLITS", "0"))


def latent_window_attention(out, q_lat, cache, page_table, seq_lens,
                            query_starts, query_lens, scale: float,
                            window: int, max_qlen: int = 1):
    mod = _dispatch_latent("latent_window_attention", q_lat)
    if mod:
        mod.latent_window_attention(out, q_lat, cache, page_table, seq_lens,
                                    query_starts, query_lens, float(scale),
                                    int(window), int(max_qlen),
                                    bool(LATENT_SIMPLE), int(LATENT_SPLITS))
    else:
        reference.latent_window_attention(out, q_lat, cache, page_table,
                                          seq_lens, query_starts, query_lens,
                                          scale, window)
    return out


def sigmoid_gate_mul(out, a, g):
    mod = _dispatch_latent("sigmoid_gate_mul", a)
    if mod:
        mod.sigmoid_gate_mul(out, a, g)
    else:
        reference.sigmoid_gate_mul(out, a, g)
    return out


def act_mul(out, gate, up, act: str):
    """out = act(gate) * up with act in {"relu", "silu"}; bf16 or fp32."""
    mod = _dispatch_latent("act_mul", gate)
    if mod:
        mod.act_mul(out, gate, up, {"relu": 0, "silu": 1}[act])
    else:
        reference.act_mul(out, gate, up, act)
    return out


def sigmoid_topk_route(weight, logits, top: int):
    mod = _dispatch_latent("sigmoid_topk_route", logits)
    if mod:
        mod.sigmoid_topk_route(weight, logits, int(top))
    else:
        reference.sigmoid_topk_route(weight, logits, top)
    return weight


def routed_scaled_silu_mul(out, gu, weight):
    mod = _dispatch_latent("routed_scaled_silu_mul", gu)
    if mod:
        mod.routed_scaled_silu_mul(out, gu, weight)
    else:
        reference.routed_scaled_silu_mul(out, gu, weight)
    return out


# ---------------------------------------------------------------------
# Scalar-gain post-norm, PolyNorm, partial rotary (+YaRN) with q/k norms,
# masked attention (chunk / window masks; softmax or sigmoid weights) over
# per-head K/V pools. Own extension (_hip_masked.so), same policy: required
# on a GPU, fp32 torch references on CPU.
# ---------------------------------------------------------------------

_masked = None
_masked_err: Optional[str] = None


def _load_masked():
    global _masked, _masked_err
    if _masked is not None or _masked_err is not None:
        return _masked
    so = os.path.join(os.path.dirname(__file__), "_hip_masked.so")
    if not os.path.exists(so):
        _masked_err = (f"HIP extension not built ({so} missing); run "
                       "python -m agentainer_amd.ops.build masked")
        return None
    try:
        import importlib.util

        spec = importlib.util.spec_from_file_location(
            "agentainer_amd.ops._hip_masked", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _masked = mod
    except Exception as exc:  # noqa: BLE001
        _masked_err = f"HIP extension failed to load: {exc}"
    return _masked


def masked_available() -> bool:
    return _load_masked() is not None


def _dispatch_masked(name: str, t: torch.Tensor):
    if t.is_cuda:
        mod = _load_masked()
        if mod is None:
            raise RuntimeError(
                f"op {name!r} on GPU requires the gfx950 HIP extension: "
                f"{_masked_err}")
        return mod
    return None


MASK_CAUSAL = reference.MASK_CAUSAL
MASK_WINDOW = reference.MASK_WINDOW
MASK_CHUNK = reference.MASK_CHUNK
rotary_frequencies = reference.rotary_frequencies


def scalar_postnorm_residual(x_res, y, gain, eps: float, h_out):
    """x_res(fp32) += gain * y / rms(y); h_out = x_res in the compute dtype."""
    mod = _dispatch_masked("scalar_postnorm_residual", x_res)
    if mod:
        mod.scalar_postnorm_residual(x_res, y, gain, float(eps), h_out)
    else:
        reference.scalar_postnorm_residual(x_res, y, gain, eps, h_out)
    return h_out


def scalar_rmsnorm(out, x, gain, eps: float):
    mod = _dispatch_masked("scalar_rmsnorm", x)
    if mod:
        mod.scalar_rmsnorm(out, x, gain, float(eps))
    else:
        reference.scalar_rmsnorm(out, x, gain, eps)
    return out


def poly_norm(out, z, coef, eps: float):
    mod = _dispatch_masked("poly_norm", z)
    if mod:
        mod.poly_norm(out, z, coef, float(eps))
    else:
        reference.poly_norm(out, z, coef, eps)
    return out


def rotary_table(positions, freqs, amp: float):
    """fp32 [T, 2*half]: cos | sin of positions[t] * freqs[i], times amp."""
    mod = _dispatch_masked("rotary_table", positions)
    if mod:
        return mod.rotary_table(positions, freqs, float(amp))
    return reference.rotary_table(positions, freqs, amp)


def rotary_norm_append(q, k, v, k_cache, v_cache, cos_sin, slot_mapping,
                       eps: float, q_w=None, k_w=None,
                       norm_first: bool = False):
    mod = _dispatch_masked("rotary_norm_append", q)
    if mod:
        mod.rotary_norm_append(q, k, v, k_cache, v_cache, cos_sin,
                               slot_mapping, float(eps), q_w, k_w,
                               bool(norm_first))
    else:
        reference.rotary_norm_append(q, k, v, k_cache, v_cache, cos_sin,
                                     slot_mapping, eps, q_w, k_w, norm_first)


# AGENTAINER_MASKED_SIMPLE=1 forces the one-wave-per-row kernel (A/B and
# numerics cross-checks against the MFMA tile kernel)
MASKED_SIMPLE = os.environ.get("AGENTAINER_MASKED_SIMPLE", "0") == "1"
# decode key-range slices per (sequence, kv head); 0 = sized to fill the chip
MASKED_SPLITS = int(os.environ.get("AGENTAINER_MASKED_SPLITS", "0"))


def masked_attention(out, q, k_cache, v_cache, page_table, seq_lens,
                     query_starts, query_lens, scale: float, mask_kind: int,
                     mask_size: int, keep_first: int = 0,
                     sigmoid_weights: bool = False, softcap: float = 0.0,
                     key_bias=None, head_gate=None, max_qlen: int = 1,
                     dist_bias=None):
    """dist_bias: fp32 [H, 2] = (r1, r2) per head; r1 * ln(1 + r2 * distance)
    is taken off every score (see reference.masked_attention)."""
    mod = _dispatch_masked("masked_attention", q)
    if mod:
        mod.masked_attention(out, q, k_cache, v_cache, page_table, seq_lens,
                             query_starts, query_lens, float(scale),
                             int(mask_kind), int(mask_size), int(keep_first),
                             bool(sigmoid_weights), float(softcap), key_bias,
                             head_gate, int(max_qlen), bool(MASKED_SIMPLE),
                             int(MASKED_SPLITS), dist_bias)
    else:
        reference.masked_attention(out, q, k_cache, v_cache, page_table,
                                   seq_lens, query_starts, query_lens, scale,
                                   mask_kind, mask_size, keep_first,
                                   sigmoid_weights, softcap, key_bias,
                                   head_gate, dist_bias)
    return out


# ---------------------------------------------------------------------
# Post-norm residual with (1 + w) RMS norm, short causal convolutions with
# a per-sequence tail, matrix-memory recurrences (gated linear attention,
# gated delta rule, mLSTM) over per-sequence state, per-head output norm +
# gate, group-limited softmax routing and clamped gated experts. Own
# extension (_hip_recurrent.so), same policy: required on a GPU, fp32
# torch references on CPU.
# ---------------------------------------------------------------------

_recurrent = None
_recurrent_err: Optional[str] = None


def _load_recurrent():
    global _recurrent, _recurrent_err
    if _recurrent is not None or _recurrent_err is not None:
        return _recurrent
    so = os.path.join(os.path.dirname(__file__), "_hip_recurrent.so")
    if not os.path.exists(so):
        _recurrent_err = (f"HIP extension not built ({so} missing); run "
                          "python -m agentainer_amd.ops.build recurrent")
        return None
    try:
        import importlib.util

        spec = importlib.util.spec_from_file_location(
            "agentainer_amd.ops._hip_recurrent", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _recurrent = mod
    except Exception as exc:  # noqa: BLE001
        _recurrent_err = f"HIP extension failed to load: {exc}"
    return _recurrent


def recurrent_available() -> bool:
    return _load_recurrent() is not None


def _dispatch_recurrent(name: str, t: torch.Tensor):
    if t.is_cuda:
        mod = _load_recurrent()
        if mod is None:
            raise RuntimeError(
                f"op {name!r} on GPU requires the gfx950 HIP extension: "
                f"{_recurrent_err}")
        return mod
    return None


SCAN_GLA = reference.SCAN_GLA
SCAN_DELTA = reference.SCAN_DELTA
SCAN_MLSTM = reference.SCAN_MLSTM


def postln_rmsnorm_residual(x_res, y, w1p, eps: float, h_out,
                            alpha: float = 1.0, y_scale: float = 1.0,
                            y2=None, y2_scale: float = 1.0, row_add=None):
    """x_res(fp32) <- rms_norm((alpha + row_add[t]) * x_res + y_scale * y
    + y2_scale * y2) * w1p; h_out = x_res in the compute dtype."""
    mod = _dispatch_recurrent("postln_rmsnorm_residual", x_res)
    if mod:
        mod.postln_rmsnorm_residual(x_res, y, float(y_scale), y2,
                                    float(y2_scale), float(alpha), row_add,
                                    w1p, float(eps), h_out)
    else:
        reference.postln_rmsnorm_residual(x_res, y, y_scale, y2, y2_scale,
                                          alpha, row_add, w1p, eps, h_out)
    return h_out


def short_conv_state(out, u, w, tail, state_slots, seq_lens, query_starts,
                     query_lens, silu: bool = False, norm_channels: int = 0,
                     head_dim: int = 1, lead_channels: int = 0,
                     lead_scale: float = 1.0, l2_eps: float = 1e-6):
    mod = _dispatch_recurrent("short_conv_state", u)
    if mod:
        mod.short_conv_state(out, u, w, tail, state_slots, seq_lens,
                             query_starts, query_lens, bool(silu),
                             int(norm_channels), int(head_dim),
                             int(lead_channels), float(lead_scale),
                             float(l2_eps))
    else:
        reference.short_conv_state(out, u, w, tail, state_slots, seq_lens,
                                   query_starts, query_lens, silu,
                                   norm_channels, head_dim, lead_channels,
                                   lead_scale, l2_eps)
    return out


# lanes that share one value column in the recurrence kernel; 0 = sized per
# launch (A/B runs)
SCAN_LANES = int(os.environ.get("AGENTAINER_SCAN_LANES", "0"))


def matrix_memory_scan(kind: int, out, q, k, v, gate, gate_bias, head_rate,
                       beta, q_scale: float, gate_param: float, S, n_state,
                       m_state, state_slots, seq_lens, query_starts,
                       query_lens):
    mod = _dispatch_recurrent("matrix_memory_scan", q)
    if mod:
        mod.matrix_memory_scan(int(kind), out, q, k, v, gate, gate_bias,
                               head_rate, beta, float(q_scale),
                               float(gate_param), S, n_state, m_state,
                               state_slots, seq_lens, query_starts,
                               query_lens, int(SCAN_LANES))
    else:
        reference.matrix_memory_scan(kind, out, q, k, v, gate, gate_bias,
                                     head_rate, beta, q_scale, gate_param, S,
                                     n_state, m_state, state_slots, seq_lens,
                                     query_starts, query_lens)
    return out


def head_rmsnorm_gate(out, o, w, gate, eps: float, silu_gate: bool):
    mod = _dispatch_recurrent("head_rmsnorm_gate", o)
    if mod:
        mod.head_rmsnorm_gate(out, o, w, gate, float(eps), bool(silu_gate))
    else:
        reference.head_rmsnorm_gate(out, o, w, gate, eps, silu_gate)
    return out


def grouped_softmax_route(weight, logits, correction, top: int,
                          n_groups: int, keep_groups: int, scale: float):
    mod = _dispatch_recurrent("grouped_softmax_route", logits)
    if mod:
        mod.grouped_softmax_route(weight, logits, correction, int(top),
                                  int(n_groups), int(keep_groups),
                                  float(scale))
    else:
        reference.grouped_softmax_route(weight, logits, correction, top,
                                        n_groups, keep_groups, scale)
    return weight


def routed_clamped_glu(out, gu, weight, n_experts: int, limit: float,
                       slope: float):
    mod = _dispatch_recurrent("routed_clamped_glu", gu)
    if mod:
        mod.routed_clamped_glu(out, gu, weight, int(n_experts), float(limit),
                               float(slope))
    else:
        reference.routed_clamped_glu(out, gu, weight, n_experts, limit, slope)
    return out


# ---------------------------------------------------------------------
# Hashed bigram embedding, sigmoid-gated residual + layer norm, xIELU,
# token-side gate, sigmoid group-limited routing, output-weighted gated
# experts with a tail expert, latent rotary append, plain K/V append and
# an elementwise output gate. Own extension (_hip_gated.so), same policy:
# required on a GPU, fp32 torch references on CPU.
# ---------------------------------------------------------------------

_gated = None
_gated_err: Optional[str] = None


def _load_gated():
    global _gated, _gated_err
    if _gated is not None or _gated_err is not None:
        return _gated
    so = os.path.join(os.path.dirname(__file__), "_hip_gated.so")
    if not os.path.exists(so):
        _gated_err = (f"HIP extension not built ({so} missing); run "
                      "python -m agentainer_amd.ops.build gated")
        return None
    try:
        import importlib.util

        spec = importlib.util.spec_from_file_location(
            "agentainer_amd.ops._hip_gated", so)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _gated = mod
    except Exception as exc:  # noqa: BLE001
        _gated_err = f"HIP extension failed to load: {exc}"
    return _gated


def gated_available() -> bool:
    return _load_gated() is not None


def _dispatch_gated(name: str, t: torch.Tensor):
    if t.is_cuda:
        mod = _load_gated()
        if mod is None:
            raise RuntimeError(
                f"op {name!r} on GPU requires the gfx950 HIP extension: "
                f"{_gated_err}")
        return mod
    return None


UPDATE_NONE = reference.UPDATE_NONE
UPDATE_SIGMOID_GATE = reference.UPDATE_SIGMOID_GATE
UPDATE_UNIT_RMS = reference.UPDATE_UNIT_RMS


def bigram_embed(x_out, ids, embed, bigram, scale: float, mul_prev: int,
                 mul_cur: int, buckets: int, prev_state, state_slots,
                 seq_lens, query_starts, query_lens):
    mod = _dispatch_gated("bigram_embed", x_out)
    if mod:
        mod.bigram_embed(x_out, ids, embed, bigram, float(scale),
                         int(mul_prev), int(mul_cur), int(buckets),
                         prev_state, state_slots, seq_lens, query_starts,
                         query_lens)
    else:
        reference.bigram_embed(x_out, ids, embed, bigram, scale, mul_prev,
                               mul_cur, buckets, prev_state, state_slots,
                               seq_lens, query_starts, query_lens)
    return x_out


def residual_update_norm(x_res, y, update: int, gate, gate_bias, rms_w,
                         eps: float, norm_w, norm_b, h_out):
    mod = _dispatch_gated("residual_update_norm", x_res)
    if mod:
        mod.residual_update_norm(x_res, y, int(update), gate, gate_bias,
                                 rms_w, float(eps), norm_w, norm_b, h_out)
    else:
        reference.residual_update_norm(x_res, y, update, gate, gate_bias,
                                       rms_w, eps, norm_w, norm_b, h_out)
    return h_out


def xielu(out, z, coef):
    mod = _dispatch_gated("xielu", z)
    if mod:
        mod.xielu(out, z, coef)
    else:
        reference.xielu(out, z, coef)
    return out


def gelu_gate_rows(out, t, table, ids, col0: int):
    mod = _dispatch_gated("gelu_gate_rows", t)
    if mod:
        mod.gelu_gate_rows(out, t, table, ids, int(col0))
    else:
        reference.gelu_gate_rows(out, t, table, ids, col0)
    return out


def grouped_sigmoid_route(weight, logits, correction, n_experts: int,
                          top: int, n_groups: int, keep_groups: int,
                          group_top: int = 2):
    mod = _dispatch_gated("grouped_sigmoid_route", logits)
    if mod:
        mod.grouped_sigmoid_route(weight, logits, correction, int(n_experts),
                                  int(top), int(n_groups), int(keep_groups),
                                  int(group_top))
    else:
        reference.grouped_sigmoid_route(weight, logits, correction, n_experts,
                                        top, n_groups, keep_groups, group_top)
    return weight


def routed_silu_glu(out, gu, weight, n_experts: int, ff: int,
                    tail_ff: int = 0):
    mod = _dispatch_gated("routed_silu_glu", gu)
    if mod:
        mod.routed_silu_glu(out, gu, weight, int(n_experts), int(ff),
                            int(tail_ff))
    else:
        reference.routed_silu_glu(out, gu, weight, n_experts, ff, tail_ff)
    return out


def latent_rotary_append(proj, heads: int, q_head: int, q_rot_off: int,
                         kv_off: int, kv_rank: int, rot_dim: int, w_kv,
                         eps: float, cos_sin, cache, slot_mapping):
    mod = _dispatch_gated("latent_rotary_append", proj)
    if mod:
        mod.latent_rotary_append(proj, int(heads), int(q_head),
                                 int(q_rot_off), int(kv_off), int(kv_rank),
                                 int(rot_dim), w_kv, float(eps), cos_sin,
                                 cache, slot_mapping)
    else:
        reference.latent_rotary_append(proj, heads, q_head, q_rot_off, kv_off,
                                       kv_rank, rot_dim, w_kv, eps, cos_sin,
                                       cache, slot_mapping)


def head_kv_append(k, v, k_cache, v_cache, slot_mapping):
    mod = _dispatch_gated("head_kv_append", k)
    if mod:
        mod.head_kv_append(k, v, k_cache, v_cache, slot_mapping)
    else:
        reference.head_kv_append(k, v, k_cache, v_cache, slot_mapping)


def sigmoid_gate_rows(out, a, gate):
    mod = _dispatch_gated("sigmoid_gate_rows", a)
    if mod:
        mod.sigmoid_gate_rows(out, a, gate)
    else:
        reference.sigmoid_gate_rows(out, a, gate)
    return out
