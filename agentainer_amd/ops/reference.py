"""Pure-PyTorch fp32 reference implementations of every HIP op.

Dual purpose (SURVEY.md §4 test strategy):
  * the numerics oracle for the GPU kernel tests (kernel output vs the
    fp32 reference of the same op, tolerance-gated);
  * the CPU execution path of the engine, so the full control plane +
    scheduler run (and are tested) on GPU-less CI.

Tensors use the same shapes/layouts as the HIP kernels, including the
paged-cache layouts k_cache [P, n_kv, D/8, PS, 8] / v_cache [P, n_kv, PS, D].
"""

from __future__ import annotations

import math


import torch


def rmsnorm(out: torch.Tensor, x: torch.Tensor, w: torch.Tensor, eps: float) -> None:
    xf = x.float()
    r = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((r * w.float()).to(out.dtype))


def fused_add_rmsnorm(out: torch.Tensor, x: torch.Tensor, residual: torch.Tensor,
                      w: torch.Tensor, eps: float) -> None:
    s = (x.float() + residual.float())
    residual.copy_(s.to(residual.dtype))
    sf = residual.float()  # match kernel: normalizes the bf16-rounded sum
    r = sf * torch.rsqrt(sf.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((r * w.float()).to(out.dtype))


def silu_mul(out: torch.Tensor, gate: torch.Tensor, up: torch.Tensor) -> None:
    g = gate.float()
    out.copy_((g * torch.sigmoid(g) * up.float()).to(out.dtype))


def make_cos_sin_table(max_pos: int, dim: int, theta: float = 500000.0,
                       device="cpu") -> torch.Tensor:
    """[max_pos, dim] f32 rows laid out [cos(0..d/2) | sin(0..d/2)]."""
    inv = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
    pos = torch.arange(max_pos, dtype=torch.float64)
    ang = torch.outer(pos, inv)
    tab = torch.cat([torch.cos(ang), torch.sin(ang)], dim=-1).float()
    return tab.contiguous().to(device)


def rope_inplace(q: torch.Tensor, k: torch.Tensor, cos_sin: torch.Tensor,
                 positions: torch.Tensor) -> None:
    D = q.size(-1)
    half = D // 2
    c = cos_sin[positions.long(), :half].unsqueeze(1).float()  # [T,1,half]
    s = cos_sin[positions.long(), half:].unsqueeze(1).float()
    for t in (q, k):
        x1 = t[..., :half].float()
        x2 = t[..., half:].float()
        t[..., :half] = (x1 * c - x2 * s).to(t.dtype)
        t[..., half:] = (x1 * s + x2 * c).to(t.dtype)


def kv_append(k_cache: torch.Tensor, v_cache: torch.Tensor, k: torch.Tensor,
              v: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    n_kv, D = k.size(1), k.size(2)
    PS = k_cache.size(3)
    for t in range(k.size(0)):
        slot = int(slot_mapping[t])
        if slot < 0:
            continue
        page, off = slot // PS, slot % PS
        # k_cache [P, n_kv, D/8, PS, 8]; .to() casts bf16 -> fp8 when the
        # pool is e4m3 (index-assignment alone won't cast to float8)
        k_cache[page, :, :, off, :] = (
            k[t].reshape(n_kv, D // 8, 8).to(k_cache.dtype))
        v_cache[page, :, off, :] = v[t].to(v_cache.dtype)


def _gather_kv(k_cache, v_cache, page_table_row, length, g):
    """K/V [length, D] f32 for kv head g of one sequence."""
    PS = k_cache.size(3)
    D = v_cache.size(3)
    ks, vs = [], []
    for tok in range(length):
        page = int(page_table_row[tok // PS])
        off = tok % PS
        ks.append(k_cache[page, g, :, off, :].reshape(D).float())
        vs.append(v_cache[page, g, off, :].float())
    return torch.stack(ks), torch.stack(vs)


def paged_decode_attention(out: torch.Tensor, q: torch.Tensor,
                           k_cache: torch.Tensor, v_cache: torch.Tensor,
                           page_table: torch.Tensor, seq_lens: torch.Tensor,
                           scale: float) -> None:
    B, n_q, D = q.shape
    n_kv = k_cache.size(1)
    ratio = n_q // n_kv
    for b in range(B):
        length = int(seq_lens[b])
        if length <= 0:
            out[b] = 0  # graph pad row (dev_seq_lens == -1); HIP kernel skips
            continue
        for g in range(n_kv):
            K, V = _gather_kv(k_cache, v_cache, page_table[b], length, g)
            for qh in range(g * ratio, (g + 1) * ratio):
                s = (K @ q[b, qh].float()) * scale
                p = torch.softmax(s, dim=-1)
                out[b, qh] = (p @ V).to(out.dtype)


def paged_prefill_attention(out: torch.Tensor, q: torch.Tensor,
                            k_cache: torch.Tensor, v_cache: torch.Tensor,
                            page_table: torch.Tensor, seq_lens: torch.Tensor,
                            query_starts: torch.Tensor, query_lens: torch.Tensor,
                            scale: float) -> None:
    n_q = q.size(1)
    n_kv = k_cache.size(1)
    ratio = n_q // n_kv
    B = seq_lens.numel()
    for b in range(B):
        qlen = int(query_lens[b])
        if qlen == 0:
            continue
        total = int(seq_lens[b])
        start = int(query_starts[b])
        ctx_start = total - qlen
        for g in range(n_kv):
            K, V = _gather_kv(k_cache, v_cache, page_table[b], total, g)
            for qh in range(g * ratio, (g + 1) * ratio):
                Q = q[start:start + qlen, qh].float()       # [qlen, D]
                s = Q @ K.t() * scale                       # [qlen, total]
                qpos = ctx_start + torch.arange(qlen).unsqueeze(1)
                kpos = torch.arange(total).unsqueeze(0)
                s = s.masked_fill(kpos > qpos, float("-inf"))
                p = torch.softmax(s, dim=-1)
                out[start:start + qlen, qh] = (p @ V).to(out.dtype)


def greedy_sample(out: torch.Tensor, logits: torch.Tensor) -> None:
    out.copy_(logits.float().argmax(dim=-1))


def topp_sample(out: torch.Tensor, logits: torch.Tensor, temps: torch.Tensor,
                top_ps: torch.Tensor, seeds: torch.Tensor) -> None:
    """Reference nucleus sampling. Uses torch RNG seeded per row so results
    are deterministic given seeds (NOT bitwise-matched to the HIP kernel —
    distribution-level tests only)."""
    B, V = logits.shape
    for b in range(B):
        gen = torch.Generator(device="cpu").manual_seed(int(seeds[b]) & 0x7FFFFFFF)
        p = torch.softmax(logits[b].float() / max(float(temps[b]), 1e-6), dim=-1)
        sp, idx = p.sort(descending=True)
        cum = sp.cumsum(0)
        cut = int(torch.searchsorted(cum, float(top_ps[b])).item()) + 1
        cut = min(cut, V)
        sp = sp[:cut] / sp[:cut].sum()
        pick = idx[torch.multinomial(sp.cpu(), 1, generator=gen)]
        out[b] = pick.to(out.device)


def gather_kv_pages(dst: torch.Tensor, k_cache: torch.Tensor,
                    v_cache: torch.Tensor, page_ids: torch.Tensor) -> None:
    n_kv = k_cache.size(1)
    D = v_cache.size(3)
    PS = k_cache.size(3)
    plane = n_kv * D * PS
    flat = dst.view(-1)
    for i, p in enumerate(page_ids.tolist()):
        flat[i * 2 * plane:(i * 2 + 1) * plane] = k_cache[p].reshape(-1)
        flat[(i * 2 + 1) * plane:(i + 1) * 2 * plane] = v_cache[p].reshape(-1)


def scatter_kv_pages(k_cache: torch.Tensor, v_cache: torch.Tensor,
                     src: torch.Tensor, page_ids: torch.Tensor) -> None:
    n_kv = k_cache.size(1)
    D = v_cache.size(3)
    PS = k_cache.size(3)
    plane = n_kv * D * PS
    flat = src.view(-1)
    for i, p in enumerate(page_ids.tolist()):
        k_cache[p] = flat[i * 2 * plane:(i * 2 + 1) * plane].view_as(k_cache[p])
        v_cache[p] = flat[(i * 2 + 1) * plane:(i + 1) * 2 * plane].view_as(v_cache[p])


# ---------------------------------------------------------------------
# Grouped norm, latent window attention, sigmoid-routed experts
# (fp32 math; outputs take the dtype of the tensor they are written to)
# ---------------------------------------------------------------------

def residual_grouped_rmsnorm(x_res: torch.Tensor, add_a, add_b, mult: float,
                             weights, outs, groups: int, eps: float) -> None:
    """x_res (fp32, in place) += mult * (add_a + add_b); then for every
    (w, out) pair: out = x_res / sqrt(mean_g(x_res^2) + eps) * w, the mean
    taken separately over each of `groups` equal consecutive parts."""
    if add_a is not None or add_b is not None:
        s = torch.zeros_like(x_res)
        if add_a is not None:
            s = s + add_a.float()
        if add_b is not None:
            s = s + add_b.float()
        x_res.add_(s * mult)
    T, W = x_res.shape
    parts = x_res.view(T, groups, W // groups)
    unit = (parts * torch.rsqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
            ).reshape(T, W)
    for w, out in zip(weights, outs):
        out.copy_((unit * w.float()).to(out.dtype))


def latent_norm_append(proj: torch.Tensor, q_off: int, q_rank: int,
                       kv_off: int, kv_rank: int, wq: torch.Tensor,
                       wkv: torch.Tensor, eps: float, cq_out: torch.Tensor,
                       cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """RMS-norm the query latent and the key/value latent held in two
    column ranges of `proj`; the first goes to cq_out, the second into
    the paged latent pool cache[P, PS, Rp] at each token's slot (columns
    past kv_rank are zero-filled; slot < 0 skips the append)."""
    def unit(v):
        return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)

    cq = proj[:, q_off:q_off + q_rank].float()
    cq_out.copy_((unit(cq) * wq.float()).to(cq_out.dtype))
    c = proj[:, kv_off:kv_off + kv_rank].float()
    c = (unit(c) * wkv.float()).to(cache.dtype)
    PS, Rp = cache.size(1), cache.size(2)
    flat = cache.view(-1, Rp)
    ok = slot_mapping >= 0
    rows = slot_mapping[ok].long()
    flat[rows, :kv_rank] = c[ok]
    if Rp > kv_rank:
        flat[rows, kv_rank:] = 0


def latent_window_attention(out: torch.Tensor, q_lat: torch.Tensor,
                            cache: torch.Tensor, page_table: torch.Tensor,
                            seq_lens: torch.Tensor, query_starts,
                            query_lens, scale: float, window: int) -> None:
    """Multi-query attention in latent space: every head's query q_lat[h, t]
    (already mapped into the latent basis) scores the cached latents
    themselves, and the output is the softmax-weighted sum of the same
    latents. A query at position p sees keys at p - window < j <= p.
    q_lat/out: [H, T, Rp]; cache [P, PS, Rp]. query_starts/query_lens None
    means one new token per sequence (decode)."""
    H = q_lat.size(0)
    PS, Rp = cache.size(1), cache.size(2)
    flat = cache.view(-1, Rp)
    B = seq_lens.numel()
    for b in range(B):
        total = int(seq_lens[b])
        qlen = 1 if query_lens is None else int(query_lens[b])
        start = b if query_starts is None else int(query_starts[b])
        if total <= 0 or qlen == 0:
            if total <= 0 and query_lens is None:
                out[:, start] = 0
            continue
        ctx = total - qlen
        lo = max(0, ctx - window + 1)
        pos = torch.arange(lo, total)
        rows = (page_table[b, (pos // PS).long()].long() * PS + pos % PS)
        C = flat[rows].float()                          # [n, Rp]
        Q = q_lat[:, start:start + qlen].float()        # [H, qlen, Rp]
        s = torch.einsum("hqr,nr->hqn", Q, C) * scale
        qpos = (ctx + torch.arange(qlen)).view(1, qlen, 1)
        kpos = pos.view(1, 1, -1)
        seen = (kpos <= qpos) & (qpos - kpos < window)
        s = s.masked_fill(~seen, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, start:start + qlen] = torch.einsum("hqn,nr->hqr", p, C
                                                  ).to(out.dtype)


def sigmoid_gate_mul(out: torch.Tensor, a: torch.Tensor, g: torch.Tensor) -> None:
    """out[t, h*E + e] = a[h, t, e] * sigmoid(g[t, h*E + e])."""
    H, T, E = a.shape
    av = a.permute(1, 0, 2).reshape(T, H * E).float()
    out.copy_((av * torch.sigmoid(g.float())).to(out.dtype))


def act_mul(out: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
            act: str) -> None:
    g = gate.float()
    if act == "relu":
        a = torch.relu(g)
    elif act == "silu":
        a = g * torch.sigmoid(g)
    else:
        raise ValueError(act)
    out.copy_((a * up.float()).to(out.dtype))


def sigmoid_topk_route(weight: torch.Tensor, logits: torch.Tensor,
                       top: int) -> None:
    """weight[t, e] = sigmoid(logits[t, e]) for the `top` largest entries
    of row t (ties: lowest index first), 0 elsewhere. fp32 throughout."""
    s = torch.sigmoid(logits.float())
    val, idx = s.topk(top, dim=-1)
    weight.zero_()
    weight.scatter_(1, idx, val)


def routed_scaled_silu_mul(out: torch.Tensor, gu: torch.Tensor,
                           weight: torch.Tensor) -> None:
    """Stacked-expert activation with the routing weight applied on the
    INPUT side: gu [T, E, 2F] holds every expert's gate|up projections of
    the unscaled input, so the scaled-input projections are w*gate and
    w*up; out[t, e, :] = silu(w g) * (w u), which is 0 where w == 0."""
    T, E = weight.shape
    F_ = gu.size(-1) // (2 * E)
    g3 = gu.view(T, E, 2 * F_).float()
    w = weight.view(T, E, 1).float()
    g = g3[..., :F_] * w
    u = g3[..., F_:] * w
    out.copy_((g * torch.sigmoid(g) * u).view(T, E * F_).to(out.dtype))


# ---------------------------------------------------------------------
# Scalar-gain norms, PolyNorm, partial rotary (+YaRN) with q/k norms, and
# masked attention (chunk / window-with-kept-prefix masks, softmax or
# per-key sigmoid weights) over per-head paged K/V pools.
# ---------------------------------------------------------------------

def _unit(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)


def scalar_postnorm_residual(x_res: torch.Tensor, y: torch.Tensor,
                             gain: torch.Tensor, eps: float,
                             h_out: torch.Tensor) -> None:
    """Post-norm residual step: x_res (fp32, in place) += gain * y/rms(y)
    with ONE gain for the whole row; h_out receives the updated stream in
    the compute dtype (the next sublayer's GEMM input)."""
    x_res.add_(_unit(y.float(), eps) * gain.float().reshape(()))
    h_out.copy_(x_res.to(h_out.dtype))


def scalar_rmsnorm(out: torch.Tensor, x: torch.Tensor, gain: torch.Tensor,
                   eps: float) -> None:
    out.copy_((_unit(x.float(), eps) * gain.float().reshape(())
               ).to(out.dtype))


def poly_norm(out: torch.Tensor, z: torch.Tensor, coef: torch.Tensor,
              eps: float) -> None:
    """out = a U(z) + b U(z^2) + c U(z^3) + e, U = unit rms over the row,
    powers elementwise, coef = (a, b, c, e) fp32."""
    zf = z.float()
    c = coef.float()
    z2 = zf * zf
    out.copy_((c[0] * _unit(zf, eps) + c[1] * _unit(z2, eps)
               + c[2] * _unit(z2 * zf, eps) + c[3]).to(out.dtype))


def rotary_frequencies(dims: int, base: float, scaling=None, device=None):
    """(freqs fp32 [dims/2], amplitude) of a rotary embedding over `dims`
    coordinates: f_i = base^(-2i/dims). `scaling` = dict(factor, original,
    fast, slow) applies YaRN: with d(t) = dims ln(original / (2 pi t)) /
    (2 ln base), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)),
    dims-1) and ramp_i = clamp((i-lo)/max(hi-lo, .001), 0, 1), the
    frequency becomes f_i/factor * ramp_i + f_i (1-ramp_i) and cos/sin are
    scaled by 0.1 ln(factor) + 1. Computed in double on the host, stored
    fp32 on `device` (default: the current default device)."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64, device="cpu")
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64, device="cpu"),
                  -2.0 * i / dims)
    amp = 1.0
    if scaling:
        factor = float(scaling["factor"])
        orig = float(scaling["original"])

        def corr(turns):
            return (dims * math.log(orig / (2 * math.pi * turns))
                    / (2 * math.log(base)))

        lo = max(math.floor(corr(float(scaling["fast"]))), 0)
        hi = min(math.ceil(corr(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    f = f.to(torch.float32)
    if device is None:      # follow an enclosing `with torch.device(...)`
        device = torch.empty(0).device
    return f.to(device), float(amp)


def rotary_table(positions: torch.Tensor, freqs: torch.Tensor,
                 amp: float) -> torch.Tensor:
    """fp32 [T, 2*half] = cos(a) * amp | sin(a) * amp with a = position *
    freq in fp32: one row per token of the step, shared by every layer and
    head with this rotary setting."""
    ang = positions.to(torch.float32).unsqueeze(1) * freqs.unsqueeze(0)
    return torch.cat([torch.cos(ang) * amp, torch.sin(ang) * amp], dim=1)


def _rotate_half(u: torch.Tensor, cos_sin: torch.Tensor) -> torch.Tensor:
    """u fp32 [T, heads, D]; the first 2*half coordinates of every head
    rotate, coordinate i paired with i + half; cos_sin [T, 2*half]."""
    half = cos_sin.size(1) // 2
    c = cos_sin[:, :half].unsqueeze(1)
    s = cos_sin[:, half:].unsqueeze(1)
    a, b = u[..., :half], u[..., half:2 * half]
    return torch.cat([a * c - b * s, b * c + a * s, u[..., 2 * half:]], -1)


def rotary_norm_append(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor,
                       cos_sin: torch.Tensor, slot_mapping: torch.Tensor,
                       eps: float, q_w=None, k_w=None,
                       norm_first: bool = False) -> None:
    """Prepare one step's queries and keys and append K/V to the pools.

    q [T, H, D] (rewritten in place), k [T, G, D], v [T, G, Dv]; pools
    k_cache [P, G, PS, D], v_cache [P, G, PS, Dv] (per page and kv head, PS
    consecutive token rows); slot = page*PS + offset (slot < 0 skips the
    append); cos_sin = rotary_table(...) of the step. Per head, in fp32:
      norm_first: u <- rms_norm(u) * w, then rotate   (w = q_w / k_w [D])
      otherwise : u <- rotate(u), then unit rms (no weight)."""
    def prep(u, w):
        u = u.float()
        if norm_first:
            u = _unit(u, eps)
            if w is not None:
                u = u * w.float()
            return _rotate_half(u, cos_sin)
        return _unit(_rotate_half(u, cos_sin), eps)

    q.copy_(prep(q, q_w).to(q.dtype))
    kk = prep(k, k_w).to(k_cache.dtype)
    PS = k_cache.size(2)
    ok = slot_mapping >= 0
    rows = slot_mapping[ok].long()
    page, off = rows // PS, rows % PS
    k_cache[page, :, off] = kk[ok]
    v_cache[page, :, off] = v[ok].to(v_cache.dtype)


MASK_CAUSAL, MASK_WINDOW, MASK_CHUNK = 0, 1, 2


def mask_visible(qpos: torch.Tensor, kpos: torch.Tensor, kind: int,
                 size: int, keep_first: int) -> torch.Tensor:
    """Boolean visibility of key positions for query positions.
    causal: j <= p.  window: j <= p and (p - j < size or j < keep_first).
    chunk: j <= p and floor(p/size) == floor(j/size)."""
    seen = kpos <= qpos
    if kind == MASK_WINDOW:
        seen = seen & ((qpos - kpos < size) | (kpos < keep_first))
    elif kind == MASK_CHUNK:
        seen = seen & (torch.div(qpos, size, rounding_mode="floor")
                       == torch.div(kpos, size, rounding_mode="floor"))
    return seen


def masked_attention(out: torch.Tensor, q: torch.Tensor,
                     k_cache: torch.Tensor, v_cache: torch.Tensor,
                     page_table: torch.Tensor, seq_lens: torch.Tensor,
                     query_starts, query_lens, scale: float, mask_kind: int,
                     mask_size: int, keep_first: int, sigmoid_weights: bool,
                     softcap: float, key_bias, head_gate,
                     dist_bias=None) -> None:
    """Grouped-query attention over paged per-head K/V pools.

    out [T, H, Dv], q [T, H, D]; query head h reads kv head h // (H/G).
    score = <q, k> * scale, then softcap * tanh(score / softcap) when
    softcap > 0. Weights are a softmax over the visible keys, or (with
    sigmoid_weights) sigmoid(score + key_bias[h]) per visible key without
    normalization. head_gate [T, H], when given, multiplies head h's
    output by sigmoid(head_gate[t, h]); with H * Dv columns it gates every
    output coordinate. query_starts/query_lens None means
    one new token per sequence; rows with seq_len <= 0 come back zero.
    dist_bias fp32 [H, 2] = (r1, r2) per head takes r1 * ln(1 + r2 * (p - j))
    off the (capped) score of key j for the query at position p."""
    H = q.size(1)
    G, PS = k_cache.size(1), k_cache.size(2)
    rep = H // G
    B = seq_lens.numel()
    for b in range(B):
        total = int(seq_lens[b])
        qlen = 1 if query_lens is None else int(query_lens[b])
        start = b if query_starts is None else int(query_starts[b])
        if total <= 0 or qlen == 0:
            if total <= 0 and query_lens is None:
                out[start] = 0
            continue
        pos = torch.arange(total)
        pages = page_table[b, (pos // PS).long()].long()
        K = k_cache[pages, :, pos % PS].float().repeat_interleave(rep, dim=1)
        V = v_cache[pages, :, pos % PS].float().repeat_interleave(rep, dim=1)
        Q = q[start:start + qlen].float()                     # K [n, H, D]
        s = torch.einsum("qhd,nhd->hqn", Q, K) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        qpos = (total - qlen + torch.arange(qlen)).view(1, qlen, 1)
        seen = mask_visible(qpos, pos.view(1, 1, -1), mask_kind, mask_size,
                            keep_first)
        if dist_bias is not None:
            db = dist_bias.float()
            dist = (qpos - pos.view(1, 1, -1)).clamp(min=0).float()
            s = s - db[:, 0].view(H, 1, 1) * torch.log1p(
                db[:, 1].view(H, 1, 1) * dist)
        if sigmoid_weights:
            if key_bias is not None:
                s = s + key_bias.float().view(H, 1, 1)
            p = torch.sigmoid(s) * seen
        else:
            p = torch.softmax(s.masked_fill(~seen, float("-inf")), dim=-1)
        o = torch.einsum("hqn,nhe->qhe", p, V)
        if head_gate is not None:
            gt = torch.sigmoid(head_gate[start:start + qlen].float())
            # [q, H]: one gate per head; [q, H * Dv]: one per coordinate
            o = o * (gt.unsqueeze(-1) if gt.size(1) == H
                     else gt.view(qlen, H, -1))
        out[start:start + qlen] = o.to(out.dtype)


# ---------------------------------------------------------------------
# Post-norm residual with a (1 + w) RMS norm, short causal convolutions
# with a per-sequence tail, matrix-memory recurrences (gated linear
# attention, gated delta rule, mLSTM), per-head output norm + gate, and
# group-limited softmax routing with clamped gated experts.
# ---------------------------------------------------------------------

def postln_rmsnorm_residual(x_res: torch.Tensor, y, y_scale: float, y2,
                            y2_scale: float, alpha: float, row_add,
                            w1p: torch.Tensor, eps: float,
                            h_out: torch.Tensor) -> None:
    """s = (alpha + row_add[t]) * x + y_scale * y + y2_scale * y2;
    x <- s / sqrt(mean(s^2) + eps) * w1p; h_out = x in the compute dtype.
    x_res is the fp32 residual (rewritten); y, y2, row_add may be None;
    w1p holds 1 + w."""
    a = x_res.new_full((x_res.size(0), 1), float(alpha))
    if row_add is not None:
        a = a + row_add.float().view(-1, 1)
    s = x_res * a
    if y is not None:
        s = s + y.float() * y_scale
    if y2 is not None:
        s = s + y2.float() * y2_scale
    r = s * torch.rsqrt(s.pow(2).mean(-1, keepdim=True) + eps) * w1p.float()
    x_res.copy_(r)
    h_out.copy_(r.to(h_out.dtype))


def _step_rows(b: int, seq_lens, query_starts, query_lens):
    """(first row, row count, position of the first row) of sequence b in a
    step; query_starts / query_lens None = one new token per sequence."""
    total = int(seq_lens[b])
    if query_lens is None:
        return b, 1, total - 1
    n = int(query_lens[b])
    return int(query_starts[b]), n, total - n


def short_conv_state(out: torch.Tensor, u: torch.Tensor, w: torch.Tensor,
                     tail: torch.Tensor, state_slots: torch.Tensor,
                     seq_lens, query_starts, query_lens, silu: bool,
                     norm_channels: int, head_dim: int, lead_channels: int,
                     lead_scale: float, l2_eps: float) -> None:
    """Depthwise causal convolution over time with the last taps-1 inputs
    of every sequence kept in tail [slots, taps-1, C] (fp32).

    y[t, c] = sum_j w[j, c] * u[t - taps + 1 + j, c] (w is tap-major,
    [taps, C]); inputs before this
    step's rows come from the tail, inputs before position 0 are zero (a
    sequence whose first row sits at position 0 ignores its tail). Then
    optionally silu, and for the first norm_channels channels, cut into
    heads of head_dim, y / sqrt(sum(y^2) + l2_eps); the first lead_channels
    of those are multiplied by lead_scale. The tail is rewritten."""
    taps = w.size(0)
    wf = w.float()
    for b in range(seq_lens.numel()):
        s0, n, pos0 = _step_rows(b, seq_lens, query_starts, query_lens)
        if n <= 0:
            continue
        slot = int(state_slots[b])
        hist = tail[slot].float().clone()
        hist[:max(0, taps - 1 - max(pos0, 0))] = 0      # before position 0
        full = torch.cat([hist, u[s0:s0 + n].float()], dim=0)
        y = torch.zeros(n, u.size(1))
        for j in range(taps):
            y = y + wf[j] * full[j:j + n]
        if taps > 1:
            tail[slot] = full[-(taps - 1):]
        if silu:
            y = y * torch.sigmoid(y)
        if norm_channels > 0:
            yh = y[:, :norm_channels].reshape(n, -1, head_dim)
            yh = yh / torch.sqrt(yh.pow(2).sum(-1, keepdim=True) + l2_eps)
            y[:, :norm_channels] = yh.reshape(n, norm_channels)
            y[:, :lead_channels] = y[:, :lead_channels] * lead_scale
        out[s0:s0 + n] = y.to(out.dtype)


SCAN_GLA, SCAN_DELTA, SCAN_MLSTM = 0, 1, 2


def matrix_memory_scan(kind: int, out: torch.Tensor, q: torch.Tensor,
                       k: torch.Tensor, v: torch.Tensor, gate: torch.Tensor,
                       gate_bias, head_rate, beta, q_scale: float,
                       gate_param: float, S: torch.Tensor, n_state, m_state,
                       state_slots: torch.Tensor, seq_lens, query_starts,
                       query_lens) -> None:
    """Token-by-token matrix-memory recurrences over per-sequence state.

    q, k [T, G, D]; v [T, H, Dv]; out [T, H, Dv] fp32; head h reads q/k
    head h // (H/G). S [slots, H, Dv, D] fp32 holds every head's memory
    transposed (one row per value coordinate). A sequence whose first row
    sits at position 0 starts from zero state. q is multiplied by q_scale.

    SCAN_GLA:   a = exp(logsigmoid(gate + gate_bias) * gate_param), per key
                channel (gate [T, H*D]); S <- a S + k v^T; o = S^T q.
    SCAN_DELTA: g = exp(-exp(head_rate[h]) * softplus(gate + gate_bias)),
                b = sigmoid(beta[t, h]); S <- g S; u = b (v - S^T k);
                S <- S + k u^T; o = S^T q.
    SCAN_MLSTM: gate [T, 2H] = log-input | forget pre-activations,
                i = c tanh((gate_i + bias_i) / c), f = logsigmoid(c tanh(
                (gate_f + bias_f) / c)), c = gate_param; m' = max(f + m, i);
                S <- e^(f+m-m') S + e^(i-m') k v^T, n likewise with k;
                o = S^T q / (max(|n.q|, e^(-m')) + 1e-6).
                n_state [slots, H, D], m_state [slots, H]."""
    H, Dv = v.size(1), v.size(2)
    G, D = k.size(1), k.size(2)
    rep = H // G
    gb = gate_bias.float() if gate_bias is not None else None
    lsig = torch.nn.functional.logsigmoid
    for b in range(seq_lens.numel()):
        s0, n, pos0 = _step_rows(b, seq_lens, query_starts, query_lens)
        if n <= 0:
            continue
        slot = int(state_slots[b])
        fresh = pos0 <= 0
        St = torch.zeros(H, Dv, D) if fresh else S[slot].clone()
        if kind == SCAN_MLSTM:
            nv = torch.zeros(H, D) if fresh else n_state[slot].clone()
            mv = torch.zeros(H) if fresh else m_state[slot].clone()
        for t in range(s0, s0 + n):
            qt = q[t].float().repeat_interleave(rep, 0) * q_scale   # [H, D]
            kt = k[t].float().repeat_interleave(rep, 0)
            vt = v[t].float()                                       # [H, Dv]
            z = gate[t].float()
            if kind == SCAN_GLA:
                a = torch.exp(lsig(z + gb) * gate_param).view(H, D)
                St = St * a.unsqueeze(1) + vt.unsqueeze(2) * kt.unsqueeze(1)
                out[t] = torch.einsum("hvd,hd->hv", St, qt)
            elif kind == SCAN_DELTA:
                g = torch.exp(-torch.exp(head_rate.float()).view(H, 1)
                              * torch.nn.functional.softplus(
                                  (z + gb).view(H, D)))
                St = St * g.unsqueeze(1)
                bt = torch.sigmoid(beta[t].float()).view(H, 1)
                u = bt * (vt - torch.einsum("hvd,hd->hv", St, kt))
                St = St + u.unsqueeze(2) * kt.unsqueeze(1)
                out[t] = torch.einsum("hvd,hd->hv", St, qt)
            else:
                c = gate_param
                zb = z + gb
                ig = c * torch.tanh(zb[:H] / c)
                fg = lsig(c * torch.tanh(zb[H:] / c))
                mn = torch.maximum(fg + mv, ig)
                df = torch.exp(fg + mv - mn).view(H, 1)
                di = torch.exp(ig - mn).view(H, 1)
                St = (St * df.unsqueeze(2)
                      + (di * vt).unsqueeze(2) * kt.unsqueeze(1))
                nv = nv * df + di * kt
                mv = mn
                den = torch.maximum((nv * qt).sum(-1).abs(),
                                    torch.exp(-mv)) + 1e-6
                out[t] = torch.einsum("hvd,hd->hv", St, qt) / den.view(H, 1)
        S[slot] = St
        if kind == SCAN_MLSTM:
            n_state[slot] = nv
            m_state[slot] = mv


def head_rmsnorm_gate(out: torch.Tensor, o: torch.Tensor, w: torch.Tensor,
                      gate: torch.Tensor, eps: float, silu_gate: bool) -> None:
    """out[t, h*Dv + e] = o[t, h, e] / rms_e(o[t, h]) * w * act(gate):
    o fp32 [T, H, Dv]; w has Dv entries (shared by the heads) or H*Dv;
    act = silu or sigmoid of gate [T, H*Dv]."""
    T, H, Dv = o.shape
    r = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)
    wf = w.float()
    r = r * (wf.view(1, 1, Dv) if wf.numel() == Dv else wf.view(1, H, Dv))
    g = gate.float().reshape(T, H, Dv)
    a = g * torch.sigmoid(g) if silu_gate else torch.sigmoid(g)
    out.copy_((r * a).reshape(T, H * Dv).to(out.dtype))


def grouped_softmax_route(weight: torch.Tensor, logits: torch.Tensor,
                          correction, top: int, n_groups: int,
                          keep_groups: int, scale: float) -> None:
    """Dense routing weights [T, E] (0 = not chosen), fp32 throughout.
    s = softmax(logits); choice score c = s + correction; experts form
    n_groups equal consecutive groups, a group scores max(c) over its
    members and only the keep_groups best groups stay eligible; the `top`
    eligible experts with the largest c are chosen and weigh
    s / (sum of chosen s + 1e-20) * scale."""
    T, E = logits.shape
    s = torch.softmax(logits.float(), dim=-1)
    c = s if correction is None else s + correction.float()
    if n_groups > 1 and keep_groups < n_groups:
        gs = c.view(T, n_groups, E // n_groups).max(-1).values
        keep = torch.zeros(T, n_groups, dtype=torch.bool)
        keep.scatter_(1, gs.topk(keep_groups, dim=-1).indices, True)
        ok = keep.unsqueeze(-1).expand(T, n_groups, E // n_groups)
        c = c.masked_fill(~ok.reshape(T, E), float("-inf"))
    idx = c.topk(top, dim=-1).indices
    ws = s.gather(1, idx)
    ws = ws / (ws.sum(-1, keepdim=True) + 1e-20) * scale
    weight.zero_()
    weight.scatter_(1, idx, ws)


def routed_clamped_glu(out: torch.Tensor, gu: torch.Tensor,
                       weight: torch.Tensor, n_experts: int, limit: float,
                       slope: float) -> None:
    """Stacked-expert activation with the routing weight on the OUTPUT
    side: gu [T, E*2F] (expert e: gate | up), weight [T, >= E] (columns
    past n_experts belong to weightless experts and are ignored);
    g = min(gate, limit), u = clamp(up, -limit, limit);
    out[t, e, :] = weight[t, e] * g * sigmoid(slope * g) * (u + 1), and 0
    where the weight is 0."""
    T = gu.size(0)
    E = n_experts
    F_ = gu.size(1) // (2 * E)
    g3 = gu.view(T, E, 2 * F_).float()
    g = g3[..., :F_].clamp(max=limit)
    u = g3[..., F_:].clamp(-limit, limit)
    w = weight[:, :E].float().unsqueeze(-1)
    y = g * torch.sigmoid(slope * g) * (u + 1.0) * w
    y = torch.where(w == 0, torch.zeros_like(y), y)
    out.copy_(y.view(T, E * F_).to(out.dtype))


# ---------------------------------------------------------------------
# Hashed bigram embedding, sigmoid-gated residual with layer norm, xIELU,
# token-side gate, sigmoid group-limited routing with always-on experts,
# output-weighted gated experts with an odd-sized tail expert, latent
# rotary append, plain K/V append, elementwise output gate.
# ---------------------------------------------------------------------

UPDATE_NONE, UPDATE_SIGMOID_GATE, UPDATE_UNIT_RMS = 0, 1, 2


def bigram_embed(x_out: torch.Tensor, ids: torch.Tensor, embed: torch.Tensor,
                 bigram, scale: float, mul_prev: int, mul_cur: int,
                 buckets: int, prev_state, state_slots, seq_lens,
                 query_starts, query_lens) -> None:
    """x_out (fp32 [T, W]) = scale * embed[id] + bigram[row], row =
    (mul_prev * previous id + mul_cur * id) mod buckets; a sequence's first
    token (position 0) takes row `buckets`. The previous id of a portion's
    first row comes from prev_state [slots] (int32), which is rewritten
    with the portion's last id. bigram None: plain scaled embedding."""
    x_out.copy_(embed[ids].float() * scale)
    if bigram is None:
        return
    for b in range(seq_lens.numel()):
        s0, n, pos0 = _step_rows(b, seq_lens, query_starts, query_lens)
        if n <= 0:
            continue
        slot = int(state_slots[b])
        prev = int(prev_state[slot])
        for r in range(s0, s0 + n):
            tok = int(ids[r])
            if r == s0 and pos0 <= 0:
                row = buckets
            else:
                row = (prev * mul_prev + tok * mul_cur) % buckets
            x_out[r] += bigram[row].float()
            prev = tok
        prev_state[slot] = prev


def residual_update_norm(x_res: torch.Tensor, y, update: int, gate, gate_bias,
                         rms_w, eps: float, norm_w, norm_b,
                         h_out) -> None:
    """fp32 residual update fused with the norm that feeds the next GEMM.
    update: NONE; SIGMOID_GATE x += sigmoid(gate + gate_bias) * y;
    UNIT_RMS x += y / sqrt(mean(y^2) + eps) * rms_w. Then h_out = layer
    norm of x ((x - mean) / sqrt(var + eps) * norm_w + norm_b), or just x
    in h_out's dtype when norm_w is None; h_out None skips it."""
    if update == UPDATE_SIGMOID_GATE:
        g = gate.float()
        if gate_bias is not None:
            g = g + gate_bias.float()
        x_res.add_(torch.sigmoid(g) * y.float())
    elif update == UPDATE_UNIT_RMS:
        x_res.add_(_unit(y.float(), eps) * rms_w.float())
    if h_out is None:
        return
    if norm_w is None:
        h_out.copy_(x_res.to(h_out.dtype))
        return
    d = x_res - x_res.mean(-1, keepdim=True)
    r = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps)
    r = r * norm_w.float()
    if norm_b is not None:
        r = r + norm_b.float()
    h_out.copy_(r.to(h_out.dtype))


def xielu(out: torch.Tensor, z: torch.Tensor, coef: torch.Tensor) -> None:
    """coef = (a_pos, a_neg) fp32: z > 0 -> a_pos z^2 + z/2; z <= 0 ->
    a_neg (e^z - 1 - z) + z/2."""
    zf = z.float()
    zn = zf.clamp(max=0.0)
    out.copy_(torch.where(zf > 0, coef[0] * zf * zf + 0.5 * zf,
                          coef[1] * (torch.expm1(zn) - zn) + 0.5 * zn
                          ).to(out.dtype))


def gelu_gate_rows(out: torch.Tensor, t: torch.Tensor, table: torch.Tensor,
                   ids: torch.Tensor, col0: int) -> None:
    """out[r, d] = gelu_tanh(t[r, d]) * table[ids[r], col0 + d]."""
    z = t.float()
    g = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654
                                    * (z + 0.044715 * z * z * z)))
    e = table[ids, col0:col0 + t.size(1)].float()
    out.copy_((g * e).to(out.dtype))


def grouped_sigmoid_route(weight: torch.Tensor, logits: torch.Tensor,
                          correction, n_experts: int, top: int, n_groups: int,
                          keep_groups: int, group_top: int) -> None:
    """Dense routing weights [T, E + A] (0 = not chosen), fp32 throughout.
    s = sigmoid(logits); choice score c = s + correction (columns < E);
    experts form n_groups equal consecutive groups, a group scores the sum
    of its group_top largest c and only the keep_groups best groups stay
    eligible (the others count as -inf); the `top` eligible experts with
    the largest c weigh s, not renormalized. Columns >= E are always-on
    gates: weight = sigmoid(logit)."""
    T, E = logits.size(0), n_experts
    s_all = torch.sigmoid(logits.float())
    s = s_all[:, :E]
    c = s if correction is None else s + correction.float()
    if n_groups > 1 and keep_groups < n_groups:
        per = E // n_groups
        gs = c.view(T, n_groups, per).topk(min(group_top, per), dim=-1
                                           ).values.sum(-1)
        keep = torch.zeros(T, n_groups, dtype=torch.bool)
        keep.scatter_(1, gs.topk(keep_groups, dim=-1).indices, True)
        ok = keep.unsqueeze(-1).expand(T, n_groups, per)
        c = c.masked_fill(~ok.reshape(T, E), float("-inf"))
    idx = c.topk(top, dim=-1).indices
    weight.zero_()
    weight[:, :E].scatter_(1, idx, s.gather(1, idx))
    weight[:, E:] = s_all[:, E:]


def routed_silu_glu(out: torch.Tensor, gu: torch.Tensor, weight: torch.Tensor,
                    n_experts: int, ff: int, tail_ff: int) -> None:
    """Stacked gated experts with the routing weight on the OUTPUT side.
    gu [T, E*2F + 2Ft]: expert e owns gate | up at e*2F; a tail expert of
    inner size Ft (0 = none) follows at E*2F and is weighed by weight[:, E].
    out[t, e*F + f] = weight[t, e] * silu(gate) * up, 0 where the weight is
    0; out [T, E*F + Ft]."""
    T, E, F_ = gu.size(0), n_experts, ff
    g3 = gu[:, :E * 2 * F_].reshape(T, E, 2 * F_).float()
    g, u = g3[..., :F_], g3[..., F_:]
    w = weight[:, :E].float().unsqueeze(-1)
    y = g * torch.sigmoid(g) * u * w
    y = torch.where(w == 0, torch.zeros_like(y), y)
    out[:, :E * F_] = y.view(T, E * F_).to(out.dtype)
    if tail_ff > 0:
        tg = gu[:, E * 2 * F_:E * 2 * F_ + tail_ff].float()
        tu = gu[:, E * 2 * F_ + tail_ff:E * 2 * F_ + 2 * tail_ff].float()
        out[:, E * F_:] = (tg * torch.sigmoid(tg) * tu
                           * weight[:, E:E + 1].float()).to(out.dtype)


def latent_rotary_append(proj: torch.Tensor, heads: int, q_head: int,
                         q_rot_off: int, kv_off: int, kv_rank: int,
                         rot_dim: int, w_kv: torch.Tensor, eps: float,
                         cos_sin: torch.Tensor, cache: torch.Tensor,
                         slot_mapping: torch.Tensor) -> None:
    """One step's rows of a latent-attention input projection:
    proj[:, h*q_head + q_rot_off : +rot_dim] (every query head's rotated
    part) is rotated IN PLACE; proj[:, kv_off : kv_off+kv_rank] is
    RMS-normed with w_kv into cache[slot, :kv_rank]; the shared key part
    proj[:, kv_off+kv_rank : +rot_dim] is rotated into cache[slot,
    kv_rank : kv_rank+rot_dim]; the pool's remaining columns are zeroed.
    Rotation pairs coordinate i with i + half (cos_sin [T, 2*half] from
    rotary_table, 2*half <= rot_dim; the rest passes). slot < 0 skips the
    append."""
    T = proj.size(0)
    q = proj[:, :heads * q_head].view(T, heads, q_head)
    qr = q[:, :, q_rot_off:q_rot_off + rot_dim]
    qr.copy_(_rotate_half(qr.float(), cos_sin).to(proj.dtype))
    c = proj[:, kv_off:kv_off + kv_rank].float()
    c = (_unit(c, eps) * w_kv.float()).to(cache.dtype)
    kr = proj[:, kv_off + kv_rank:kv_off + kv_rank + rot_dim].float()
    kr = _rotate_half(kr.unsqueeze(1), cos_sin).squeeze(1).to(cache.dtype)
    Rp = cache.size(2)
    flat = cache.view(-1, Rp)
    ok = slot_mapping >= 0
    rows = slot_mapping[ok].long()
    flat[rows, :kv_rank] = c[ok]
    flat[rows, kv_rank:kv_rank + rot_dim] = kr[ok]
    if Rp > kv_rank + rot_dim:
        flat[rows, kv_rank + rot_dim:] = 0


def head_kv_append(k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
              v_cache: torch.Tensor, slot_mapping: torch.Tensor) -> None:
    """k [T, G, D], v [T, G, Dv] -> pools [P, G, PS, D] / [P, G, PS, Dv] at
    slot = page*PS + offset (slot < 0 skips)."""
    PS = k_cache.size(2)
    ok = slot_mapping >= 0
    rows = slot_mapping[ok].long()
    page, off = rows // PS, rows % PS
    k_cache[page, :, off] = k[ok].to(k_cache.dtype)
    v_cache[page, :, off] = v[ok].to(v_cache.dtype)


def sigmoid_gate_rows(out: torch.Tensor, a: torch.Tensor,
                      gate: torch.Tensor) -> None:
    """out[t, c] = a[t, c] * sigmoid(gate[t, c])."""
    out.copy_((a.float() * torch.sigmoid(gate.float())).to(out.dtype))
