"""Plain, slow float64 oracle for the Pekarax design — one function per
mechanism, written from the design's equations and sharing no code with
the serving path (no cache manager, no state slots, no batching, no
kernels). Whole sequences only.

Notation: x is the residual stream [T, W]; linear weights are stored
[out, in] and applied as y = W x; t counts positions from 0.

A layer is normed AFTER the sum: x <- N1(alpha x + mixer(x)),
x <- N2(alpha x + ff(x)), N(s) = s / sqrt(mean(s^2) + eps) * (1 + w).
Mixers: "gla", "channel_delta", "parallel" (convolved softmax attention
beside an mLSTM memory). The feed-forward is a mixture of clamped gated
experts with group-limited routing and identity experts.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def unit_rms(v, eps):
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def offset_norm(s, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(s, eps) * (1.0 + w)


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros
    before the sequence's start (the last column weighs the current token)."""
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotate_leading(v, base, dims):
    """v [T, heads, D]: the first `dims` coordinates rotate, i paired with
    i + dims/2, by the angle t * base^(-2i/dims)."""
    half = dims // 2
    out = v.clone()
    for t in range(v.shape[0]):
        for i in range(half):
            a = t * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            p, q = v[t, :, i], v[t, :, i + half]
            out[t, :, i] = p * c - q * s
            out[t, :, i + half] = q * c + p * s
    return out


def conv_attention(h, w, p, mx, eps):
    """Causal softmax attention: projections -> short convolution ->
    rotary -> weightless unit rms of q and k -> scaled scores."""
    T = h.shape[0]
    H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    q = causal_conv(h @ w[p + "q"].T, w[p + "q.conv"]).view(T, H, D)
    k = causal_conv(h @ w[p + "k"].T, w[p + "k.conv"]).view(T, G, D)
    v = causal_conv(h @ w[p + "v"].T, w[p + "v.conv"]).view(T, G, Dv)
    rot = mx["rot"]
    q = unit_rms(rotate_leading(q, rot["base"], rot["dims"]), eps)
    k = unit_rms(rotate_leading(k, rot["base"], rot["dims"]), eps)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for t in range(T):
            sc = (k[:t + 1, g] @ q[t, hd]) * mx["scale"]
            out[t, hd] = torch.softmax(sc, dim=0) @ v[:t + 1, g]
    return out.reshape(T, H * Dv) @ w[p + "o"].T


def mlstm_memory(h, w, p, mx, eps):
    """mLSTM matrix memory with capped log gates and a running maximum
    that starts at 0."""
    T = h.shape[0]
    H, D, Dv, cap = mx["heads"], mx["dim"], mx["vdim"], mx["gate_cap"]
    q = (h @ w[p + "q"].T).view(T, H, D) / math.sqrt(D)
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, Dv)
    li = cap * torch.tanh((h @ w[p + "i"].T + w[p + "i.b"]) / cap)
    lf = torch.nn.functional.logsigmoid(
        cap * torch.tanh((h @ w[p + "f"].T + w[p + "f.b"]) / cap))
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        n = torch.zeros(D, dtype=F64)
        m = 0.0
        for t in range(T):
            m_new = max(float(lf[t, hd]) + m, float(li[t, hd]))
            keep = math.exp(float(lf[t, hd]) + m - m_new)
            take = math.exp(float(li[t, hd]) - m_new)
            S = keep * S + take * torch.outer(k[t, hd], v[t, hd])
            n = keep * n + take * k[t, hd]
            m = m_new
            den = max(abs(float(n @ q[t, hd])), math.exp(-m)) + 1e-6
            o[t, hd] = (S.T @ q[t, hd]) / den
    o = unit_rms(o, eps).reshape(T, H * Dv) * w[p + "norm"]
    return (o * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def gated_linear_attention(h, w, p, mx, eps):
    T = h.shape[0]
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, D) / math.sqrt(D)
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, Dv)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / mx["tau"]).view(T, H, D)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[t, hd].unsqueeze(1) * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps) * w[p + "norm"]
    return (o.reshape(T, H * Dv)
            * torch.nn.functional.silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def channel_delta(h, w, p, mx, eps):
    """Gated delta rule with one decay per head and key channel."""
    T = h.shape[0]
    H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
    silu = torch.nn.functional.silu

    def unit(v):
        return v / torch.sqrt((v * v).sum(-1, keepdim=True) + 1e-6)

    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, Dv)
    q, k = unit(q) / math.sqrt(D), unit(k)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    z = (h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]
    sp = torch.nn.functional.softplus(z).view(T, H, D)
    o = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        rate = math.exp(float(w[p + "A_log"][hd]))
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = torch.exp(-rate * sp[t, hd]).unsqueeze(1) * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            o[t, hd] = S.T @ q[t, g]
    o = unit_rms(o, eps) * w[p + "norm"]
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T)
    return (o.reshape(T, H * Dv) * gate) @ w[p + "o"].T


def route(h, w, p, r):
    """(indices [T, top], weights [T, top]) of the chosen experts."""
    total = r["experts"] + r["identity"]
    s = torch.softmax(h @ w[p + "router"].T, dim=-1)
    choice = s + w[p + "correction"]
    count = r["groups"]["count"]
    size = total // count
    idx_all, w_all = [], []
    for t in range(h.shape[0]):
        best = [max(float(choice[t, g * size + e]) for e in range(size))
                for g in range(count)]
        kept = sorted(range(count), key=lambda g: -best[g])[:r["groups"]["keep"]]
        cand = [e for e in range(total) if e // size in kept]
        cand.sort(key=lambda e: -float(choice[t, e]))
        chosen = cand[:r["top"]]
        ws = torch.stack([s[t, e] for e in chosen])
        idx_all.append(chosen)
        w_all.append(ws / (ws.sum() + 1e-20) * r["scale"])
    return idx_all, w_all


def experts(h, w, p, ml):
    r, lim = ml["router"], ml["expert"]["limit"]
    idx, ws = route(h, w, p, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(idx[t], ws[t]):
            if e >= r["experts"]:
                out[t] += wt * h[t]                      # identity expert
                continue
            g = torch.clamp(w[f"{p}e{e}.gate"] @ h[t], max=lim)
            u = torch.clamp(w[f"{p}e{e}.up"] @ h[t], -lim, lim)
            y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
            out[t] += wt * (w[f"{p}e{e}.down"] @ y)
    return out


def mixer(cfg, w, i, x):
    layer, eps = cfg["layers"][i], cfg["norm"]["eps"]
    p, mx = f"l{i}.mix.", layer["mixer"]
    if layer["type"] == "gla":
        return gated_linear_attention(x, w, p, mx, eps)
    if layer["type"] == "channel_delta":
        return channel_delta(x, w, p, mx, eps)
    if layer["type"] == "parallel":
        return (mx["left_scale"] * conv_attention(x, w, p + "left.", mx["left"], eps)
                + mx["right_scale"] * mlstm_memory(x, w, p + "right.", mx["right"], eps))
    raise ValueError(layer["type"])


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int],
            trace: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] (float32) of one whole sequence."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = w["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        x = offset_norm(alpha * x + mixer(cfg, w, i, x), w[f"l{i}.norm1"], eps)
        if layer["mlp"] is not None:
            x = offset_norm(alpha * x + experts(x, w, f"l{i}.mlp.", layer["mlp"]),
                            w[f"l{i}.norm2"], eps)
        if trace is not None:
            trace.append(x.float())
    return (offset_norm(x, w["final.norm"], eps) @ w["head"].T).float()


# ---- builders of small random configurations ------------------------------

def gla_layer(heads=2, dim=8, vdim=12, tau=8.0, rank=4):
    return {"type": "gla", "rank": rank,
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}}


def delta_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=4, rank=4, grank=5):
    return {"type": "channel_delta", "rank": rank, "grank": grank,
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": vdim, "conv": conv}}


def parallel_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, rot_dims=4,
                   base=100.0, scale=0.7, left_scale=0.75, right_scale=1.2,
                   m_heads=2, m_dim=8, m_vdim=10, cap=8.0):
    return {"type": "parallel", "mixer": {
        "left": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                 "vdim": vdim, "conv": conv, "scale": scale,
                 "rot": {"base": base, "dims": rot_dims}},
        "right": {"heads": m_heads, "dim": m_dim, "vdim": m_vdim,
                  "gate_cap": cap},
        "left_scale": left_scale, "right_scale": right_scale}}


def moe(experts=6, identity=2, top=3, ff=10, limit=1.5, groups=4, keep=2,
        scale=1.7):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "identity": identity, "top": top,
                       "scale": scale,
                       "groups": {"count": groups, "keep": keep}}}


def make_config(layers, width=32, vocab=97, eps=1e-5, alpha=2.0, mlp=None,
                no_ff=()) -> dict:
    out = []
    for i, l in enumerate(layers):
        l = dict(l)
        if "mlp" not in l:
            l["mlp"] = None if i in no_ff else (mlp or moe())
        out.append(l)
    return {"architecture": "Pekarax", "vocab": vocab, "width": width,
            "postln_alpha": alpha, "norm": {"eps": eps}, "layers": out}


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """bf16-representable fp32 weights named as the checkpoint names them.
    The low-rank sizes ("rank", "grank" of a layer entry) exist only as
    tensor shapes, as in a checkpoint."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, std=1.0):
        return (torch.randn(o, i, generator=g) * std / math.sqrt(i)
                ).bfloat16().float()

    def vec(n, mean=0.0, dev=0.3):
        return (mean + dev * torch.randn(n, generator=g)).bfloat16().float()

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).bfloat16().float(),
         "final.norm": vec(W), "head": mat(cfg["vocab"], W)}

    def conv_w(c, taps):
        return (torch.randn(c, taps, generator=g) * 0.6).bfloat16().float()

    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.mix.", layer["mixer"]
        w[f"l{i}.norm1"] = vec(W)
        if layer["type"] == "parallel":
            a, pl = mx["left"], p + "left."
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for nm, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                w[pl + nm] = mat(rows, W, 2.0)
                w[pl + nm + ".conv"] = conv_w(rows, a["conv"])
            w[pl + "o"] = mat(W, H * Dv)
            r, pr = mx["right"], p + "right."
            H, D, Dv = r["heads"], r["dim"], r["vdim"]
            w[pr + "q"] = mat(H * D, W)
            w[pr + "k"] = mat(H * D, W)
            w[pr + "v"] = mat(H * Dv, W)
            w[pr + "g"] = mat(H * Dv, W)
            w[pr + "o"] = mat(W, H * Dv)
            w[pr + "norm"] = vec(H * Dv, 1.0)
            w[pr + "i"] = mat(H, W, 3.0)
            w[pr + "f"] = mat(H, W, 3.0)
            w[pr + "i.b"] = vec(H, 0.0, 1.0)
            w[pr + "f.b"] = vec(H, 2.0, 1.0)
        elif layer["type"] == "gla":
            H, D, Dv, r = mx["heads"], mx["dim"], mx["vdim"], layer["rank"]
            w[p + "q"] = mat(H * D, W)
            w[p + "k"] = mat(H * D, W)
            w[p + "v"] = mat(H * Dv, W)
            w[p + "g"] = mat(H * Dv, W)
            w[p + "o"] = mat(W, H * Dv)
            w[p + "norm"] = vec(Dv, 1.0)
            w[p + "a1"] = mat(r, W)
            w[p + "a2"] = mat(H * D, r, 2.0)
            w[p + "a2.b"] = vec(H * D, 1.0, 1.0)
        else:
            H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            r, rg = layer["rank"], layer["grank"]
            for nm, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                w[p + nm] = mat(rows, W, 2.0)
                w[p + nm + ".conv"] = conv_w(rows, mx["conv"])
            w[p + "b"] = mat(H, W, 2.0)
            w[p + "A_log"] = vec(H, -1.0, 0.7)
            w[p + "norm"] = vec(Dv, 1.0)
            w[p + "a1"] = mat(r, W)
            w[p + "a2"] = mat(H * D, r, 2.0)
            w[p + "dt_bias"] = vec(H * D, 0.0, 1.0)
            w[p + "g1"] = mat(rg, W)
            w[p + "g2"] = mat(H * Dv, rg, 2.0)
            w[p + "o"] = mat(W, H * Dv)
        ml = layer["mlp"]
        if ml is None:
            continue
        q = f"l{i}.mlp."
        r = ml["router"]
        w[f"l{i}.norm2"] = vec(W)
        w[q + "router"] = mat(r["experts"] + r["identity"], W, 2.0)
        w[q + "correction"] = vec(r["experts"] + r["identity"], -0.05, 0.1)
        for e in range(r["experts"]):
            w[f"{q}e{e}.gate"] = mat(ml["expert"]["ff"], W, 2.0)
            w[f"{q}e{e}.up"] = mat(ml["expert"]["ff"], W, 2.0)
            w[f"{q}e{e}.down"] = mat(W, ml["expert"]["ff"])
    return w


def checkpoint_config(cfg: dict) -> dict:
    """The config as a checkpoint's config.json holds it (the builders'
    low-rank sizes are not part of it)."""
    out = dict(cfg)
    out["layers"] = [{k: v for k, v in l.items() if k not in ("rank", "grank")}
                     for l in cfg["layers"]]
    return out


def save_checkpoint(path: str, cfg: dict, weights: Dict[str, torch.Tensor]):
    """Write config.json + model.safetensors (bf16) into `path`."""
    import json
    import os

    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(checkpoint_config(cfg), f)
    save_file({k: v.bfloat16().contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
