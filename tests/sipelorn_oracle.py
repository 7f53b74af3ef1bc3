"""Plain, slow float64 oracle for the Sipelorn design — one function per
mechanism, written from the design's equations and sharing no code with
the serving path (no cache manager, no state slots, no batching, no
kernels, no absorbed or re-ordered weights). Whole sequences only.

Notation: x is the residual stream [T, W]; linear weights are stored
[out, in] and applied as y = W x; t counts positions from 0; w maps tensor
names to float64 tensors.

  embedding   x_t = scale * embed[tok_t] + bigram[r_t],
              r_t = (mul_prev tok_(t-1) + mul_cur tok_t) mod buckets, and
              r_0 = buckets (the table's last row)
  layer       h = LN1(x); x += sigmoid(Rg1 h + b1) * mixer(h)
              h = LN2(x); x += sigmoid(Rg2 h + b2) * ff(h)
              then the token side input:
              e = side_embed[tok][i*d:(i+1)*d]; g = gelu_tanh(Sg x) * e;
              y = Sp g; x += y / rms(y) * s
  mixers      "attention": biased q/k/v -> short causal convolution ->
              scores q.k*scale - r1 ln(1 + r2 (i-j)) over a sliding window,
              softmax, elementwise sigmoid output gate; K/V may be borrowed
              from an earlier layer.
              "latent_attention": keys and values expanded from an
              RMS-normed latent, plus one rotated key part shared by all
              heads (interleaved pairs, YaRN-stretched), causal softmax.
  ff          dense xIELU, or sigmoid-routed experts with group-limited
              choice and a gated shared expert.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

F64 = torch.float64


# ----------------------------------------------------------------- pieces

def rms_unit(v, eps):
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, wt, bias, eps):
    mu = x.mean(dim=-1, keepdim=True)
    d = x - mu
    var = (d * d).mean(dim=-1, keepdim=True)
    return d / torch.sqrt(var + eps) * wt + bias


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def softplus(v):
    return torch.log1p(torch.exp(v))


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (e^z - 1 - z)
    + z/2."""
    ap = softplus(p)
    an = 0.5 + softplus(q)
    zn = torch.clamp(z, max=0.0)
    return torch.where(z > 0, ap * z * z + 0.5 * z,
                       an * (torch.exp(zn) - 1.0 - zn) + 0.5 * zn)


def bigram_rows(tokens: List[int], bg: dict) -> List[int]:
    rows = []
    for t, tok in enumerate(tokens):
        if t == 0:
            rows.append(bg["buckets"])
        else:
            rows.append((tokens[t - 1] * bg["mul_prev"] + tok * bg["mul_cur"])
                        % bg["buckets"])
    return rows


def embed_tokens(tokens: List[int], w, cfg: dict):
    em = cfg.get("embedding") or {}
    x = w["embed"][tokens] * float(em.get("scale", 1.0))
    if em.get("bigram"):
        x = x + w["bigram"][bigram_rows(tokens, em["bigram"])]
    return x


def causal_conv(u, cw):
    """u [T, C], cw [C, taps]: y_t = sum_j cw[:, j] u_(t - taps + 1 + j), zeros
    before the sequence's start (the last column weighs the current token)."""
    taps = cw.shape[1]
    y = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += cw[:, j] * u[s]
    return y


def yarn_frequencies(dims: int, base: float, sc: Optional[dict]):
    """(list of dims/2 angular frequencies, amplitude on cos and sin)."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(t):
        return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(sc["fast"])), 0)
    hi = min(math.ceil(turn_dim(sc["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_interleaved(v, rot: dict):
    """v [T, ..., D]: coordinates 2i and 2i+1 (i < dims/2) of the last axis
    rotate by t * f_i; the rest pass."""
    dims = int(rot["dims"])
    freqs, amp = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    out = v.clone()
    for t in range(v.shape[0]):
        for i in range(dims // 2):
            a = t * freqs[i]
            c, s = math.cos(a) * amp, math.sin(a) * amp
            p, q = v[t, ..., 2 * i], v[t, ..., 2 * i + 1]
            out[t, ..., 2 * i] = p * c - q * s
            out[t, ..., 2 * i + 1] = q * c + p * s
    return out


# ----------------------------------------------------------------- mixers

def conv_keys_values(h, w, p, mx):
    """Keys and values of an "attention" layer as its cache holds them
    (after the projection's bias and the convolution)."""
    T = h.shape[0]
    G, D, Dv = mx["kv_heads"], mx["dim"], mx["vdim"]
    k = causal_conv(h @ w[p + "k"].T + w[p + "k.b"], w[p + "k.conv"])
    v = causal_conv(h @ w[p + "v"].T + w[p + "v.b"], w[p + "v.conv"])
    return k.view(T, G, D), v.view(T, G, Dv)


def biased_window_softmax(q, k, v, scale, size, r1, r2):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; query i of head hd sees keys
    j with 0 <= i - j < size and scores q.k * scale - r1[hd] ln(1 + r2[hd]
    (i - j)); softmax over the seen keys. Returns [T, H, Dv]."""
    T, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            j0 = max(0, i - size + 1)
            dist = torch.arange(i - j0, -1, -1, dtype=F64)      # i - j
            sc = (k[j0:i + 1, g] @ q[i, hd]) * scale \
                - float(r1[hd]) * torch.log1p(float(r2[hd]) * dist)
            out[i, hd] = torch.softmax(sc, dim=0) @ v[j0:i + 1, g]
    return out


def window_attention(h, w, p, mx, kv=None):
    """kv: (k, v) borrowed from another layer, or None to make its own.
    Returns (mixer output, (k, v))."""
    T = h.shape[0]
    H, D, Dv = mx["heads"], mx["dim"], mx["vdim"]
    q = causal_conv(h @ w[p + "q"].T + w[p + "q.b"],
                    w[p + "q.conv"]).view(T, H, D)
    k, v = kv if kv is not None else conv_keys_values(h, w, p, mx)
    out = biased_window_softmax(q, k, v, mx["scale"], int(mx["mask"]["size"]),
                                w[p + "r1"], w[p + "r2"])
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return (out.reshape(T, H * Dv) * gate) @ w[p + "o"].T, (k, v)


def latent_attention(h, w, p, mx, eps):
    T = h.shape[0]
    H, D, Dr, Dv, R = (mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"],
                       mx["kv_rank"])
    q = (h @ w[p + "q"].T).view(T, H, D + Dr)
    q_plain, q_rot = q[..., :D], rotate_interleaved(q[..., D:], mx["rot"])
    dkv = h @ w[p + "dkv"].T
    c = rms_unit(dkv[:, :R], eps) * w[p + "dkv.norm"]
    k_rot = rotate_interleaved(dkv[:, R:], mx["rot"])            # [T, Dr]
    k_plain = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for hd in range(H):
        for i in range(T):
            sc = (k_plain[:i + 1, hd] @ q_plain[i, hd]
                  + k_rot[:i + 1] @ q_rot[i, hd]) * mx["scale"]
            out[i, hd] = torch.softmax(sc, dim=0) @ v[:i + 1, hd]
    return out.reshape(T, H * Dv) @ w[p + "o"].T


# ----------------------------------------------------------- feed-forward

def dense_ff(h, w, p):
    a = w[p + "act"]
    return xielu(h @ w[p + "up"].T, a[0], a[1]) @ w[p + "down"].T


def gated_expert(h, w, p):
    g = h @ w[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, w, p, r):
    """Per token the chosen experts and their weights: [(expert, weight)]."""
    E, top = int(r["experts"]), int(r["top"])
    grp = r.get("groups") or {}
    n_groups, keep = int(grp.get("count", 1)), int(grp.get("keep", 1))
    s = torch.sigmoid(h @ w[p + "router"].T)
    choice = s + w[p + "correction"]
    out = []
    per = E // n_groups
    for t in range(h.shape[0]):
        c = choice[t].tolist()
        gscore = []
        for g in range(n_groups):
            best = sorted(c[g * per:(g + 1) * per], reverse=True)[:2]
            gscore.append(sum(best))
        kept = sorted(range(n_groups), key=lambda g: (-gscore[g], g))[:keep]
        cand = [e for e in range(E) if e // per in kept]
        cand.sort(key=lambda e: (-c[e], e))
        out.append([(e, s[t, e]) for e in cand[:top]])
    return out


def expert_mixture(h, w, p, ml):
    y = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F64)
    for t, chosen in enumerate(route(h, w, p, ml["router"])):
        for e, wt in chosen:
            y[t] += wt * gated_expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if ml.get("shared"):
        y = y + torch.sigmoid(h @ w[p + "shared.sg"].T) \
            * gated_expert(h, w, p + "shared.")
    return y


def token_side(x, tokens, w, i, dim, eps):
    e = w["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ w[f"l{i}.side.gate"].T) * e
    y = g @ w[f"l{i}.side.proj"].T
    return x + rms_unit(y, eps) * w[f"l{i}.side.norm"]


# ---------------------------------------------------------------- forward

def forward(tokens: List[int], weights: Dict[str, torch.Tensor], cfg: dict,
            trace: Optional[list] = None):
    """Logits [T, vocab] of one whole sequence; `trace` (a list) receives the
    residual stream after every layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    side = (cfg.get("token_side") or {}).get("dim", 0)
    x = embed_tokens(tokens, w, cfg)
    kvs = {}
    for i, layer in enumerate(cfg["layers"]):
        L, p, mx = f"l{i}.", f"l{i}.mix.", layer["mixer"]
        h = layer_norm(x, w[L + "norm1"], w[L + "norm1.b"], eps)
        if layer["type"] == "attention":
            src = mx.get("kv_from")
            y, kvs[i] = window_attention(h, w, p, mx,
                                         None if src is None else kvs[src])
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, w, p, mx, eps)
        else:
            raise ValueError(layer["type"])
        x = x + torch.sigmoid(h @ w[L + "rg1"].T + w[L + "rg1.b"]) * y
        ml = layer.get("mlp")
        if ml is not None:
            h = layer_norm(x, w[L + "norm2"], w[L + "norm2.b"], eps)
            f = (dense_ff(h, w, L + "mlp.") if ml["kind"] == "dense"
                 else expert_mixture(h, w, L + "mlp.", ml))
            x = x + torch.sigmoid(h @ w[L + "rg2"].T + w[L + "rg2.b"]) * f
        if side:
            x = token_side(x, tokens, w, i, side, eps)
        if trace is not None:
            trace.append(x.clone())
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return x @ w["head"].T


# ----------------------------------------------- small random checkpoints

def latent_mixer(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24,
                 scale=None, base=10000.0, scaling=None):
    return {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
        "kv_rank": kv_rank,
        "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
        "rot": {"base": base, "dims": rot_dim,
                **({"scaling": scaling} if scaling else {})}}}


def window_mixer(heads=4, kv_heads=2, dim=16, vdim=16, window=12, conv=3,
                 scale=None, kv_from=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
          "conv": conv, "mask": {"size": window},
          "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        mx["kv_from"] = kv_from
    return {"type": "attention", "mixer": mx}


def dense_mlp(ff=64):
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts=8, top=2, ff=16, groups=2, keep=1, shared_ff=24):
    ml = {"kind": "moe", "expert": {"ff": ff},
          "router": {"experts": experts, "top": top,
                     "groups": {"count": groups, "keep": keep}}}
    if shared_ff:
        ml["shared"] = {"ff": shared_ff}
    return ml


def make_config(layers, vocab=96, width=64, eps=1e-5, side_dim=8,
                embed_scale=4.0, bigram=(53, 7, 11)) -> dict:
    """layers: [(mixer dict from latent_mixer/window_mixer, mlp dict or
    None)]."""
    cfg = {"architecture": "Sipelorn", "vocab": vocab, "width": width,
           "norm": {"eps": eps},
           "embedding": {"scale": embed_scale},
           "layers": [dict(m, mlp=ml) for m, ml in layers]}
    if bigram:
        cfg["embedding"]["bigram"] = {"buckets": bigram[0],
                                      "mul_prev": bigram[1],
                                      "mul_cur": bigram[2]}
    if side_dim:
        cfg["token_side"] = {"dim": side_dim}
    return cfg


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random weights (values representable in bf16) for a config dict."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(rows, cols, gain=1.0):
        return (torch.randn(rows, cols, generator=g) * gain / math.sqrt(cols)
                ).bfloat16().float()

    def vec(n, mean=0.0, std=0.1):
        return (mean + torch.randn(n, generator=g) * std).bfloat16().float()

    w = {"embed": mat(V, W, math.sqrt(W) * 0.3), "head": mat(V, W),
         "final.norm": vec(W, 1.0), "final.norm.b": vec(W, 0.0, 0.05)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        w["bigram"] = mat(bg["buckets"] + 1, W, math.sqrt(W) * 0.5)
    side = (cfg.get("token_side") or {}).get("dim", 0)
    n_layers = len(cfg["layers"])
    if side:
        w["side.embed"] = mat(V, side * n_layers, math.sqrt(side * n_layers))
    for i, layer in enumerate(cfg["layers"]):
        L, p, mx = f"l{i}.", f"l{i}.mix.", layer["mixer"]
        w[L + "norm1"] = vec(W, 1.0)
        w[L + "norm1.b"] = vec(W, 0.0, 0.05)
        w[L + "rg1"] = mat(W, W)
        w[L + "rg1.b"] = vec(W, 0.5, 0.3)
        if layer["type"] == "attention":
            H, G, D, Dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            names = [("q", H * D)]
            if mx.get("kv_from") is None:
                names += [("k", G * D), ("v", G * Dv)]
            for nm, rows in names:
                w[p + nm] = mat(rows, W, 2.0)
                w[p + nm + ".b"] = vec(rows, 0.0, 0.2)
                w[p + nm + ".conv"] = (torch.randn(rows, mx["conv"],
                                                   generator=g) * 0.6
                                       ).bfloat16().float()
            w[p + "r1"] = vec(H, 0.6, 0.3).abs()
            w[p + "r2"] = (vec(H, 0.5, 0.2).abs() + 0.05).bfloat16().float()
            w[p + "g"] = mat(H * Dv, W)
            w[p + "o"] = mat(W, H * Dv)
        else:
            H, D, Dr, Dv, R = (mx["heads"], mx["dim"], mx["rot_dim"],
                               mx["vdim"], mx["kv_rank"])
            w[p + "q"] = mat(H * (D + Dr), W, 2.0)
            w[p + "dkv"] = mat(R + Dr, W, 2.0)
            w[p + "dkv.norm"] = vec(R, 1.0)
            w[p + "uk"] = mat(H * D, R, 1.5)
            w[p + "uv"] = mat(H * Dv, R)
            w[p + "o"] = mat(W, H * Dv)
        ml = layer.get("mlp")
        if ml is not None:
            q = L + "mlp."
            w[L + "norm2"] = vec(W, 1.0)
            w[L + "norm2.b"] = vec(W, 0.0, 0.05)
            w[L + "rg2"] = mat(W, W)
            w[L + "rg2.b"] = vec(W, 0.5, 0.3)
            if ml["kind"] == "dense":
                w[q + "up"] = mat(ml["ff"], W, 1.5)
                w[q + "down"] = mat(W, ml["ff"])
                w[q + "act"] = vec(2, 0.3, 0.5)
            else:
                E, Fe = ml["router"]["experts"], ml["expert"]["ff"]
                # wide logits: choices do not sit on rounding-sized margins
                w[q + "router"] = mat(E, W, 4.0)
                w[q + "correction"] = vec(E, 0.0, 0.15)
                forms = [(f"e{e}.", Fe) for e in range(E)]
                if ml.get("shared"):
                    forms.append(("shared.", ml["shared"]["ff"]))
                    w[q + "shared.sg"] = mat(1, W, 2.0)
                for nm, ff in forms:
                    w[q + nm + "gate"] = mat(ff, W, 2.0)
                    w[q + nm + "up"] = mat(ff, W, 2.0)
                    w[q + nm + "down"] = mat(W, ff)
        if side:
            w[L + "side.gate"] = mat(side, W, 2.0)
            w[L + "side.proj"] = mat(W, side)
            w[L + "side.norm"] = vec(W, 0.5, 0.2)
    return w


def save_checkpoint(path: str, cfg: dict, weights: Dict[str, torch.Tensor]):
    """Write config.json + model.safetensors (bf16) into `path`."""
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.bfloat16().contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
