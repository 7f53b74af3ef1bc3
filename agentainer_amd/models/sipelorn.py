"""Sipelorn family — pre-normed decoder with gated residuals, a hashed
bigram embedding, per-layer token inputs, two attention mixers and
group-routed experts.

Every layer updates an fp32 residual stream x; LN is a layer norm with
weight and bias:

    h = LN1(x);  x <- x + sigmoid(Rg1 h + b1) * mixer(h)
    h = LN2(x);  x <- x + sigmoid(Rg2 h + b2) * ff(h)
    e = side_embed[token][i*d : (i+1)*d];  g = gelu_tanh(Sg x) * e
    y = Sp g;    x <- x + y / rms(y) * s                  (layer i's slice)

The stream starts as scale * embed[token] + bigram[row], row = (mul_prev *
previous token + mul_cur * token) mod buckets (the table's last row for a
sequence's first token). The layer list of config.json picks per layer:

  * "attention"        grouped-query attention: biased q/k/v, a short
    causal convolution over time on each, no rotation; every score loses
    r1 ln(1 + r2 * distance) (two numbers per head); sliding window;
    softmax; a sigmoid gate per output coordinate read from the mixer
    input. With `kv_from: j` the layer has no keys and values of its own
    and attends layer j's cached ones with its own queries.
  * "latent_attention" keys and values are expanded from one RMS-normed
    latent per token; a second, rotated key part (interleaved pairs,
    YaRN-stretched frequencies) is shared by all heads; causal softmax.

and a feed-forward: dense down(xIELU(up h)), or sigmoid-scored experts
with a choice-only correction, group-limited top-k (a group scores the sum
of its two best), un-renormalized weights and a shared expert behind a
per-token sigmoid gate.

Serving design (what runs on the MI355X):

  * Everything that reads one sublayer input rides in ONE GEMM: q | k | v
    | output gate | residual gate for the mixers, every expert's gate|up |
    the shared expert's | residual gate for the feed-forward.
  * ops.residual_update_norm fuses the gated (or unit-rms) fp32 residual
    update with the layer norm that feeds the next GEMM.
  * "attention" layers reuse the masked-attention kernels (distance bias
    as an argument) over HeadKV pools; a borrowing layer is handed its
    source layer's pools, so shared keys cost no memory and no append.
  * "latent_attention" runs in the latent basis: the key up-projection is
    folded into the query, the pool row is [latent | rotated key part] and
    the latent-attention kernels treat it as K = V (the value up-projection
    has zero rows for the rotated columns). The checkpoint's interleaved
    rotary pairs are re-ordered to (i, i + half) at load — a permutation of
    q and k rows that leaves every score unchanged.
  * The previous token id and the convolution tails are per-sequence state
    owned by the engine's KVCacheManager (HybridStateLayout).

compute dtype: bf16 (serving default; positions, angles, scores, softmax,
norms, router and the residual stay fp32) or float32 (everything fp32 — a
verification mode).
"""

from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from .llama import AttnMetadata
from .volalorn import MaskedAttention, MaskedAttentionConfig, _align, _param

RANK_ALIGN = 32          # the latent kernels contract the pool row by 32s
CAUSAL_WINDOW = 1 << 30  # a window no sequence outgrows
GROUP_TOP = 2            # a group scores the sum of its two best experts


@dataclass
class RotaryLatentConfig:
    heads: int
    dim: int                  # unrotated query/key size per head
    rot_dim: int              # rotated query/key size (key part is shared)
    vdim: int
    kv_rank: int
    scale: float
    rot_dims: int             # leading coordinates of the rotated part
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None   # YaRN: factor, original, fast, slow

    @property
    def padded_rank(self) -> int:
        n = self.kv_rank + self.rot_dim
        return -(-n // RANK_ALIGN) * RANK_ALIGN


@dataclass
class SipelornFeedForwardConfig:
    kind: str                 # "dense" | "moe"
    ff: int                   # inner size (per expert for moe)
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep_groups: int = 1
    shared_ff: int = 0        # 0: no shared expert


@dataclass
class SipelornLayerConfig:
    kind: str
    attn: Optional[MaskedAttentionConfig] = None
    latent: Optional[RotaryLatentConfig] = None
    mlp: Optional[SipelornFeedForwardConfig] = None


@dataclass
class SipelornConfig:
    name: str = "tiny-sipelorn"
    vocab_size: int = 512
    hidden_size: int = 128
    layers: List[SipelornLayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-6
    embed_scale: float = 1.0
    bigram_buckets: int = 0   # 0: no bigram table
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0
    side_dim: int = 0         # 0: no per-layer token input
    family: str = "sipelorn"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def max_position(self) -> int:
        return 1 << 30

    def _kv_shapes(self):
        out = []
        for l in self.layers:
            if l.latent is not None:
                out.append((l.latent.padded_rank,))
            elif l.attn.kv_from is None:
                out.append((l.attn.kv_heads, l.attn.dim, l.attn.vdim))
            else:
                out.append(None)
        return out

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(s[0] if len(s) == 1 else s[0] * (s[1] + s[2])
                   for s in self._kv_shapes() if s is not None) * dtype_bytes

    def state_shapes(self) -> List[Dict[str, tuple]]:
        out = []
        for i, l in enumerate(self.layers):
            d: Dict[str, tuple] = {}
            a = l.attn
            if a is not None and a.conv_taps > 0:
                ch = a.heads * a.dim
                if a.kv_from is None:
                    ch += a.kv_heads * (a.dim + a.vdim)
                d["conv"] = (a.conv_taps - 1, ch)
            if i == 0:
                d["prev_token"] = ()
            out.append(d)
        return out

    def cache_layout(self):
        from ..engine.kvcache import HybridStateLayout
        shapes = self.state_shapes()
        return HybridStateLayout(
            self._kv_shapes(), shapes,
            [{"prev_token": torch.int32} if "prev_token" in d else {}
             for d in shapes])

    def state_bytes_per_seq(self) -> int:
        return self.cache_layout().state_bytes_per_seq()


def config_from_dict(d: dict, name: str = "sipelorn") -> SipelornConfig:
    """SipelornConfig from a parsed config.json."""
    layers: List[SipelornLayerConfig] = []
    for i, ld in enumerate(d["layers"]):
        kind, mx = ld["type"], ld["mixer"]
        lc = SipelornLayerConfig(kind)
        if kind == "attention":
            src = mx.get("kv_from")
            lc.attn = MaskedAttentionConfig(
                heads=int(mx["heads"]), kv_heads=int(mx["kv_heads"]),
                dim=int(mx["dim"]), vdim=int(mx["vdim"]),
                scale=float(mx["scale"]), mask_kind=ops.MASK_WINDOW,
                mask_size=int(mx["mask"]["size"]), qkv_bias=True,
                conv_taps=int(mx.get("conv") or 0), plain_qk=True,
                dist_bias=True, elem_gate=True,
                kv_from=None if src is None else int(src))
            a = lc.attn
            if a.heads % a.kv_heads:
                raise ValueError(f"layer {i}: heads % kv_heads != 0")
            if a.mask_size < 1:
                raise ValueError(f"layer {i}: mask.size must be >= 1")
            if a.kv_from is not None:
                s = layers[a.kv_from].attn if 0 <= a.kv_from < i else None
                if (s is None or s.kv_from is not None
                        or (s.kv_heads, s.dim, s.vdim)
                        != (a.kv_heads, a.dim, a.vdim)):
                    raise ValueError(f"layer {i}: cannot take keys and "
                                     f"values from layer {a.kv_from}")
        elif kind == "latent_attention":
            rot = mx.get("rot") or {}
            lc.latent = RotaryLatentConfig(
                heads=int(mx["heads"]), dim=int(mx["dim"]),
                rot_dim=int(mx["rot_dim"]), vdim=int(mx["vdim"]),
                kv_rank=int(mx["kv_rank"]), scale=float(mx["scale"]),
                rot_dims=int(rot.get("dims", mx["rot_dim"])),
                rot_base=float(rot.get("base", 10000.0)),
                rot_scaling=(dict(rot["scaling"]) if rot.get("scaling")
                             else None))
            m = lc.latent
            if m.rot_dims % 2 or m.rot_dims > m.rot_dim:
                raise ValueError(f"layer {i}: bad rot.dims {m.rot_dims}")
        else:
            raise ValueError(f"layer {i}: unsupported mixer {kind!r}")
        ml = ld.get("mlp")
        if ml is not None:
            if ml["kind"] == "dense":
                lc.mlp = SipelornFeedForwardConfig("dense", int(ml["ff"]))
            elif ml["kind"] == "moe":
                r = ml["router"]
                g = r.get("groups") or {}
                fc = SipelornFeedForwardConfig(
                    "moe", int(ml["expert"]["ff"]), experts=int(r["experts"]),
                    top=int(r["top"]), groups=int(g.get("count", 1)),
                    keep_groups=int(g.get("keep", 1)),
                    shared_ff=int((ml.get("shared") or {}).get("ff", 0)))
                if (fc.experts % fc.groups
                        or not 1 <= fc.keep_groups <= fc.groups):
                    raise ValueError(f"layer {i}: bad expert groups")
                if not 1 <= fc.top <= fc.keep_groups * (fc.experts
                                                        // fc.groups):
                    raise ValueError(f"layer {i}: top out of range")
                lc.mlp = fc
            else:
                raise ValueError(f"layer {i}: unsupported mlp {ml['kind']!r}")
        layers.append(lc)
    em = d.get("embedding") or {}
    bg = em.get("bigram") or {}
    return SipelornConfig(
        name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        layers=layers, norm_eps=float(d["norm"]["eps"]),
        embed_scale=float(em.get("scale", 1.0)),
        bigram_buckets=int(bg.get("buckets", 0)),
        bigram_mul_prev=int(bg.get("mul_prev", 0)),
        bigram_mul_cur=int(bg.get("mul_cur", 0)),
        side_dim=int((d.get("token_side") or {}).get("dim", 0)))


def config_from_checkpoint(path: str) -> SipelornConfig:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=path)


def _step_shape(md: AttnMetadata):
    if md.is_prefill:
        return md.query_starts, md.query_lens
    return None, None


class RotaryLatentAttention(torch.nn.Module):
    """Causal latent attention with a shared rotated key part. forward
    returns (output, the extra rows' columns of the input GEMM)."""

    def __init__(self, width: int, mc: RotaryLatentConfig, eps: float, dtype,
                 extra_rows: int = 0):
        super().__init__()
        self.mc, self.eps = mc, eps
        H, Rp = mc.heads, mc.padded_rank
        self.q_head = mc.dim + mc.rot_dim
        self.kv_off = _align(H * self.q_head)
        self.extra_rows = extra_rows
        self.extra_off = _align(self.kv_off + mc.kv_rank + mc.rot_dim)
        self.n_in = _align(self.extra_off + extra_rows)
        # one GEMM from the mixer input: [q | latent | rotated key | extra]
        self.w_in = _param(self.n_in, width, dtype=dtype)
        self.kv_norm = _param(mc.kv_rank, dtype=torch.float32)
        # q_full[h] = [q_plain[h] W_uk[h] | rotated q part | 0]: the pool
        # row's basis
        self.w_ukx = _param(H, self.q_head, Rp, dtype=dtype)
        self.w_uv = _param(H, Rp, mc.vdim, dtype=dtype)
        self.w_o = _param(width, H * mc.vdim, dtype=dtype)
        freqs, self.rot_amp = ops.rotary_frequencies(
            mc.rot_dims, mc.rot_base, mc.rot_scaling)
        self.register_buffer("rot_freqs", freqs, persistent=False)

    def _pair_order(self) -> torch.Tensor:
        """Checkpoint order (2i, 2i+1 rotate together) -> serving order
        (i, i + half rotate together) of the rotated part's rows."""
        mc = self.mc
        idx = list(range(0, mc.rot_dims, 2)) + list(range(1, mc.rot_dims, 2))
        return torch.tensor(idx + list(range(mc.rot_dims, mc.rot_dim)),
                            dtype=torch.long)

    def fix_padding(self):
        """Constant parts of the latent maps (also after a random init)."""
        mc = self.mc
        R, D, Dr = mc.kv_rank, mc.dim, mc.rot_dim
        self.w_ukx[:, :D, R:] = 0
        self.w_ukx[:, D:, :] = 0
        self.w_ukx[:, D:, R:R + Dr] = torch.eye(
            Dr, dtype=self.w_ukx.dtype, device=self.w_ukx.device)
        self.w_uv[:, R:, :] = 0

    @torch.no_grad()
    def load(self, get, extra=None):
        mc = self.mc
        H, R, D, Dr = mc.heads, mc.kv_rank, mc.dim, mc.rot_dim
        order = self._pair_order().to(self.w_in.device)
        wq = get("q").view(H, self.q_head, -1).clone()
        wq[:, D:] = wq[:, D:][:, order]
        dkv = get("dkv")
        self.w_in.zero_()
        self.w_in[:H * self.q_head].copy_(wq.view(H * self.q_head, -1))
        self.w_in[self.kv_off:self.kv_off + R].copy_(dkv[:R])
        self.w_in[self.kv_off + R:self.kv_off + R + Dr].copy_(dkv[R:][order])
        if extra is not None:
            self.w_in[self.extra_off:self.extra_off + self.extra_rows].copy_(
                extra)
        self.kv_norm.copy_(get("dkv.norm").float())
        self.w_ukx.zero_()
        self.w_ukx[:, :D, :R].copy_(get("uk").view(H, D, R))
        self.w_uv.zero_()
        self.w_uv[:, :R, :].copy_(get("uv").view(H, mc.vdim, R
                                                 ).transpose(1, 2))
        self.fix_padding()
        self.w_o.copy_(get("o"))

    def rotary_key(self):
        mc = self.mc
        sc = mc.rot_scaling
        return (mc.rot_dims, mc.rot_base,
                tuple(sorted(sc.items())) if sc else None)

    def forward(self, h: torch.Tensor, cache: torch.Tensor, md: AttnMetadata,
                tables: Optional[dict] = None):
        mc = self.mc
        T, H = h.size(0), mc.heads
        key = self.rotary_key()
        cos_sin = tables.get(key) if tables is not None else None
        if cos_sin is None:
            cos_sin = ops.rotary_table(md.positions, self.rot_freqs,
                                       self.rot_amp)
            if tables is not None:
                tables[key] = cos_sin
        proj = ops.linear(h, self.w_in)
        ops.latent_rotary_append(proj, H, self.q_head, mc.dim, self.kv_off,
                                 mc.kv_rank, mc.rot_dim, self.kv_norm,
                                 self.eps, cos_sin, cache, md.slot_mapping)
        q = proj[:, :H * self.q_head].view(T, H, self.q_head)
        q_lat = torch.bmm(q.transpose(0, 1), self.w_ukx)       # [H, T, Rp]
        o_lat = torch.empty_like(q_lat)
        ops.latent_window_attention(
            o_lat, q_lat, cache, md.page_table, md.seq_lens,
            md.query_starts if md.is_prefill else None,
            md.query_lens if md.is_prefill else None,
            mc.scale, CAUSAL_WINDOW,
            max_qlen=md.max_qlen if md.is_prefill else 1)
        a = torch.bmm(o_lat, self.w_uv)                        # [H, T, vdim]
        y = ops.linear(a.transpose(0, 1).reshape(T, H * mc.vdim), self.w_o)
        return y, proj[:, self.extra_off:self.extra_off + self.extra_rows]


class XieluFeedForward(torch.nn.Module):
    """down( xIELU(up h) ); forward returns (output, extra columns)."""

    def __init__(self, width: int, ff: int, dtype, extra_rows: int = 0):
        super().__init__()
        self.ff, self.extra_rows = ff, extra_rows
        self.extra_off = _align(ff)
        self.up = _param(_align(self.extra_off + extra_rows), width,
                         dtype=dtype)
        self.down = _param(width, ff, dtype=dtype)
        # (softplus(p), 1/2 + softplus(q)): the two curvatures
        self.coef = _param(2, dtype=torch.float32)

    @torch.no_grad()
    def load(self, get, extra=None):
        self.up.zero_()
        self.up[:self.ff].copy_(get("up"))
        if extra is not None:
            self.up[self.extra_off:self.extra_off + self.extra_rows].copy_(
                extra)
        self.down.copy_(get("down"))
        pq = get("act").float()
        self.coef.copy_(F.softplus(pq) + torch.tensor(
            [0.0, 0.5], device=pq.device))

    def forward(self, h, allow_gather: bool = True):
        z = ops.linear(h, self.up)
        act = torch.empty(h.size(0), self.ff, dtype=h.dtype, device=h.device)
        ops.xielu(act, z[:, :self.ff], self.coef)
        return (ops.linear(act, self.down),
                z[:, self.extra_off:self.extra_off + self.extra_rows])


class GroupedSigmoidExperts(torch.nn.Module):
    """Sigmoid-scored experts, group-limited top-k choice with a
    choice-only correction, un-renormalized weights on the expert output,
    and a shared expert behind a per-token sigmoid gate (it rides as an
    always-chosen tail expert whose weight is that gate). forward returns
    (output, extra columns)."""

    SPARSE_MIN_TOKENS = 256   # from here on rows are gathered per expert

    def __init__(self, width: int, fc: SipelornFeedForwardConfig, dtype,
                 extra_rows: int = 0):
        super().__init__()
        self.fc, self.extra_rows = fc, extra_rows
        E, Fh, Fs = fc.experts, fc.ff, fc.shared_ff
        f32 = torch.float32
        self.n_gates = 1 if Fs > 0 else 0
        # fp32 router; the shared expert's gate is its last row
        self.router = _param(E + self.n_gates, width, dtype=f32)
        self.correction = _param(E, dtype=f32)
        # expert e owns rows [e*2F, e*2F+F) = gate, [e*2F+F, (e+1)*2F) = up;
        # then the shared expert's gate | up, then the caller's rows
        self.gu_rows = E * 2 * Fh + 2 * Fs
        self.extra_off = _align(self.gu_rows)
        self.gate_up = _param(_align(self.extra_off + extra_rows), width,
                              dtype=dtype)
        # expert e owns columns [e*F, (e+1)*F); the shared expert the rest
        self.down = _param(width, E * Fh + Fs, dtype=dtype)

    @torch.no_grad()
    def load(self, get, extra=None):
        fc = self.fc
        E = fc.experts
        rows = [get("router").float()]
        if fc.shared_ff > 0:
            rows.append(get("shared.sg").float().view(1, -1))
        self.router.copy_(torch.cat(rows, dim=0))
        self.correction.copy_(get("correction").float())
        names = [f"e{e}." for e in range(E)]
        if fc.shared_ff > 0:
            names.append("shared.")
        self.gate_up.zero_()
        self.gate_up[:self.gu_rows].copy_(torch.cat(
            [torch.cat([get(n + "gate"), get(n + "up")], dim=0)
             for n in names], dim=0))
        if extra is not None:
            self.gate_up[self.extra_off:self.extra_off + self.extra_rows
                         ].copy_(extra)
        self.down.copy_(torch.cat([get(n + "down") for n in names], dim=1))

    def forward(self, h, allow_gather: bool = True):
        """allow_gather=False keeps the step free of host syncs (decode
        steps are captured into a hipGraph)."""
        fc = self.fc
        T, E, Fh, Fs = h.size(0), fc.experts, fc.ff, fc.shared_ff
        logits = F.linear(h.float(), self.router)              # fp32 router
        weight = torch.empty(T, E + self.n_gates, dtype=torch.float32,
                             device=h.device)
        ops.grouped_sigmoid_route(weight, logits, self.correction, E, fc.top,
                                  fc.groups, fc.keep_groups, GROUP_TOP)
        if allow_gather and T >= self.SPARSE_MIN_TOKENS and E > fc.top:
            return self._gathered(h, weight)
        gu = ops.linear(h, self.gate_up)
        act = torch.empty(T, E * Fh + Fs, dtype=h.dtype, device=h.device)
        ops.routed_silu_glu(act, gu[:, :self.gu_rows], weight, E, Fh, Fs)
        return (ops.linear(act, self.down),
                gu[:, self.extra_off:self.extra_off + self.extra_rows])

    def _gathered(self, h, weight):
        """Per-expert execution for prompt-sized batches: the rows routed
        to an expert are gathered, run through that expert only, and added
        back in fp32 in a fixed expert order; the shared expert and the
        caller's rows stay one dense GEMM."""
        fc = self.fc
        T, W = h.shape
        E, Fh, Fs = fc.experts, fc.ff, fc.shared_ff
        dense = ops.linear(h, self.gate_up[E * 2 * Fh:])
        extra0 = self.extra_off - E * 2 * Fh
        out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
        if Fs > 0:
            act = torch.empty(T, Fs, dtype=h.dtype, device=h.device)
            ops.routed_silu_glu(act, dense[:, :2 * Fs], weight[:, E:], 0, Fh,
                                Fs)
            out += ops.linear(act, self.down[:, E * Fh:]).float()
        hit = weight[:, :E] > 0
        counts = hit.sum(dim=0).tolist()                       # host sync
        for e in range(E):
            if counts[e] == 0:
                continue
            rows = hit[:, e].nonzero(as_tuple=True)[0]
            w = weight[rows, e].unsqueeze(1).contiguous()      # [n, 1] fp32
            gu = ops.linear(h.index_select(0, rows),
                            self.gate_up[e * 2 * Fh:(e + 1) * 2 * Fh])
            act = torch.empty(rows.numel(), Fh, dtype=h.dtype, device=h.device)
            ops.routed_silu_glu(act, gu, w, 1, Fh, 0)
            out.index_add_(0, rows, ops.linear(
                act, self.down[:, e * Fh:(e + 1) * Fh]).float())
        return out.to(h.dtype), dense[:, extra0:extra0 + self.extra_rows]


class SipelornLayer(torch.nn.Module):
    def __init__(self, cfg: SipelornConfig, lc: SipelornLayerConfig, dtype):
        super().__init__()
        W = cfg.hidden_size
        f32 = torch.float32
        self.lc = lc
        self.norm1_w, self.norm1_b = _param(W, dtype=f32), _param(W, dtype=f32)
        self.rg1_b = _param(W, dtype=f32)
        # the residual gate's projection rides in the sublayer's input GEMM
        if lc.attn is not None:
            self.mix = MaskedAttention(W, lc.attn, cfg.norm_eps, dtype,
                                       extra_rows=W)
        else:
            self.mix = RotaryLatentAttention(W, lc.latent, cfg.norm_eps,
                                             dtype, extra_rows=W)
        if lc.mlp is None:
            self.mlp = None
        else:
            self.norm2_w = _param(W, dtype=f32)
            self.norm2_b = _param(W, dtype=f32)
            self.rg2_b = _param(W, dtype=f32)
            self.mlp = (XieluFeedForward(W, lc.mlp.ff, dtype, extra_rows=W)
                        if lc.mlp.kind == "dense" else
                        GroupedSigmoidExperts(W, lc.mlp, dtype, extra_rows=W))
        if cfg.side_dim > 0:
            d = cfg.side_dim
            self.side_gate = _param(d, W, dtype=dtype)
            self.side_proj = _param(W, d, dtype=dtype)
            self.side_norm = _param(W, dtype=f32)


class SipelornForCausalLM(torch.nn.Module):
    def __init__(self, cfg: SipelornConfig, device="cpu", tp_rank: int = 0,
                 tp_size: int = 1, seed: int = 0, dtype=torch.bfloat16):
        super().__init__()
        if tp_size != 1:
            raise ValueError("Sipelorn: tensor parallelism is not implemented")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Sipelorn: unsupported compute dtype {dtype}")
        self.cfg = cfg
        self.dtype = dtype
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        W = cfg.hidden_size
        f32 = torch.float32
        with torch.device(device):
            self.embed = _param(cfg.vocab_size, W, dtype=dtype)
            self.bigram = (_param(cfg.bigram_buckets + 1, W, dtype=dtype)
                           if cfg.bigram_buckets > 0 else None)
            self.side_embed = (_param(cfg.vocab_size,
                                      cfg.side_dim * cfg.n_layers, dtype=dtype)
                               if cfg.side_dim > 0 else None)
            self.layers = torch.nn.ModuleList(
                [SipelornLayer(cfg, lc, dtype) for lc in cfg.layers])
            self.final_norm_w = _param(W, dtype=f32)
            self.final_norm_b = _param(W, dtype=f32)
            self.lm_head = _param(cfg.vocab_size, W, dtype=dtype)
        self.random_init(seed)
        # test hook: when a list, receives the residual after every layer
        self.residual_trace: Optional[list] = None

    @torch.no_grad()
    def random_init(self, seed: int = 0):
        gen = torch.Generator(device=self.embed.device).manual_seed(seed)

        def normal(p, std, mean=0.0):
            p.copy_((mean + torch.randn(p.shape, generator=gen,
                                        device=p.device, dtype=torch.float32)
                     * std).to(p.dtype))

        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1_w", "norm2_w", "final_norm_w", "kv_norm"):
                p.fill_(1.0)
            elif leaf == "side_norm":
                p.fill_(0.5)
            elif leaf == "coef":
                p.copy_(torch.tensor([0.8, 1.2], device=p.device))
            elif leaf == "dist_bias":
                p.copy_(torch.tensor([0.5, 0.4], device=p.device
                                     ).expand_as(p))
            elif leaf == "correction":
                normal(p, 0.05)
            elif leaf == "w_conv":
                normal(p, 0.5)
            elif leaf == "b_in":
                normal(p, 0.1)
            elif leaf == "w_ukx":
                normal(p, 1.0 / p.size(1) ** 0.5)
            elif p.dim() >= 2:
                normal(p, 1.0 / p.size(-1) ** 0.5)
            else:
                p.fill_(0.0)
        normal(self.embed, 1.0)
        for layer in self.layers:
            if isinstance(layer.mix, RotaryLatentAttention):
                layer.mix.fix_padding()

    def pack_decode_weights(self):
        """Projections run on hipBLASLt in both phases; nothing to repack."""

    @torch.no_grad()
    def load_safetensors(self, path: str):
        from safetensors.torch import load_file
        import glob

        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no safetensors under {path}")
        sd: Dict[str, torch.Tensor] = {}
        for f in files:
            sd.update(load_file(f))
        self.load_state(sd)

    @torch.no_grad()
    def load_state(self, sd: Dict[str, torch.Tensor]):
        """Copy checkpoint tensors (embed, bigram, side.embed, l<i>.norm1/2
        (+ .b), l<i>.rg1/2 (+ .b), l<i>.mix.*, l<i>.mlp.*, l<i>.side.*,
        final.norm (+ .b), head) into the fused serving layout."""
        dev, dt = self.embed.device, self.dtype

        def getter(prefix):
            def get(name):
                return sd[prefix + name].to(device=dev, dtype=dt)
            return get

        top = getter("")
        self.embed.copy_(top("embed"))
        if self.bigram is not None:
            self.bigram.copy_(top("bigram"))
        if self.side_embed is not None:
            self.side_embed.copy_(top("side.embed"))
        self.lm_head.copy_(top("head"))
        self.final_norm_w.copy_(top("final.norm").float())
        self.final_norm_b.copy_(top("final.norm.b").float())
        for i, layer in enumerate(self.layers):
            g = getter(f"l{i}.")
            layer.norm1_w.copy_(g("norm1").float())
            layer.norm1_b.copy_(g("norm1.b").float())
            layer.rg1_b.copy_(g("rg1.b").float())
            layer.mix.load(getter(f"l{i}.mix."), extra=g("rg1"))
            if layer.mlp is not None:
                layer.norm2_w.copy_(g("norm2").float())
                layer.norm2_b.copy_(g("norm2.b").float())
                layer.rg2_b.copy_(g("rg2.b").float())
                layer.mlp.load(getter(f"l{i}.mlp."), extra=g("rg2"))
            if self.cfg.side_dim > 0:
                layer.side_gate.copy_(g("side.gate"))
                layer.side_proj.copy_(g("side.proj"))
                layer.side_norm.copy_(g("side.norm").float())

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, md: AttnMetadata,
                kv_caches: List, last_rows: Optional[torch.Tensor] = None
                ) -> torch.Tensor:
        cfg = self.cfg
        eps, W, d = cfg.norm_eps, cfg.hidden_size, cfg.side_dim
        if md.state_slots is None:
            raise ValueError("Sipelorn needs per-sequence state slots")
        T, dev = input_ids.size(0), input_ids.device
        q_starts, q_lens = _step_shape(md)
        x = torch.empty(T, W, dtype=torch.float32, device=dev)
        ops.bigram_embed(
            x, input_ids, self.embed, self.bigram, cfg.embed_scale,
            cfg.bigram_mul_prev, cfg.bigram_mul_cur, cfg.bigram_buckets,
            kv_caches[0][2].get("prev_token"), md.state_slots, md.seq_lens,
            q_starts, q_lens)

        def step(y, update, gate, gate_bias, rms_w, norm):
            """One residual update; `norm` = (w, b) of the layer norm that
            feeds the next GEMM, "cast" for the plain stream, None for
            nothing."""
            if norm is None:
                out, nw, nb = None, None, None
            else:
                out = torch.empty(T, W, dtype=self.dtype, device=dev)
                nw, nb = (None, None) if norm == "cast" else norm
            ops.residual_update_norm(x, y, update, gate, gate_bias, rms_w,
                                     eps, nw, nb, out)
            return out

        n = len(self.layers)
        l0 = self.layers[0]
        h = step(None, ops.UPDATE_NONE, None, None, None,
                 (l0.norm1_w, l0.norm1_b))
        tables: dict = {}      # rotary setting -> this step's cos/sin rows
        for i, layer in enumerate(self.layers):
            lc = layer.lc
            state = kv_caches[i][2]
            if lc.attn is not None:
                src = i if lc.attn.kv_from is None else lc.attn.kv_from
                y, gate = layer.mix(h, kv_caches[src][0], kv_caches[src][1],
                                    md, tables, conv_tail=state.get("conv"))
            else:
                y, gate = layer.mix(h, kv_caches[i][0], md, tables)
            nxt = (None if i + 1 == n else
                   (self.layers[i + 1].norm1_w, self.layers[i + 1].norm1_b))
            after_ff = "cast" if d > 0 else nxt
            if layer.mlp is not None:
                h = step(y, ops.UPDATE_SIGMOID_GATE, gate, layer.rg1_b, None,
                         (layer.norm2_w, layer.norm2_b))
                f, gate = layer.mlp(h, allow_gather=md.is_prefill)
                h = step(f, ops.UPDATE_SIGMOID_GATE, gate, layer.rg2_b, None,
                         after_ff)
            else:
                h = step(y, ops.UPDATE_SIGMOID_GATE, gate, layer.rg1_b, None,
                         after_ff)
            if d > 0:
                t = ops.linear(h, layer.side_gate)             # [T, d]
                g = torch.empty_like(t)
                ops.gelu_gate_rows(g, t, self.side_embed, input_ids, i * d)
                h = step(ops.linear(g, layer.side_proj), ops.UPDATE_UNIT_RMS,
                         None, None, layer.side_norm, nxt)
            if self.residual_trace is not None:
                self.residual_trace.append(x.clone())
        if last_rows is not None:
            x = x[last_rows]
        final = torch.empty(x.size(0), W, dtype=self.dtype, device=dev)
        ops.residual_update_norm(x, None, ops.UPDATE_NONE, None, None, None,
                                 eps, self.final_norm_w, self.final_norm_b,
                                 final)
        return ops.linear(final, self.lm_head).float()


def _tiny(name: str) -> SipelornConfig:
    latent = RotaryLatentConfig(
        heads=4, dim=32, rot_dim=16, vdim=32, kv_rank=48, scale=48 ** -0.5,
        rot_dims=16, rot_base=10000.0,
        rot_scaling={"factor": 4.0, "original": 256, "fast": 16.0,
                     "slow": 2.0})

    def attn(kv_from=None):
        return MaskedAttentionConfig(
            heads=4, kv_heads=2, dim=32, vdim=32, scale=32 ** -0.5,
            mask_kind=ops.MASK_WINDOW, mask_size=48, qkv_bias=True,
            conv_taps=4, plain_qk=True, dist_bias=True, elem_gate=True,
            kv_from=kv_from)

    moe = SipelornFeedForwardConfig("moe", 64, experts=8, top=2, groups=4,
                                    keep_groups=2, shared_ff=96)
    layers = [
        SipelornLayerConfig("latent_attention", latent=latent,
                            mlp=SipelornFeedForwardConfig("dense", 256)),
        SipelornLayerConfig("attention", attn=attn(), mlp=moe),
        SipelornLayerConfig("attention", attn=attn(kv_from=1), mlp=moe),
    ]
    return SipelornConfig(name=name, vocab_size=512, hidden_size=128,
                          layers=layers, norm_eps=1e-5, embed_scale=8.0,
                          bigram_buckets=251, bigram_mul_prev=13,
                          bigram_mul_cur=29, side_dim=8)


SIPELORN_CONFIGS: Dict[str, SipelornConfig] = {
    "tiny-sipelorn": _tiny("tiny-sipelorn"),
}


def make_sipelorn_instance(name: str, device: str, engine_cfg,
                           weights_path: Optional[str] = None):
    """ModelInstance over a Sipelorn model (engine factory hook): a named
    random-init config, or a checkpoint directory."""
    from ..engine.llm import ModelInstance

    cfg = (config_from_checkpoint(weights_path) if weights_path
           else SIPELORN_CONFIGS[name])
    if device.startswith("cuda") and not (
            ops.gated_available() and ops.masked_available()
            and ops.latent_available() and ops.recurrent_available()):
        raise RuntimeError(
            "GPU engine requires the gfx950 gated, masked-attention, latent "
            "and recurrent extensions (python -m agentainer_amd.ops.build "
            "gated masked latent recurrent)")
    return ModelInstance(name, cfg, device, engine_cfg,
                         weights_path=weights_path,
                         model_cls=SipelornForCausalLM)
