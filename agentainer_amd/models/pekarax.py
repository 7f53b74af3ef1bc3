"""Pekarax family — post-normed hybrid decoder: matrix-memory recurrences,
convolved softmax attention, group-routed experts.

Every layer rewrites an fp32 residual stream x with a norm AFTER the sum;
the sublayers read x itself:

    x <- N1(alpha x + mixer(x));   x <- N2(alpha x + ff(x))
    N(s) = s / sqrt(mean(s^2) + eps) * (1 + w)

The layer list of config.json picks one mixer per layer:

  * "gla"           gated linear attention: S <- diag(a) S + k v^T,
                    o = S^T q, one decay a = sigmoid(z)^(1/tau) per key
                    channel from a low-rank projection; per-head RMS norm,
                    SiLU output gate.
  * "channel_delta" gated delta rule with per-key-channel decay: q, k, v
                    pass a short causal convolution + SiLU, q and k become
                    unit vectors; S <- g S; u = beta (v - S^T k);
                    S <- S + k u^T; o = S^T q; per-head RMS norm, low-rank
                    sigmoid output gate.
  * "parallel"      two mixers side by side on the same input, summed with
                    config weights: LEFT causal softmax attention whose
                    q, k, v pass a short causal convolution, then rotary
                    on the leading coordinates, then weightless unit-rms
                    of q and k; RIGHT an mLSTM matrix memory with capped
                    log gates and a running-maximum stabilizer.

The feed-forward is a mixture of clamped gated experts with softmax
scores, a per-expert correction that only influences the CHOICE,
group-limited selection, and weightless identity experts whose output is
the input itself.

Serving design (what runs on the MI355X):

  * Recurrent memories, the mLSTM normalizer / maximum and the convolution
    tails are per-SEQUENCE state: the engine's KVCacheManager owns them
    through HybridStateLayout, one fp32 tensor [slots, ...] per layer and
    name, addressed by the sequence slot; the left attention's K/V live in
    the same manager's page pools. One kernel family
    (ops.matrix_memory_scan) steps the recurrences token by token with the
    state in registers — prompt portions and single decoded tokens take the
    same code, so a position's result does not depend on how the prompt was
    cut. Decays, gates, softplus / exponentials are evaluated in fp32 inside
    that kernel from fp32 pre-activations.
  * The wide projections of a mixer are ONE GEMM in the compute dtype; the
    narrow ones that feed decays and gates (low-rank stages, per-head
    gates, the router) are ONE fp32 GEMM read straight from the fp32
    residual.
  * ops.short_conv_state convolves q|k|v in one launch (+ SiLU, unit
    vectors, query scale where the mixer has them); the attention then
    reuses ops.rotary_norm_append / ops.masked_attention.
  * ops.postln_rmsnorm_residual fuses the weighted sum of up to two mixer
    outputs, the identity experts' share (a per-row addition to alpha), the
    norm and the cast that feeds the next GEMM.
  * Experts run stacked (one gate|up GEMM, ops.routed_clamped_glu, one
    down GEMM) in decode steps and gathered per expert for prompt-sized
    batches.

compute dtype: bf16 (serving default) or float32 (everything fp32).
"""

from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from .llama import AttnMetadata
from .volalorn import MaskedAttention, MaskedAttentionConfig

PROJ_ALIGN = 8          # rows of a stacked projection: 16-byte aligned bf16
EXPERT_SLOPE = 1.702    # sigmoid slope of the expert activation
DEFAULT_RANK = 16       # low-rank stages of named random-init configs


@dataclass
class MatrixMemoryConfig:
    kind: int                 # ops.SCAN_GLA / SCAN_DELTA / SCAN_MLSTM
    heads: int                # value heads (= memories per layer)
    qk_heads: int             # query/key heads; heads % qk_heads == 0
    dim: int                  # key channels per head
    vdim: int                 # value channels per head
    conv_taps: int = 0        # short convolution on q, k, v (delta rule)
    decay_rank: int = 0       # low-rank stage of the per-channel decay
    gate_rank: int = 0        # low-rank stage of the output gate (0: full)
    tau: float = 1.0          # gla: decay = sigmoid(z)^(1/tau)
    gate_cap: float = 0.0     # mLSTM: gates are cap * tanh(z / cap)


@dataclass
class GroupedExpertsConfig:
    experts: int              # experts with weights
    identity: int             # weightless experts appended to the router
    top: int
    ff: int
    limit: float              # gate <= limit, |up| <= limit
    groups: int = 1
    keep_groups: int = 1
    scale: float = 1.0


@dataclass
class PekaraxLayerConfig:
    kind: str
    attn: Optional[MaskedAttentionConfig] = None
    memory: Optional[MatrixMemoryConfig] = None
    attn_scale: float = 1.0
    memory_scale: float = 1.0
    mlp: Optional[GroupedExpertsConfig] = None


@dataclass
class PekaraxConfig:
    name: str = "tiny-pekarax"
    vocab_size: int = 512
    hidden_size: int = 128
    layers: List[PekaraxLayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-5
    postln_alpha: float = 1.0
    family: str = "pekarax"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def max_position(self) -> int:
        return 1 << 30

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l.attn.kv_heads * (l.attn.dim + l.attn.vdim)
                   for l in self.layers if l.attn is not None) * dtype_bytes

    def state_shapes(self) -> List[Dict[str, tuple]]:
        out = []
        for l in self.layers:
            d: Dict[str, tuple] = {}
            a, m = l.attn, l.memory
            if a is not None and a.conv_taps > 0:
                ch = a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)
                d["attn_conv"] = (a.conv_taps - 1, ch)
            if m is not None:
                d["S"] = (m.heads, m.vdim, m.dim)
                if m.kind == ops.SCAN_MLSTM:
                    d["n"] = (m.heads, m.dim)
                    d["m"] = (m.heads,)
                if m.conv_taps > 0:
                    d["conv"] = (m.conv_taps - 1,
                                 2 * m.qk_heads * m.dim + m.heads * m.vdim)
            out.append(d)
        return out

    def cache_layout(self):
        from ..engine.kvcache import HybridStateLayout
        return HybridStateLayout(
            [None if l.attn is None else
             (l.attn.kv_heads, l.attn.dim, l.attn.vdim) for l in self.layers],
            self.state_shapes())

    def state_bytes_per_seq(self) -> int:
        return self.cache_layout().state_bytes_per_seq()


def _attention_from_dict(mx: dict) -> MaskedAttentionConfig:
    rot = mx.get("rot") or {}
    return MaskedAttentionConfig(
        heads=int(mx["heads"]), kv_heads=int(mx["kv_heads"]),
        dim=int(mx["dim"]), vdim=int(mx["vdim"]), scale=float(mx["scale"]),
        mask_kind=ops.MASK_CAUSAL, mask_size=0,
        rot_dims=int(rot.get("dims", 0)),
        rot_base=float(rot.get("base", 10000.0)), norm_first=False,
        conv_taps=int(mx.get("conv", 0)))


def _rank(shapes: Optional[dict], name: str, mx: dict, key: str) -> int:
    """Row count of a low-rank stage: from the checkpoint's tensor shape,
    else an optional config key, else the default."""
    if shapes is not None and name in shapes:
        return int(shapes[name][0])
    return int(mx.get(key, DEFAULT_RANK))


def _memory_from_dict(kind: str, mx: dict, shapes: Optional[dict],
                      prefix: str) -> MatrixMemoryConfig:
    heads, dim, vdim = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
    if kind == "gla":
        return MatrixMemoryConfig(
            ops.SCAN_GLA, heads, heads, dim, vdim,
            decay_rank=_rank(shapes, prefix + "a1", mx, "decay_rank"),
            tau=float(mx["tau"]))
    if kind == "channel_delta":
        return MatrixMemoryConfig(
            ops.SCAN_DELTA, heads, int(mx.get("kv_heads", heads)), dim, vdim,
            conv_taps=int(mx.get("conv", 0)),
            decay_rank=_rank(shapes, prefix + "a1", mx, "decay_rank"),
            gate_rank=_rank(shapes, prefix + "g1", mx, "gate_rank"))
    if kind == "mlstm":
        return MatrixMemoryConfig(ops.SCAN_MLSTM, heads, heads, dim, vdim,
                                  gate_cap=float(mx["gate_cap"]))
    raise ValueError(f"unsupported matrix memory {kind!r}")


def config_from_dict(d: dict, name: str = "pekarax",
                     shapes: Optional[dict] = None) -> PekaraxConfig:
    """PekaraxConfig from a parsed config.json; `shapes` (tensor name ->
    shape, from the checkpoint header) supplies the sizes that only the
    tensors carry."""
    layers = []
    for i, ld in enumerate(d["layers"]):
        kind, mx = ld["type"], ld["mixer"]
        lc = PekaraxLayerConfig(kind)
        if kind == "parallel":
            lc.attn = _attention_from_dict(mx["left"])
            lc.memory = _memory_from_dict("mlstm", mx["right"], shapes,
                                          f"l{i}.mix.right.")
            lc.attn_scale = float(mx.get("left_scale", 1.0))
            lc.memory_scale = float(mx.get("right_scale", 1.0))
        elif kind in ("gla", "channel_delta"):
            lc.memory = _memory_from_dict(kind, mx, shapes, f"l{i}.mix.")
        else:
            raise ValueError(f"layer {i}: unsupported mixer {kind!r}")
        a, m = lc.attn, lc.memory
        if a is not None:
            if a.heads % a.kv_heads:
                raise ValueError(f"layer {i}: heads % kv_heads != 0")
            if a.rot_dims % 2 or a.rot_dims > a.dim:
                raise ValueError(f"layer {i}: bad rot.dims {a.rot_dims}")
        if m.heads % m.qk_heads:
            raise ValueError(f"layer {i}: heads % kv_heads != 0")
        ml = ld.get("mlp")
        if ml is not None:
            if ml.get("kind") != "moe":
                raise ValueError(f"layer {i}: unsupported mlp {ml.get('kind')!r}")
            r, ex = ml["router"], ml["expert"]
            g = r.get("groups") or {}
            fc = GroupedExpertsConfig(
                experts=int(r["experts"]), identity=int(r.get("identity", 0)),
                top=int(r["top"]), ff=int(ex["ff"]), limit=float(ex["limit"]),
                groups=int(g.get("count", 1)), keep_groups=int(g.get("keep", 1)),
                scale=float(r.get("scale", 1.0)))
            tot = fc.experts + fc.identity
            if tot % fc.groups or not 1 <= fc.keep_groups <= fc.groups:
                raise ValueError(f"layer {i}: bad expert groups")
            if not 1 <= fc.top <= fc.keep_groups * (tot // fc.groups):
                raise ValueError(f"layer {i}: top out of range")
            lc.mlp = fc
        layers.append(lc)
    return PekaraxConfig(
        name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        layers=layers, norm_eps=float(d["norm"]["eps"]),
        postln_alpha=float(d.get("postln_alpha", 1.0)))


def safetensors_shapes(path: str) -> Dict[str, List[int]]:
    """Tensor name -> shape from the headers of a directory's safetensors
    files (8-byte little-endian length, then that many bytes of JSON)."""
    import glob

    out: Dict[str, List[int]] = {}
    for f in sorted(glob.glob(os.path.join(path, "*.safetensors"))):
        with open(f, "rb") as fh:
            (n,) = struct.unpack("<Q", fh.read(8))
            head = json.loads(fh.read(n))
        for k, v in head.items():
            if k != "__metadata__":
                out[k] = list(v["shape"])
    return out


def config_from_checkpoint(path: str) -> PekaraxConfig:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=path,
                                shapes=safetensors_shapes(path))


def _param(*shape, dtype):
    return torch.nn.Parameter(torch.empty(*shape, dtype=dtype),
                              requires_grad=False)


def _pad(n: int) -> int:
    return -(-n // PROJ_ALIGN) * PROJ_ALIGN


def _step_shape(md: AttnMetadata):
    if md.is_prefill:
        return md.query_starts, md.query_lens
    return None, None


class MatrixMemoryMixer(torch.nn.Module):
    """Linear-recurrent mixer over a per-head matrix memory S [dim, vdim]
    (see MatrixMemoryConfig.kind); the memory is per-sequence state."""

    def __init__(self, width: int, mc: MatrixMemoryConfig, eps: float, dtype):
        super().__init__()
        self.mc, self.eps = mc, eps
        H, G, D, Dv = mc.heads, mc.qk_heads, mc.dim, mc.vdim
        f32 = torch.float32
        self.q_sz = self.k_sz = G * D
        self.v_sz = H * Dv
        kind = mc.kind
        # wide projections, one GEMM in the compute dtype: q | k | v
        # (| full-rank output gate)
        self.full_gate = kind in (ops.SCAN_GLA, ops.SCAN_MLSTM)
        n = self.q_sz + self.k_sz + self.v_sz + (self.v_sz if self.full_gate
                                                 else 0)
        self.w_in = _param(_pad(n), width, dtype=dtype)
        # narrow projections that feed decays and gates, one fp32 GEMM on
        # the fp32 residual
        if kind == ops.SCAN_GLA:
            n_small = mc.decay_rank
        elif kind == ops.SCAN_DELTA:
            n_small = mc.decay_rank + mc.gate_rank + H
        else:
            n_small = 2 * H
        self.w_small = _param(n_small, width, dtype=f32)
        if kind == ops.SCAN_MLSTM:
            self.gate_bias = _param(2 * H, dtype=f32)
            self.norm_w = _param(H * Dv, dtype=f32)
        else:
            self.a2 = _param(H * D, mc.decay_rank, dtype=f32)
            self.gate_bias = _param(H * D, dtype=f32)
            self.norm_w = _param(Dv, dtype=f32)
        if kind == ops.SCAN_DELTA:
            self.g2 = _param(H * Dv, mc.gate_rank, dtype=f32)
            self.head_rate = _param(H, dtype=f32)
        self.conv_channels = self.q_sz + self.k_sz + self.v_sz
        self.w_conv = (_param(mc.conv_taps, self.conv_channels, dtype=f32)
                       if mc.conv_taps > 0 else None)
        self.w_o = _param(width, H * Dv, dtype=dtype)

    @torch.no_grad()
    def load(self, get):
        mc = self.mc
        q0, k0, v0 = 0, self.q_sz, self.q_sz + self.k_sz
        g0 = v0 + self.v_sz
        self.w_in.zero_()
        self.w_in[q0:k0].copy_(get("q"))
        self.w_in[k0:v0].copy_(get("k"))
        self.w_in[v0:g0].copy_(get("v"))
        if self.full_gate:
            self.w_in[g0:g0 + self.v_sz].copy_(get("g"))
        f = lambda name: get(name).float()          # noqa: E731
        if mc.kind == ops.SCAN_GLA:
            self.w_small.copy_(f("a1"))
            self.a2.copy_(f("a2"))
            self.gate_bias.copy_(f("a2.b"))
        elif mc.kind == ops.SCAN_DELTA:
            self.w_small.copy_(torch.cat([f("a1"), f("g1"), f("b")], dim=0))
            self.a2.copy_(f("a2"))
            self.g2.copy_(f("g2"))
            self.gate_bias.copy_(f("dt_bias"))
            self.head_rate.copy_(f("A_log"))
        else:
            self.w_small.copy_(torch.cat([f("i"), f("f")], dim=0))
            self.gate_bias.copy_(torch.cat([f("i.b"), f("f.b")], dim=0))
        self.norm_w.copy_(f("norm"))
        if mc.conv_taps > 0:
            # checkpoint [channels, taps] -> tap-major [taps, channels]
            self.w_conv.copy_(torch.cat([f("q.conv"), f("k.conv"),
                                         f("v.conv")], dim=0).t())
        self.w_o.copy_(get("o"))

    def forward(self, h: torch.Tensor, x: torch.Tensor, state: dict,
                md: AttnMetadata) -> torch.Tensor:
        """h: the mixer input in the compute dtype; x: the same rows of the
        fp32 residual; state: this layer's per-sequence state tensors."""
        mc = self.mc
        T, H, G, D, Dv = h.size(0), mc.heads, mc.qk_heads, mc.dim, mc.vdim
        kind = mc.kind
        q_starts, q_lens = _step_shape(md)
        proj = ops.linear(h, self.w_in)
        small = F.linear(x, self.w_small)
        k0, v0 = self.q_sz, self.q_sz + self.k_sz
        g0 = v0 + self.v_sz
        qkv, q_scale = proj, D ** -0.5
        if mc.conv_taps > 0:
            # conv + SiLU, q and k to unit vectors, q scaled: fp32 out
            qkv = torch.empty(T, g0, dtype=torch.float32, device=h.device)
            ops.short_conv_state(
                qkv, proj[:, :g0], self.w_conv, state["conv"], md.state_slots,
                md.seq_lens, q_starts, q_lens, silu=True, norm_channels=v0,
                head_dim=D, lead_channels=k0, lead_scale=q_scale)
            q_scale = 1.0
        q = qkv[:, :k0].view(T, G, D)
        k = qkv[:, k0:v0].view(T, G, D)
        v = qkv[:, v0:g0].view(T, H, Dv)
        beta = head_rate = None
        n_state = m_state = None
        if kind == ops.SCAN_GLA:
            gate = F.linear(small, self.a2)
            param = 1.0 / mc.tau
            out_gate = proj[:, g0:g0 + self.v_sz]
        elif kind == ops.SCAN_DELTA:
            r, rg = mc.decay_rank, mc.gate_rank
            gate = F.linear(small[:, :r], self.a2)
            out_gate = F.linear(small[:, r:r + rg], self.g2)
            beta = small[:, r + rg:]
            head_rate, param = self.head_rate, 0.0
        else:
            gate, param = small, mc.gate_cap
            out_gate = proj[:, g0:g0 + self.v_sz]
            n_state, m_state = state["n"], state["m"]
        o = torch.empty(T, H, Dv, dtype=torch.float32, device=h.device)
        ops.matrix_memory_scan(kind, o, q, k, v, gate, self.gate_bias,
                               head_rate, beta, q_scale, param, state["S"],
                               n_state, m_state, md.state_slots, md.seq_lens,
                               q_starts, q_lens)
        y = torch.empty(T, H * Dv, dtype=h.dtype, device=h.device)
        ops.head_rmsnorm_gate(y, o, self.norm_w, out_gate, self.eps,
                              silu_gate=(kind == ops.SCAN_GLA))
        return ops.linear(y, self.w_o)


class GroupRoutedExperts(torch.nn.Module):
    """Softmax-scored experts with group-limited top-k choice, a choice-only
    correction, clamped gated activation and weightless identity experts.

    forward returns (y, identity_weight): y sums the chosen weighted
    experts; identity_weight [T] (or None) is the total weight of the
    chosen identity experts — their output is the layer input itself, so
    the caller adds it to the residual's coefficient."""

    SPARSE_MIN_TOKENS = 256   # from here on rows are gathered per expert

    def __init__(self, width: int, fc: GroupedExpertsConfig, dtype):
        super().__init__()
        self.fc = fc
        E, Fh = fc.experts, fc.ff
        f32 = torch.float32
        self.router = _param(E + fc.identity, width, dtype=f32)
        self.correction = _param(E + fc.identity, dtype=f32)
        # expert e owns rows [e*2F, e*2F+F) = gate, [e*2F+F, (e+1)*2F) = up
        self.gate_up = _param(E * 2 * Fh, width, dtype=dtype)
        # expert e owns columns [e*F, (e+1)*F)
        self.down = _param(width, E * Fh, dtype=dtype)

    @torch.no_grad()
    def load(self, get):
        E = self.fc.experts
        self.router.copy_(get("router").float())
        self.correction.copy_(get("correction").float())
        self.gate_up.copy_(torch.cat(
            [torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")], dim=0)
             for e in range(E)], dim=0))
        self.down.copy_(torch.cat([get(f"e{e}.down") for e in range(E)],
                                  dim=1))

    def forward(self, h, x, allow_gather: bool = True):
        fc = self.fc
        T, E = h.size(0), fc.experts
        logits = F.linear(x, self.router)                      # fp32 router
        weight = torch.empty(T, E + fc.identity, dtype=torch.float32,
                             device=h.device)
        ops.grouped_softmax_route(weight, logits, self.correction, fc.top,
                                  fc.groups, fc.keep_groups, fc.scale)
        ident = (weight[:, E:].sum(dim=-1) if fc.identity > 0 else None)
        if allow_gather and T >= self.SPARSE_MIN_TOKENS and E > fc.top:
            return self._gathered(h, weight), ident
        gu = ops.linear(h, self.gate_up)                       # [T, E*2F]
        act = torch.empty(T, E * fc.ff, dtype=h.dtype, device=h.device)
        ops.routed_clamped_glu(act, gu, weight, E, fc.limit, EXPERT_SLOPE)
        return ops.linear(act, self.down), ident

    def _gathered(self, h, weight):
        """Per-expert execution for prompt-sized batches: the rows routed
        to an expert are gathered, run through that expert only, and added
        back in fp32 in a fixed expert order."""
        fc = self.fc
        T, W = h.shape
        Fh = fc.ff
        out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
        hit = weight[:, :fc.experts] > 0
        counts = hit.sum(dim=0).tolist()                       # host sync
        for e in range(fc.experts):
            if counts[e] == 0:
                continue
            rows = hit[:, e].nonzero(as_tuple=True)[0]
            w = weight[rows, e].unsqueeze(1).contiguous()      # [n, 1] fp32
            gu = ops.linear(h.index_select(0, rows),
                            self.gate_up[e * 2 * Fh:(e + 1) * 2 * Fh])
            act = torch.empty(rows.numel(), Fh, dtype=h.dtype, device=h.device)
            ops.routed_clamped_glu(act, gu, w, 1, fc.limit, EXPERT_SLOPE)
            out.index_add_(0, rows, ops.linear(
                act, self.down[:, e * Fh:(e + 1) * Fh]).float())
        return out


class PekaraxLayer(torch.nn.Module):
    def __init__(self, cfg: PekaraxConfig, lc: PekaraxLayerConfig, dtype):
        super().__init__()
        W = cfg.hidden_size
        self.lc = lc
        # norm weights are kept as 1 + w
        self.norm1 = _param(W, dtype=torch.float32)
        self.attn = (MaskedAttention(W, lc.attn, cfg.norm_eps, dtype)
                     if lc.attn is not None else None)
        self.memory = MatrixMemoryMixer(W, lc.memory, cfg.norm_eps, dtype)
        if lc.mlp is None:
            self.norm2, self.mlp = None, None
        else:
            self.norm2 = _param(W, dtype=torch.float32)
            self.mlp = GroupRoutedExperts(W, lc.mlp, dtype)


class PekaraxForCausalLM(torch.nn.Module):
    def __init__(self, cfg: PekaraxConfig, device="cpu", tp_rank: int = 0,
                 tp_size: int = 1, seed: int = 0, dtype=torch.bfloat16):
        super().__init__()
        if tp_size != 1:
            raise ValueError("Pekarax: tensor parallelism is not implemented")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Pekarax: unsupported compute dtype {dtype}")
        self.cfg = cfg
        self.dtype = dtype
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        W = cfg.hidden_size
        with torch.device(device):
            self.embed = _param(cfg.vocab_size, W, dtype=dtype)
            self.layers = torch.nn.ModuleList(
                [PekaraxLayer(cfg, lc, dtype) for lc in cfg.layers])
            self.final_norm = _param(W, dtype=torch.float32)
            self.lm_head = _param(cfg.vocab_size, W, dtype=dtype)
        self.random_init(seed)
        # test hook: when a list, receives the residual after every layer
        self.residual_trace: Optional[list] = None

    @torch.no_grad()
    def random_init(self, seed: int = 0):
        gen = torch.Generator(device=self.embed.device).manual_seed(seed)

        def normal(p, std):
            p.copy_((torch.randn(p.shape, generator=gen, device=p.device,
                                 dtype=torch.float32) * std).to(p.dtype))

        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "norm_w"):
                p.fill_(1.0)
            elif leaf == "gate_bias":
                normal(p, 1.0)
            elif leaf == "head_rate":
                normal(p, 0.5)
            elif leaf == "correction":
                normal(p, 0.05)
            elif leaf == "w_conv":
                normal(p, 0.5)
            elif leaf in ("a2", "g2"):
                normal(p, 1.0)
            elif p.dim() >= 2:
                normal(p, 1.0 / p.size(-1) ** 0.5)
            else:
                p.fill_(0.0)
        normal(self.embed, 1.0)

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
        """Copy checkpoint tensors (embed, l<i>.norm1/2, l<i>.mix.*,
        l<i>.mlp.*, final.norm, head) into the fused serving layout."""
        dev, dt = self.embed.device, self.dtype

        def getter(prefix):
            def get(name):
                return sd[prefix + name].to(device=dev, dtype=dt)
            return get

        top = getter("")
        self.embed.copy_(top("embed"))
        self.lm_head.copy_(top("head"))
        self.final_norm.copy_(1.0 + top("final.norm").float())
        for i, layer in enumerate(self.layers):
            g = getter(f"l{i}.")
            layer.norm1.copy_(1.0 + g("norm1").float())
            if layer.attn is not None:
                layer.attn.load(getter(f"l{i}.mix.left."))
                layer.memory.load(getter(f"l{i}.mix.right."))
            else:
                layer.memory.load(getter(f"l{i}.mix."))
            if layer.mlp is not None:
                layer.norm2.copy_(1.0 + g("norm2").float())
                layer.mlp.load(getter(f"l{i}.mlp."))

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, md: AttnMetadata,
                kv_caches: List, last_rows: Optional[torch.Tensor] = None
                ) -> torch.Tensor:
        cfg = self.cfg
        eps, alpha = cfg.norm_eps, cfg.postln_alpha
        if md.state_slots is None:
            raise ValueError("Pekarax needs per-sequence state slots")
        h = F.embedding(input_ids, self.embed)           # GEMM input
        x = h.float() if h.dtype != torch.float32 else h.clone()
        tables: dict = {}      # rotary setting -> this step's cos/sin rows
        for i, layer in enumerate(self.layers):
            k_cache, v_cache, state = kv_caches[i]
            lc = layer.lc
            y = layer.memory(h, x, state, md)
            y2 = None
            if layer.attn is not None:
                y2 = layer.attn(h, k_cache, v_cache, md, tables,
                                conv_tail=state.get("attn_conv"))
            nxt = torch.empty_like(h)
            ops.postln_rmsnorm_residual(
                x, y, layer.norm1, eps, nxt, alpha=alpha,
                y_scale=lc.memory_scale, y2=y2, y2_scale=lc.attn_scale)
            h = nxt
            if layer.mlp is not None:
                y, ident = layer.mlp(h, x, allow_gather=md.is_prefill)
                nxt = torch.empty_like(h)
                ops.postln_rmsnorm_residual(x, y, layer.norm2, eps, nxt,
                                            alpha=alpha, row_add=ident)
                h = nxt
            if self.residual_trace is not None:
                self.residual_trace.append(x.clone())
        if last_rows is not None:
            x = x[last_rows]
        final = torch.empty(x.size(0), x.size(1), dtype=self.dtype,
                            device=x.device)
        ops.postln_rmsnorm_residual(x, None, self.final_norm, eps, final)
        return ops.linear(final, self.lm_head).float()


def _tiny(name: str) -> PekaraxConfig:
    experts = GroupedExpertsConfig(experts=6, identity=2, top=2, ff=64,
                                   limit=3.0, groups=4, keep_groups=2,
                                   scale=1.5)
    attn = MaskedAttentionConfig(
        heads=4, kv_heads=2, dim=32, vdim=32, scale=0.15,
        mask_kind=ops.MASK_CAUSAL, mask_size=0, rot_dims=16, rot_base=5e4,
        conv_taps=3)
    layers = [
        PekaraxLayerConfig("gla", memory=MatrixMemoryConfig(
            ops.SCAN_GLA, 2, 2, 32, 64, decay_rank=8, tau=8.0), mlp=experts),
        PekaraxLayerConfig("parallel", attn=attn, memory=MatrixMemoryConfig(
            ops.SCAN_MLSTM, 2, 2, 32, 32, gate_cap=10.0),
            attn_scale=0.7, memory_scale=1.1, mlp=experts),
        PekaraxLayerConfig("channel_delta", memory=MatrixMemoryConfig(
            ops.SCAN_DELTA, 4, 2, 32, 32, conv_taps=4, decay_rank=8,
            gate_rank=8), mlp=None),
    ]
    return PekaraxConfig(name=name, vocab_size=512, hidden_size=128,
                         layers=layers, norm_eps=1e-5, postln_alpha=2.0)


PEKARAX_CONFIGS: Dict[str, PekaraxConfig] = {
    "tiny-pekarax": _tiny("tiny-pekarax"),
}


def make_pekarax_instance(name: str, device: str, engine_cfg,
                          weights_path: Optional[str] = None):
    """ModelInstance over a Pekarax model (engine factory hook): a named
    random-init config, or a checkpoint directory."""
    from ..engine.llm import ModelInstance

    cfg = (config_from_checkpoint(weights_path) if weights_path
           else PEKARAX_CONFIGS[name])
    if device.startswith("cuda") and not (ops.masked_available()
                                          and ops.recurrent_available()):
        raise RuntimeError(
            "GPU engine requires the gfx950 masked-attention and recurrent "
            "extensions (python -m agentainer_amd.ops.build masked recurrent)")
    return ModelInstance(name, cfg, device, engine_cfg,
                         weights_path=weights_path,
                         model_cls=PekaraxForCausalLM)
