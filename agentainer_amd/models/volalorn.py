"""Volalorn family — post-normed decoder with two masked-attention mixers.

Every layer updates an fp32 residual stream x with NORMED sublayer
outputs; the sublayers read x itself:

    x <- x + n1(mixer(x));   x <- x + n2(ff(x));   n(y) = g * y / rms(y)

with a single scalar gain g per norm. The layer list of config.json picks,
per layer, one of two grouped-query attention mixers (each with its own
head counts, key size, value size, rotary settings and mask):

  * "attention"   — rotary on the first `rot.dims` coordinates (optionally
    YaRN-stretched), then weightless unit-rms of q and k; tanh soft-capped
    scores; CHUNK mask (a query sees the earlier keys of its own block of
    `mask.size` positions); every visible key is weighted by
    sigmoid(score + bias[head]) with no normalization over keys; a
    sigmoid gate per head, read from the mixer input, scales the head.
  * "attention_2" — biased q/k/v projections; weighted rms norm of q and k
    (one weight vector shared by all heads) BEFORE the rotary; sliding
    WINDOW that also keeps the first `mask.keep_first` positions; softmax.

The feed-forward is down(PolyNorm(up x)), PolyNorm(z) = a U(z) + b U(z^2)
+ c U(z^3) + e with U = unit rms over the row. The head multiplies the
logits by `logit_scale`.

Serving design (what runs on the MI355X):

  * q, k, v (and the head-gate logits) come out of ONE GEMM; one fused
    kernel (ops.rotary_norm_append) rotates / normalizes q in place and k
    on its way into the paged pool and copies v there. The cos/sin rows of
    a step's positions (ops.rotary_table, fp32 angles) are computed once
    per step and rotary setting and shared by all layers that have it. The engine's
    KVCacheManager owns the pools through HeadKVLayout — per layer
    K [pages, G, page, dim] and V [pages, G, page, vdim].
  * ops.masked_attention serves prompt portions and single decoded tokens
    with one kernel family: mask kind / size / kept prefix, soft cap,
    sigmoid-vs-softmax weighting, per-head key bias and the per-head
    output gate are arguments, so scores never leave registers and the
    gate costs no extra pass.
  * ops.scalar_postnorm_residual fuses norm, gain, the fp32 residual
    update and the cast that feeds the next GEMM; ops.poly_norm is one
    pass over the ff activations.
  * Plain projections go to hipBLASLt through ops.linear.

compute dtype: bf16 (serving default; rotary angles, norms, scores,
weights, PolyNorm statistics and the residual stay fp32) or float32
(everything fp32 — a verification mode).
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import ops
from .llama import AttnMetadata

# the fused input GEMM's row count is padded so every token row of its
# output starts 16-byte aligned (bf16)
PROJ_ALIGN = 8


@dataclass
class MaskedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int                  # query/key size per head
    vdim: int                 # value size per head
    scale: float
    mask_kind: int            # ops.MASK_CAUSAL / MASK_WINDOW / MASK_CHUNK
    mask_size: int
    keep_first: int = 0       # window mask: positions < keep_first stay seen
    rot_dims: int = 0         # leading coordinates of a head that rotate
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None   # YaRN: factor, original, fast, slow
    softcap: float = 0.0      # 0 = scores are not capped
    sigmoid_weights: bool = False        # per-key sigmoid instead of softmax
    key_bias: bool = False    # per-head number added to every score
    head_gate: bool = False   # per-head sigmoid gate read from the input
    qkv_bias: bool = False
    norm_first: bool = False  # True: weighted q/k norm, then rotary;
    #                           False: rotary, then weightless unit rms
    conv_taps: int = 0        # > 0: a depthwise causal convolution over time
    #                           on the projected q, k, v (before norm and
    #                           rotary); its last taps-1 inputs are
    #                           per-sequence state
    plain_qk: bool = False    # q and k enter the scores as projected (and
    #                           convolved): no rotary, no norm
    dist_bias: bool = False   # per head (r1, r2): r1 ln(1 + r2 (p - j)) is
    #                           taken off the score of key j at query p
    elem_gate: bool = False   # sigmoid gate per OUTPUT COORDINATE, read
    #                           from the mixer input
    kv_from: Optional[int] = None   # this layer has no k/v projections: it
    #                           attends the pools of that (earlier) layer


@dataclass
class PolyFeedForwardConfig:
    ff: int


@dataclass
class VolalornLayerConfig:
    kind: str                                  # the config's mixer type
    mixer: MaskedAttentionConfig
    mlp: Optional[PolyFeedForwardConfig]


@dataclass
class VolalornConfig:
    name: str = "tiny-volalorn"
    vocab_size: int = 512
    hidden_size: int = 128
    layers: List[VolalornLayerConfig] = field(default_factory=list)
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    family: str = "volalorn"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def max_position(self) -> int:
        return 1 << 30   # rotary angles are computed from the position

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return sum(l.mixer.kv_heads * (l.mixer.dim + l.mixer.vdim)
                   for l in self.layers) * dtype_bytes

    def cache_layout(self):
        from ..engine.kvcache import HeadKVLayout
        return HeadKVLayout([(l.mixer.kv_heads, l.mixer.dim, l.mixer.vdim)
                             for l in self.layers])


def mixer_from_dict(kind: str, mx: dict) -> MaskedAttentionConfig:
    """One layer's mixer section -> MaskedAttentionConfig."""
    rot = mx.get("rot") or {}
    mask = mx.get("mask") or {}
    common = dict(
        heads=int(mx["heads"]), kv_heads=int(mx["kv_heads"]),
        dim=int(mx["dim"]), vdim=int(mx["vdim"]), scale=float(mx["scale"]),
        mask_size=int(mask.get("size", 0)),
        rot_dims=int(rot.get("dims", 0)),
        rot_base=float(rot.get("base", 10000.0)),
        rot_scaling=(dict(rot["scaling"]) if rot.get("scaling") else None),
        softcap=float(mx.get("softcap") or 0.0))
    if kind == "attention":
        return MaskedAttentionConfig(
            mask_kind=ops.MASK_CHUNK, sigmoid_weights=True, key_bias=True,
            head_gate=True, norm_first=False, **common)
    if kind == "attention_2":
        return MaskedAttentionConfig(
            mask_kind=ops.MASK_WINDOW,
            keep_first=int(mask.get("keep_first", 0)), qkv_bias=True,
            norm_first=True, **common)
    raise ValueError(f"unsupported mixer {kind!r}")


def config_from_dict(d: dict, name: str = "volalorn") -> VolalornConfig:
    """VolalornConfig from a parsed config.json."""
    layers = []
    for i, ld in enumerate(d["layers"]):
        mixer = mixer_from_dict(ld["type"], ld["mixer"])
        if mixer.heads % mixer.kv_heads:
            raise ValueError(f"layer {i}: heads % kv_heads != 0")
        if mixer.rot_dims % 2 or mixer.rot_dims > mixer.dim:
            raise ValueError(f"layer {i}: bad rot.dims {mixer.rot_dims}")
        if mixer.mask_size < 1:
            raise ValueError(f"layer {i}: mask.size must be >= 1")
        ml = ld.get("mlp")
        if ml is None:
            mlp = None
        elif ml["kind"] == "dense":
            mlp = PolyFeedForwardConfig(int(ml["ff"]))
        else:
            raise ValueError(f"layer {i}: unsupported mlp {ml['kind']!r}")
        layers.append(VolalornLayerConfig(ld["type"], mixer, mlp))
    return VolalornConfig(
        name=name, vocab_size=int(d["vocab"]), hidden_size=int(d["width"]),
        layers=layers, norm_eps=float(d["norm"]["eps"]),
        logit_scale=float(d.get("logit_scale", 1.0)))


def config_from_checkpoint(path: str) -> VolalornConfig:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=path)


def _param(*shape, dtype):
    return torch.nn.Parameter(torch.empty(*shape, dtype=dtype),
                              requires_grad=False)


def _align(n: int) -> int:
    return -(-n // PROJ_ALIGN) * PROJ_ALIGN


class MaskedAttention(torch.nn.Module):
    """Grouped-query attention with a configurable mask, weighting, q/k
    normalization order and output gate (see MaskedAttentionConfig)."""

    def __init__(self, width: int, mc: MaskedAttentionConfig, eps: float,
                 dtype, extra_rows: int = 0):
        """extra_rows: that many more rows ride in the input GEMM (a
        projection of the same input that belongs to the caller, e.g. a
        residual gate); forward then returns (output, their columns)."""
        super().__init__()
        self.mc = mc
        self.eps = eps
        H, G = mc.heads, mc.kv_heads
        own_kv = mc.kv_from is None
        self.q_sz = H * mc.dim
        self.k_sz = G * mc.dim if own_kv else 0
        self.v_sz = G * mc.vdim if own_kv else 0
        self.gate_sz = (H if mc.head_gate else
                        H * mc.vdim if mc.elem_gate else 0)
        # segment starts stay 16-byte aligned for the kernels' vector loads
        self.gate_off = _align(self.q_sz + self.k_sz + self.v_sz)
        self.extra_rows = extra_rows
        self.extra_off = _align(self.gate_off + self.gate_sz)
        self.n_in = _align(self.extra_off + extra_rows)
        # one GEMM from the mixer input: [q | k | v | gate logits | extra]
        self.w_in = _param(self.n_in, width, dtype=dtype)
        self.b_in = _param(self.n_in, dtype=dtype) if mc.qkv_bias else None
        f32 = torch.float32
        self.q_norm = _param(mc.dim, dtype=f32) if mc.norm_first else None
        self.k_norm = _param(mc.dim, dtype=f32) if mc.norm_first else None
        self.key_bias = _param(H, dtype=f32) if mc.key_bias else None
        self.dist_bias = _param(H, 2, dtype=f32) if mc.dist_bias else None
        self.w_o = _param(width, H * mc.vdim, dtype=dtype)
        self.conv_channels = self.q_sz + self.k_sz + self.v_sz
        self.w_conv = (_param(mc.conv_taps, self.conv_channels, dtype=f32)
                       if mc.conv_taps > 0 else None)
        freqs, self.rot_amp = ops.rotary_frequencies(
            mc.rot_dims, mc.rot_base, mc.rot_scaling)
        self.register_buffer("rot_freqs", freqs, persistent=False)

    @torch.no_grad()
    def load(self, get, extra=None):
        """extra: weight rows [extra_rows, width] of the caller's
        projection."""
        mc = self.mc
        own_kv = mc.kv_from is None
        q0, k0, v0 = 0, self.q_sz, self.q_sz + self.k_sz
        g0 = self.gate_off
        self.w_in.zero_()
        self.w_in[q0:k0].copy_(get("q"))
        if own_kv:
            self.w_in[k0:v0].copy_(get("k"))
            self.w_in[v0:v0 + self.v_sz].copy_(get("v"))
        if self.gate_sz:
            self.w_in[g0:g0 + self.gate_sz].copy_(get("g"))
        if extra is not None:
            self.w_in[self.extra_off:self.extra_off + self.extra_rows].copy_(
                extra)
        if mc.qkv_bias:
            self.b_in.zero_()
            self.b_in[q0:k0].copy_(get("q.b"))
            if own_kv:
                self.b_in[k0:v0].copy_(get("k.b"))
                self.b_in[v0:v0 + self.v_sz].copy_(get("v.b"))
        if mc.norm_first:
            self.q_norm.copy_(get("q.norm").float())
            self.k_norm.copy_(get("k.norm").float())
        if mc.key_bias:
            self.key_bias.copy_(get("pb").float())
        if mc.dist_bias:
            self.dist_bias.copy_(torch.stack(
                [get("r1").float(), get("r2").float()], dim=1))
        self.w_o.copy_(get("o"))
        if mc.conv_taps > 0:
            # checkpoint [channels, taps] -> tap-major [taps, channels]
            names = ["q.conv"] + (["k.conv", "v.conv"] if own_kv else [])
            self.w_conv.copy_(torch.cat([get(n) for n in names],
                                        dim=0).float().t())

    def rotary_key(self):
        """Layers with equal keys share one cos/sin table per step."""
        mc = self.mc
        sc = mc.rot_scaling
        return (mc.rot_dims, mc.rot_base,
                tuple(sorted(sc.items())) if sc else None)

    def forward(self, h: torch.Tensor, k_cache: torch.Tensor,
                v_cache: torch.Tensor, md: AttnMetadata,
                tables: Optional[dict] = None,
                conv_tail: Optional[torch.Tensor] = None) -> torch.Tensor:
        """conv_tail [slots, taps-1, q+k+v channels] fp32 (the cache
        manager's per-sequence state) is required when conv_taps > 0."""
        mc = self.mc
        cos_sin = None
        if not mc.plain_qk:
            key = self.rotary_key()
            cos_sin = tables.get(key) if tables is not None else None
            if cos_sin is None:
                cos_sin = ops.rotary_table(md.positions, self.rot_freqs,
                                           self.rot_amp)
                if tables is not None:
                    tables[key] = cos_sin
        T, H, G = h.size(0), mc.heads, mc.kv_heads
        own_kv = mc.kv_from is None
        proj = ops.linear(h, self.w_in, bias=self.b_in)
        k0, v0 = self.q_sz, self.q_sz + self.k_sz
        c_end = v0 + self.v_sz
        g0 = self.gate_off
        qkv = proj
        if mc.conv_taps > 0:
            qkv = torch.empty(T, c_end, dtype=h.dtype, device=h.device)
            ops.short_conv_state(
                qkv, proj[:, :c_end], self.w_conv, conv_tail, md.state_slots,
                md.seq_lens, md.query_starts if md.is_prefill else None,
                md.query_lens if md.is_prefill else None)
        # strided views into the GEMM output: the kernels take row strides
        q = qkv[:, :k0].view(T, H, mc.dim)
        if own_kv:
            k = qkv[:, k0:v0].view(T, G, mc.dim)
            v = qkv[:, v0:c_end].view(T, G, mc.vdim)
            if mc.plain_qk:
                ops.head_kv_append(k, v, k_cache, v_cache,
                                   md.slot_mapping)
            else:
                ops.rotary_norm_append(q, k, v, k_cache, v_cache, cos_sin,
                                       md.slot_mapping, self.eps, self.q_norm,
                                       self.k_norm, mc.norm_first)
        out = torch.empty(T, H, mc.vdim, dtype=h.dtype, device=h.device)
        ops.masked_attention(
            out, q, k_cache, v_cache, md.page_table, md.seq_lens,
            md.query_starts if md.is_prefill else None,
            md.query_lens if md.is_prefill else None,
            mc.scale, mc.mask_kind, mc.mask_size, mc.keep_first,
            mc.sigmoid_weights, mc.softcap, self.key_bias,
            proj[:, g0:g0 + self.gate_sz] if self.gate_sz else None,
            max_qlen=md.max_qlen if md.is_prefill else 1,
            dist_bias=self.dist_bias)
        y = ops.linear(out.view(T, H * mc.vdim), self.w_o)
        if self.extra_rows:
            return y, proj[:, self.extra_off:self.extra_off + self.extra_rows]
        return y


class PolyNormFeedForward(torch.nn.Module):
    """down( PolyNorm(up h) )."""

    def __init__(self, width: int, ff: int, eps: float, dtype):
        super().__init__()
        self.ff, self.eps = ff, eps
        self.up = _param(ff, width, dtype=dtype)
        self.down = _param(width, ff, dtype=dtype)
        self.coef = _param(4, dtype=torch.float32)     # a, b, c, e

    @torch.no_grad()
    def load(self, get):
        self.up.copy_(get("up"))
        self.down.copy_(get("down"))
        self.coef.copy_(get("act").float())

    def forward(self, h):
        z = ops.linear(h, self.up)
        act = torch.empty_like(z)
        ops.poly_norm(act, z, self.coef, self.eps)
        return ops.linear(act, self.down)


class VolalornLayer(torch.nn.Module):
    def __init__(self, cfg: VolalornConfig, lc: VolalornLayerConfig, dtype):
        super().__init__()
        W = cfg.hidden_size
        self.norm1 = _param(1, dtype=torch.float32)
        self.mix = MaskedAttention(W, lc.mixer, cfg.norm_eps, dtype)
        if lc.mlp is None:
            self.norm2, self.mlp = None, None
        else:
            self.norm2 = _param(1, dtype=torch.float32)
            self.mlp = PolyNormFeedForward(W, lc.mlp.ff, cfg.norm_eps, dtype)


class VolalornForCausalLM(torch.nn.Module):
    def __init__(self, cfg: VolalornConfig, device="cpu", tp_rank: int = 0,
                 tp_size: int = 1, seed: int = 0, dtype=torch.bfloat16):
        super().__init__()
        if tp_size != 1:
            raise ValueError("Volalorn: tensor parallelism is not implemented")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Volalorn: unsupported compute dtype {dtype}")
        self.cfg = cfg
        self.dtype = dtype
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        W = cfg.hidden_size
        with torch.device(device):
            self.embed = _param(cfg.vocab_size, W, dtype=dtype)
            self.layers = torch.nn.ModuleList(
                [VolalornLayer(cfg, lc, dtype) for lc in cfg.layers])
            self.final_norm = _param(1, dtype=torch.float32)
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
            if name.endswith(".coef"):
                p.copy_(torch.tensor([1.0, 0.5, 0.25, 0.0], device=p.device))
            elif name.endswith(".key_bias"):
                p.fill_(-1.0)
            elif name.endswith(".b_in"):
                normal(p, 0.1)
            elif p.dim() >= 2:
                normal(p, 1.0 / p.size(-1) ** 0.5)
            else:
                p.fill_(1.0)                      # gains and norm weights
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
        """Copy checkpoint tensors (named embed, l<i>.norm1/2, l<i>.mix.*,
        l<i>.mlp.*, final.norm, head) into the fused serving layout."""
        dev, dt = self.embed.device, self.dtype

        def getter(prefix):
            def get(name):
                return sd[prefix + name].to(device=dev, dtype=dt)
            return get

        top = getter("")
        self.embed.copy_(top("embed"))
        self.lm_head.copy_(top("head"))
        self.final_norm.copy_(top("final.norm").float().reshape(1))
        for i, layer in enumerate(self.layers):
            g = getter(f"l{i}.")
            layer.norm1.copy_(g("norm1").float().reshape(1))
            layer.mix.load(getter(f"l{i}.mix."))
            if layer.mlp is not None:
                layer.norm2.copy_(g("norm2").float().reshape(1))
                layer.mlp.load(getter(f"l{i}.mlp."))

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, md: AttnMetadata,
                kv_caches: List, last_rows: Optional[torch.Tensor] = None
                ) -> torch.Tensor:
        cfg = self.cfg
        eps = cfg.norm_eps
        h = F.embedding(input_ids, self.embed)           # GEMM input
        x = h.float() if h.dtype != torch.float32 else h.clone()

        def add_normed(y, gain):
            nxt = torch.empty_like(h)
            ops.scalar_postnorm_residual(x, y, gain, eps, nxt)
            return nxt

        tables: dict = {}      # rotary setting -> this step's cos/sin rows
        for i, layer in enumerate(self.layers):
            k_cache, v_cache = kv_caches[i]
            h = add_normed(layer.mix(h, k_cache, v_cache, md, tables),
                           layer.norm1)
            if layer.mlp is not None:
                h = add_normed(layer.mlp(h), layer.norm2)
            if self.residual_trace is not None:
                self.residual_trace.append(x.clone())
        if last_rows is not None:
            x = x[last_rows]
        final = torch.empty(x.size(0), x.size(1), dtype=self.dtype,
                            device=x.device)
        ops.scalar_rmsnorm(final, x, self.final_norm, eps)
        logits = ops.linear(final, self.lm_head).float()
        if cfg.logit_scale != 1.0:
            logits = logits * cfg.logit_scale
        return logits


def _tiny(name: str) -> VolalornConfig:
    sig = MaskedAttentionConfig(
        heads=4, kv_heads=2, dim=32, vdim=32, scale=32 ** -0.5,
        mask_kind=ops.MASK_CHUNK, mask_size=32, rot_dims=16,
        rot_base=10000.0, rot_scaling={"factor": 4.0, "original": 256,
                                       "fast": 16.0, "slow": 2.0},
        softcap=30.0, sigmoid_weights=True, key_bias=True, head_gate=True)
    soft = MaskedAttentionConfig(
        heads=4, kv_heads=1, dim=32, vdim=16, scale=32 ** -0.5,
        mask_kind=ops.MASK_WINDOW, mask_size=40, keep_first=2, rot_dims=32,
        rot_base=10000.0, qkv_bias=True, norm_first=True)
    layers = [VolalornLayerConfig("attention", sig, PolyFeedForwardConfig(256)),
              VolalornLayerConfig("attention_2", soft,
                                  PolyFeedForwardConfig(256))]
    return VolalornConfig(name=name, vocab_size=512, hidden_size=128,
                          layers=layers, norm_eps=1e-5, logit_scale=0.75)


VOLALORN_CONFIGS: Dict[str, VolalornConfig] = {
    "tiny-volalorn": _tiny("tiny-volalorn"),
}


def make_volalorn_instance(name: str, device: str, engine_cfg,
                           weights_path: Optional[str] = None):
    """ModelInstance over a Volalorn model (engine factory hook): a named
    random-init config, or a checkpoint directory."""
    from ..engine.llm import ModelInstance

    cfg = (config_from_checkpoint(weights_path) if weights_path
           else VOLALORN_CONFIGS[name])
    if device.startswith("cuda") and not ops.masked_available():
        raise RuntimeError(
            "GPU engine requires the gfx950 masked-attention extension "
            "(python -m agentainer_amd.ops.build masked)")
    return ModelInstance(name, cfg, device, engine_cfg,
                         weights_path=weights_path,
                         model_cls=VolalornForCausalLM)
