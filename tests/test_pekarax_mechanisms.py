"""Each Pekarax mechanism alone — op or module against the plain oracle —
on CPU (reference ops) and, marked gpu, on the HIP kernels. Where random
weights would hide a fault the inputs are built so that it shows: a key
far back that dominates the softmax, choice scores that are all negative,
a convolution tail that must be shifted rather than replaced."""

import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import pekarax_oracle as O  # noqa: E402

from agentainer_amd import ops  # noqa: E402
from agentainer_amd.models import pekarax as P  # noqa: E402
from agentainer_amd.models.llama import AttnMetadata  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64


def step_md(dev, lens_new, lens_before, slots, decode=False, page_table=None,
            slot_mapping=None):
    seq = torch.tensor([a + b for a, b in zip(lens_before, lens_new)],
                       dtype=torch.int32, device=dev)
    pos = torch.tensor([b + i for n, b in zip(lens_new, lens_before)
                        for i in range(n)], dtype=torch.int32, device=dev)
    md = AttnMetadata(page_table=page_table, seq_lens=seq,
                      slot_mapping=slot_mapping, positions=pos,
                      is_prefill=not decode,
                      state_slots=torch.tensor(slots, dtype=torch.long,
                                               device=dev))
    if not decode:
        st, acc = [], 0
        for n in lens_new:
            st.append(acc)
            acc += n
        md.query_starts = torch.tensor(st, dtype=torch.int32, device=dev)
        md.query_lens = torch.tensor(lens_new, dtype=torch.int32, device=dev)
        md.max_qlen = max(lens_new)
    return md


def rel(a, b):
    return float((a.double().cpu() - b.double()).abs().max()
                 / b.double().abs().max())


# ---- norm ------------------------------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
def test_post_norm_sum_eps_inside_root_and_offset_weight(device):
    g = torch.Generator().manual_seed(0)
    T, W, eps = 5, 24, 0.5                      # a large eps must matter
    x = torch.randn(T, W, generator=g) * 0.3
    y = torch.randn(T, W, generator=g) * 0.3
    y2 = torch.randn(T, W, generator=g) * 0.3
    w = torch.randn(W, generator=g) * 0.2       # stored around zero
    ra = torch.rand(T, generator=g)
    want = O.offset_norm((1.5 + ra.double().unsqueeze(1)) * x.double()
                         + 0.7 * y.double() + 1.3 * y2.double(), w.double(),
                         eps)
    xr = x.clone().to(device)
    h = torch.empty(T, W, device=device)
    ops.postln_rmsnorm_residual(xr, y.to(device), (1 + w).to(device), eps, h,
                                alpha=1.5, y_scale=0.7, y2=y2.to(device),
                                y2_scale=1.3, row_add=ra.to(device))
    assert rel(xr, want) < 1e-5 and rel(h, want) < 1e-5
    wrong = (1.5 * x.double() + y.double())
    wrong = wrong / (torch.sqrt((wrong ** 2).mean(-1, keepdim=True)) + eps)
    assert rel(xr, wrong * (1 + w.double())) > 1e-2


# ---- short convolution with a tail ----------------------------------------

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps", [2, 4, 5])
@pytest.mark.parametrize("sizes", [[1], [2], [3, 1, 2], [7, 1, 1, 1, 9]])
def test_short_conv_tail_over_cuts(device, taps, sizes):
    """Portions shorter than taps-1 shift the tail; the first tokens see
    zeros although the slot's tail holds another sequence's values."""
    g = torch.Generator().manual_seed(taps)
    C, T = 10, 23
    u = torch.randn(T, C, generator=g)
    w = torch.randn(C, taps, generator=g)
    want = O.causal_conv(u.double(), w.double())
    tail = torch.randn(3, taps - 1, C, generator=g).to(device)   # dirty
    out = torch.empty(T, C, device=device)
    at, k = 0, 0
    while at < T:
        n = min(sizes[k % len(sizes)], T - at)
        k += 1
        md = step_md(device, [n], [at], [1], decode=(n == 1 and at > 0))
        ops.short_conv_state(out[at:at + n], u[at:at + n].to(device),
                             w.t().contiguous().to(device), tail, md.state_slots, md.seq_lens,
                             md.query_starts, md.query_lens)
        at += n
    assert rel(out, want) < 1e-5
    assert rel(tail[1], u[T - taps + 1:]) < 1e-6


# ---- matrix memories ---------------------------------------------------------

def memory_module(kind, mx, w, prefix, width, eps, layer, device):
    mc = P._memory_from_dict(kind, mx, {k: list(v.shape) for k, v in w.items()},
                             prefix)
    mod = P.MatrixMemoryMixer(width, mc, eps, torch.float32)
    mod.load(lambda name: w[prefix + name])
    return mod.to(device), mc


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["gla", "channel_delta", "mlstm"])
def test_matrix_memory_mixers_over_cuts_and_slots(device, kind):
    """Each recurrence through its module: two sequences of unequal length
    in one batch, cut into portions and single tokens, in state slots that
    hold garbage; against the oracle on the whole sequences."""
    W, eps = 24, 1e-5
    layer = {"gla": O.gla_layer(heads=2, dim=12, vdim=20, tau=4.0, rank=3),
             "channel_delta": O.delta_layer(heads=4, kv_heads=2, dim=12,
                                            vdim=10, conv=3, rank=3, grank=4),
             "mlstm": O.parallel_layer(m_heads=3, m_dim=12, m_vdim=8,
                                       cap=6.0)}[kind]
    cfg = O.make_config([layer], width=W, no_ff=(0,))
    w = O.random_weights(cfg, seed=3)
    w64 = {k: v.double() for k, v in w.items()}
    prefix = "l0.mix.right." if kind == "mlstm" else "l0.mix."
    mx = layer["mixer"]["right"] if kind == "mlstm" else layer["mixer"]
    mod, mc = memory_module(kind, mx, w, prefix, W, eps, layer, device)
    g = torch.Generator().manual_seed(1)
    xs = {"a": torch.randn(21, W, generator=g), "b": torch.randn(9, W, generator=g)}
    fn = {"gla": O.gated_linear_attention, "channel_delta": O.channel_delta,
          "mlstm": O.mlstm_memory}[kind]
    want = {i: fn(x.double(), w64, prefix, mx, eps) for i, x in xs.items()}
    n_slots = 4
    state = {"S": torch.randn(n_slots, mc.heads, mc.vdim, mc.dim)}
    if kind == "mlstm":
        state["n"] = torch.randn(n_slots, mc.heads, mc.dim)
        state["m"] = torch.randn(n_slots, mc.heads)
    if mc.conv_taps > 0:
        state["conv"] = torch.randn(n_slots, mc.conv_taps - 1,
                                    mod.conv_channels)
    state = {k: v.to(device) for k, v in state.items()}
    slot = {"a": 2, "b": 0}
    sched = [[("a", 6), ("b", 2)], [("a", 1), ("b", 1)], [("a", 2), ("b", 1)],
             [("a", 12), ("b", 5)]]
    at = {"a": 0, "b": 0}
    got = {"a": [], "b": []}
    for step in sched:
        rows = torch.cat([xs[i][at[i]:at[i] + n] for i, n in step]).to(device)
        decode = all(n == 1 for _i, n in step)
        md = step_md(device, [n for _i, n in step], [at[i] for i, _n in step],
                     [slot[i] for i, _n in step], decode=decode)
        y = mod(rows, rows.clone(), state, md).cpu()
        k = 0
        for i, n in step:
            got[i].append(y[k:k + n])
            k += n
            at[i] += n
    for i in xs:
        assert rel(torch.cat(got[i]), want[i]) < 2e-4, (kind, i)


@pytest.mark.parametrize("device", DEVICES)
def test_mlstm_running_maximum_starts_at_zero(device):
    """With strongly negative input gates the stabilizer stays at its
    start value 0; a start at minus infinity would rescale the output."""
    H, D, Dv, T = 1, 4, 4, 3
    q = torch.ones(T, H, D)
    k = torch.ones(T, H, D) * 0.5
    v = torch.arange(T * Dv, dtype=torch.float32).view(T, H, Dv) + 1
    gate = torch.tensor([[-30.0, 30.0]] * T)          # i very small, f ~ 0
    bias = torch.zeros(2)
    S = torch.zeros(2, H, Dv, D)
    n = torch.zeros(2, H, D)
    m = torch.zeros(2, H)
    out = torch.zeros(T, H, Dv)
    md = step_md(device, [T], [0], [1])
    dv = lambda t: t.to(device)                        # noqa: E731
    S, n, m = dv(S), dv(n), dv(m)
    out = dv(out)
    ops.matrix_memory_scan(ops.SCAN_MLSTM, out, dv(q), dv(k), dv(v), dv(gate),
                           dv(bias), None, None, 1.0, 100.0, S, n, m,
                           md.state_slots, md.seq_lens, md.query_starts,
                           md.query_lens)
    # i = 100 tanh(-0.3), m stays 0: the write weighs e^i, den = e^0 = 1
    want0 = (math.exp(100.0 * math.tanh(-0.3)) * v[0, 0]
             * float((k[0, 0] * q[0, 0]).sum()))
    assert rel(out[0, 0], want0) < 1e-4
    assert float(m[1].abs().max()) < 1e-6


# ---- convolved attention -----------------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
def test_causal_attention_reads_a_key_far_back(device):
    """One key hundreds of positions back is scaled so that it dominates
    the softmax: queries at and after it return its value, queries before
    it do not; in a prompt portion and decoded, across page borders."""
    H, G, D, Dv, PS, T = 2, 1, 16, 8, 8, 300
    far = 37
    g = torch.Generator().manual_seed(5)
    kk = torch.randn(T, G, D, generator=g) * 0.1
    vv = torch.randn(T, G, Dv, generator=g)
    qq = torch.randn(T, H, D, generator=g) * 0.1
    beacon = torch.randn(D, generator=g)
    kk[far, 0] = beacon * 3
    qq[:, :] += beacon * 3
    n_pages = T // PS + 2
    perm = torch.randperm(n_pages - 1, generator=g) + 1
    pt = perm[:T // PS + 1].to(torch.int32).view(1, -1)
    k_cache = torch.zeros(n_pages, G, PS, D)
    v_cache = torch.zeros(n_pages, G, PS, Dv)
    for t in range(T):
        k_cache[pt[0, t // PS], :, t % PS] = kk[t]
        v_cache[pt[0, t // PS], :, t % PS] = vv[t]
    dv = lambda t: t.to(device)                        # noqa: E731
    # a portion of 280 tokens that ends at position 289
    n, end = 280, 290
    out = torch.zeros(n, H, Dv, device=device)
    ops.masked_attention(out, dv(qq[end - n:end].contiguous()), dv(k_cache),
                         dv(v_cache), dv(pt),
                         torch.tensor([end], dtype=torch.int32, device=device),
                         torch.tensor([0], dtype=torch.int32, device=device),
                         torch.tensor([n], dtype=torch.int32, device=device),
                         1.0, ops.MASK_CAUSAL, 0, max_qlen=n)
    out = out.cpu()
    first = end - n
    for t in (far, far + 1, 150, end - 1):
        assert float((out[t - first, 0] - vv[far, 0]).abs().max()) < 1e-2, t
    assert float((out[far - 1 - first, 0] - vv[far, 0]).abs().max()) > 0.1
    # the last token decoded alone
    o1 = torch.zeros(1, H, Dv, device=device)
    ops.masked_attention(o1, dv(qq[T - 1:T].contiguous()), dv(k_cache),
                         dv(v_cache), dv(pt),
                         torch.tensor([T], dtype=torch.int32, device=device),
                         None, None, 1.0, ops.MASK_CAUSAL, 0)
    assert float((o1.cpu()[0, 1] - vv[far, 0]).abs().max()) < 1e-2


@pytest.mark.parametrize("device", DEVICES)
def test_conv_attention_module_over_cuts(device):
    """The attention with its q|k|v convolution over a shuffled paged pool,
    cut into portions and single tokens, against the oracle."""
    W, eps, PS = 24, 1e-5, 4
    layer = O.parallel_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=4,
                             rot_dims=4, base=50.0, scale=0.9)
    cfg = O.make_config([layer], width=W, no_ff=(0,))
    w = O.random_weights(cfg, seed=7)
    mx = layer["mixer"]["left"]
    mc = P._attention_from_dict(mx)
    mod = P.MaskedAttention(W, mc, eps, torch.float32)
    mod.load(lambda name: w["l0.mix.left." + name])
    mod = mod.to(device)
    T = 27
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, W, generator=g)
    want = O.conv_attention(x.double(), {k: v.double() for k, v in w.items()},
                            "l0.mix.left.", mx, eps)
    n_pages = 12
    k_cache = torch.zeros(n_pages, 2, PS, 8, device=device)
    v_cache = torch.zeros(n_pages, 2, PS, 6, device=device)
    pages = [7, 2, 9, 4, 11, 1, 5]
    tail = torch.randn(3, 3, mod.conv_channels).to(device)
    got, at = [], 0
    for n in (5, 1, 2, 1, 1, 9, 1, 7):
        slots = torch.tensor([pages[t // PS] * PS + t % PS
                              for t in range(at, at + n)], device=device)
        md = step_md(device, [n], [at], [2], decode=(n == 1),
                     page_table=torch.tensor([pages], dtype=torch.int32,
                                             device=device),
                     slot_mapping=slots)
        got.append(mod(x[at:at + n].to(device), k_cache, v_cache, md, {},
                       conv_tail=tail).cpu())
        at += n
    assert rel(torch.cat(got), want) < 2e-4


# ---- routing and experts -----------------------------------------------------

@pytest.mark.parametrize("device", DEVICES)
def test_group_limited_choice_with_negative_scores(device):
    """All choice scores are negative (large negative correction): experts
    of dropped groups must count as minus infinity — a 0 would win. The
    weights use the scores WITHOUT the correction and sum to `scale`."""
    T, E = 40, 12
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(T, E, generator=g) * 2
    corr = -1.0 - torch.rand(E, generator=g)
    wt = torch.empty(T, E, device=device)
    ops.grouped_softmax_route(wt, logits.to(device), corr.to(device), 3, 4, 2,
                              1.75)
    wt = wt.cpu()
    s = torch.softmax(logits.double(), -1)
    c = s + corr.double()
    for t in range(T):
        best = sorted(range(4), key=lambda k: -float(c[t, 3 * k:3 * k + 3].max()))[:2]
        cand = sorted([e for e in range(E) if e // 3 in best],
                      key=lambda e: -float(c[t, e]))[:3]
        chosen = sorted(int(e) for e in wt[t].nonzero().flatten())
        assert chosen == sorted(cand), t
        want = s[t, cand] / s[t, cand].sum() * 1.75
        assert rel(wt[t, cand], want) < 1e-5
    assert rel(wt.sum(-1), torch.full((T,), 1.75)) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [7, 300])
def test_experts_module_both_forms(device, T):
    """Stacked (few tokens) and gathered (many tokens) execution, with
    identity experts, clamps that bite, against the oracle."""
    W = 16
    ml = O.moe(experts=5, identity=3, top=3, ff=12, limit=0.8, groups=4,
               keep=3, scale=1.9)
    cfg = O.make_config([O.gla_layer()], width=W, mlp=ml)
    w = O.random_weights(cfg, seed=4)
    fc = P.config_from_dict(O.checkpoint_config(cfg)).layers[0].mlp
    mod = P.GroupRoutedExperts(W, fc, torch.float32)
    mod.load(lambda name: w["l0.mlp." + name])
    mod = mod.to(device)
    g = torch.Generator().manual_seed(9)
    h = torch.randn(T, W, generator=g) * 2
    want = O.experts(h.double(), {k: v.double() for k, v in w.items()},
                     "l0.mlp.", ml)
    y, ident = mod(h.to(device), h.clone().to(device), allow_gather=True)
    got = y.double().cpu() + ident.double().cpu().unsqueeze(1) * h.double()
    assert rel(got, want) < 2e-5
    assert float(ident.max()) > 0          # identity experts were chosen


# ---- config reader -------------------------------------------------------------

def test_config_reader_takes_ranks_from_tensor_shapes(tmp_path):
    cfg = O.make_config([O.delta_layer(rank=3, grank=7), O.gla_layer(rank=5),
                         O.parallel_layer()], no_ff=(1,))
    w = O.random_weights(cfg, seed=0)
    O.save_checkpoint(str(tmp_path / "c"), cfg, w)
    pc = P.config_from_checkpoint(str(tmp_path / "c"))
    assert pc.layers[0].memory.decay_rank == 3
    assert pc.layers[0].memory.gate_rank == 7
    assert pc.layers[1].memory.decay_rank == 5 and pc.layers[1].mlp is None
    assert pc.layers[2].attn.conv_taps == 3 and pc.layers[2].attn_scale == 0.75
    assert pc.layers[2].memory.kind == ops.SCAN_MLSTM
    shapes = pc.state_shapes()
    assert shapes[0]["S"] == (4, 6, 8) and shapes[0]["conv"] == (3, 56)
    assert set(shapes[2]) == {"attn_conv", "S", "n", "m"}
    bad = O.checkpoint_config(cfg)
    bad["layers"][0]["type"] = "unknown"
    with pytest.raises(ValueError):
        P.config_from_dict(bad)
