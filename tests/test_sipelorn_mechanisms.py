"""Sipelorn's mechanisms one at a time: each framework op (CPU reference
and, marked gpu, the HIP kernel) against the plain float64 oracle function
of the same mechanism. Where random inputs would hide a fault — a key at
the window's edge, a far key, the first token's bigram row, a group whose
scores are negative — inputs are made so that it shows."""

import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import sipelorn_oracle as O  # noqa: E402

from agentainer_amd import ops  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).bfloat16().float()


def close(got, want, dtype, tol32=2e-5):
    tol = tol32 if dtype == torch.float32 else 2e-2
    err = float((got.double().cpu() - want).abs().max()
                / want.abs().max().clamp(min=1e-6))
    assert err < tol, err


# ------------------------------------------------------------- embedding

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("bigram", [True, False])
def test_bigram_embedding_with_previous_token_state(device, bigram):
    """Two sequences in portions, then one token each; slot 2 still holds a
    stranger's token when the second sequence starts at position 0 there."""
    V, W = 50, 12
    bg = {"buckets": 13, "mul_prev": 7, "mul_cur": 5}
    w = {"embed": rnd(V, W, seed=1).double(),
         "bigram": rnd(14, W, seed=2).double()}
    cfg = {"embedding": {"scale": 3.0, **({"bigram": bg} if bigram else {})}}
    seqs = {0: [4, 9, 9, 33, 2, 17], 2: [8, 41, 41, 5]}
    want = {s: O.embed_tokens(t, w, cfg) for s, t in seqs.items()}
    emb = w["embed"].float().to(device)
    big = w["bigram"].float().to(device) if bigram else None
    state = torch.full((4,), 49, dtype=torch.int32, device=device)

    def run(rows, lens_after, starts, qlens):
        ids = torch.tensor([t for _s, ts in rows for t in ts], device=device)
        x = torch.empty(ids.numel(), W, device=device)
        i32 = dict(dtype=torch.int32, device=device)
        ops.bigram_embed(
            x, ids, emb, big, 3.0, bg["mul_prev"], bg["mul_cur"],
            bg["buckets"], state,
            torch.tensor([s for s, _ in rows], device=device),
            torch.tensor(lens_after, **i32),
            None if starts is None else torch.tensor(starts, **i32),
            None if qlens is None else torch.tensor(qlens, **i32))
        return x.double().cpu()

    x = run([(0, seqs[0][:3]), (2, seqs[2][:1])], [3, 1], [0, 3], [3, 1])
    assert torch.allclose(x[:3], want[0][:3], atol=1e-5)
    assert torch.allclose(x[3:], want[2][:1], atol=1e-5)
    x = run([(0, seqs[0][3:5]), (2, seqs[2][1:3])], [5, 3], [0, 2], [2, 2])
    assert torch.allclose(x[:2], want[0][3:5], atol=1e-5)
    assert torch.allclose(x[2:], want[2][1:3], atol=1e-5)
    x = run([(0, seqs[0][5:]), (2, seqs[2][3:])], [6, 4], None, None)
    assert torch.allclose(x[:1], want[0][5:], atol=1e-5)
    assert torch.allclose(x[1:], want[2][3:], atol=1e-5)
    if bigram:
        assert state.tolist() == [17, 49, 5, 49]


# ------------------------------------------------- residual update + norm

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [64, 50, 1200])
def test_gated_residual_and_layer_norm(device, dtype, W):
    T, eps = 5, 1e-3
    x0 = rnd(T, W, seed=1, scale=3.0) + 2.0          # mean far from zero
    y, gl = rnd(T, W, seed=2), rnd(T, W, seed=3, scale=2.0)
    gb, nw, nb, rw = (rnd(W, seed=s) for s in (4, 5, 6, 7))
    xd = x0.double()
    x_gate = xd + torch.sigmoid(gl.double() + gb.double()) * y.double()
    x_rms = xd + O.rms_unit(y.double(), eps) * rw.double()
    d = lambda t: t.to(device)                       # noqa: E731
    c = lambda t: t.to(device=device, dtype=dtype)   # noqa: E731
    for upd, want_x, kw in (
            (ops.UPDATE_SIGMOID_GATE, x_gate, dict(gate=c(gl), gb=d(gb))),
            (ops.UPDATE_UNIT_RMS, x_rms, dict(rw=d(rw))),
            (ops.UPDATE_NONE, xd, {})):
        for norm in (True, False):
            x = d(x0.clone())
            h = torch.empty(T, W, device=device, dtype=dtype)
            ops.residual_update_norm(
                x, None if upd == ops.UPDATE_NONE else c(y), upd,
                kw.get("gate"), kw.get("gb"), kw.get("rw"), eps,
                d(nw) if norm else None, d(nb) if norm else None, h)
            close(x, want_x, torch.float32, 1e-6)
            want_h = (O.layer_norm(want_x, nw.double(), nb.double(), eps)
                      if norm else want_x)
            close(h, want_h, dtype, 1e-5)
    # eps sits inside both roots: tiny rows are not blown up
    x = d(torch.full((1, W), 1e-4) + rnd(1, W, seed=9, scale=1e-4))
    want = O.layer_norm(x.double().cpu(), nw.double(), nb.double(), eps)
    h = torch.empty(1, W, device=device)
    ops.residual_update_norm(x, None, ops.UPDATE_NONE, None, None, None, eps,
                             d(nw), d(nb), h)
    close(h, want, torch.float32, 1e-5)


# ------------------------------------------------------------ activations

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_xielu_both_branches_and_strided_input(device, dtype):
    p, q = torch.tensor(0.3, dtype=F64), torch.tensor(-0.7, dtype=F64)
    z = torch.cat([rnd(6, 40, seed=1, scale=2.5),
                   torch.tensor([[0.0, -1e-3, 1e-3, -9.0, 9.0] * 8])])
    wide = torch.zeros(7, 56)
    wide[:, :40] = z
    coef = torch.tensor([float(O.softplus(p)), 0.5 + float(O.softplus(q))],
                        device=device)
    out = torch.empty(7, 40, device=device, dtype=dtype)
    ops.xielu(out, wide.to(device=device, dtype=dtype)[:, :40], coef)
    close(out, O.xielu(z.double(), p, q), dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_token_side_gate(device, dtype):
    T, d, layer = 9, 6, 2
    t = rnd(T, d, seed=1, scale=2.0)
    table = rnd(30, 4 * d, seed=2)
    ids = torch.tensor([3, 3, 29, 0, 7, 7, 12, 1, 29])
    out = torch.empty(T, d, device=device, dtype=dtype)
    ops.gelu_gate_rows(out, t.to(device=device, dtype=dtype),
                       table.to(device=device, dtype=dtype), ids.to(device),
                       layer * d)
    want = O.gelu_tanh(t.double()) * table.double()[ids][:, layer * d:
                                                         (layer + 1) * d]
    close(out, want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_elementwise_output_gate_in_place(device, dtype):
    a, g = rnd(5, 24, seed=1), rnd(5, 40, seed=2, scale=3.0)
    buf = a.clone().to(device=device, dtype=dtype)
    ops.sigmoid_gate_rows(buf, buf, g.to(device=device, dtype=dtype)[:, 8:32])
    close(buf, a.double() * torch.sigmoid(g.double()[:, 8:32]), dtype)


# ---------------------------------------------------------------- routing

def oracle_weights(logits, corr, r, n_always=0):
    T, E = logits.shape[0], r["experts"]
    w = {"x.router": torch.eye(logits.shape[1], dtype=F64)[:E],
         "x.correction": corr.double()}
    dense = torch.zeros(T, E + n_always, dtype=F64)
    for t, chosen in enumerate(O.route(logits.double(), w, "x.", r)):
        for e, wt in chosen:
            dense[t, e] = wt
    dense[:, E:] = torch.sigmoid(logits.double()[:, E:])
    return dense


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,groups,keep,always", [
    (8, 2, 2, 1, 1), (12, 5, 4, 3, 0), (6, 6, 1, 1, 1), (9, 1, 3, 1, 0),
    (16, 3, 2, 1, 1), (70, 3, 10, 2, 0)])
def test_group_limited_sigmoid_routing(device, E, top, groups, keep, always):
    T = 40
    logits = rnd(T, E + always, seed=E, scale=2.0)
    corr = rnd(E, seed=top, scale=0.3)
    r = {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}
    want = oracle_weights(logits, corr, r, always)
    got = torch.empty(T, E + always, device=device)
    ops.grouped_sigmoid_route(got, logits.to(device), corr.to(device), E, top,
                              groups, keep, 2)
    assert torch.allclose(got.double().cpu(), want, atol=1e-6)
    assert int((got[:, :E] > 0).sum()) == T * top


@pytest.mark.parametrize("device", DEVICES)
def test_routing_group_sum_of_two_and_negative_choice_scores(device):
    """Group 0 holds the single best expert, group 1 the better PAIR: the
    pair's group wins. With all choice scores negative (large negative
    correction) the experts of the dropped group must not come back as
    'zero beats negative'; the weights are the uncorrected scores."""
    z = torch.tensor([[4.0, -6.0, -6.0, 1.0, 1.2, -6.0]])
    corr = torch.zeros(6)
    got = torch.empty(1, 6, device=device)
    ops.grouped_sigmoid_route(got, z.to(device), corr.to(device), 6, 2, 2, 1,
                              2)
    s = torch.sigmoid(z)
    assert got[0, :3].abs().max() == 0
    assert torch.allclose(got[0, 3:5].cpu(), s[0, 3:5], atol=1e-6)
    corr = torch.full((6,), -5.0)
    corr[4] = -4.0
    ops.grouped_sigmoid_route(got, z.to(device), corr.to(device), 6, 2, 2, 1,
                              2)
    want = oracle_weights(z, corr, {"experts": 6, "top": 2,
                                    "groups": {"count": 2, "keep": 1}})
    assert torch.allclose(got.double().cpu(), want, atol=1e-6)
    assert int((got > 0).sum()) == 2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,Fe,Ft", [(4, 8, 12), (3, 5, 0), (0, 4, 7),
                                     (1, 16, 0)])
def test_experts_with_output_weight_and_tail_expert(device, dtype, E, Fe, Ft):
    """Stacked activation + stacked down projection == weighted sum of the
    chosen experts' outputs plus the gated shared expert."""
    T, W = 6, 10
    gu = rnd(T, 2 * E * Fe + 2 * Ft + 8, seed=1, scale=1.5)
    weight = rnd(T, E + 1, seed=2).abs()
    weight[:, :E][rnd(T, E, seed=3) > 0.3] = 0.0
    down = rnd(W, E * Fe + Ft, seed=4)
    act = torch.empty(T, E * Fe + Ft, device=device, dtype=dtype)
    ops.routed_silu_glu(
        act, gu.to(device=device, dtype=dtype)[:, :2 * E * Fe + 2 * Ft],
        weight.to(device), E, Fe, Ft)
    got = act.double().cpu() @ down.double().T
    g = gu.double()
    want = torch.zeros(T, W, dtype=F64)
    forms = [(e, e * 2 * Fe, Fe, e * Fe) for e in range(E)]
    if Ft:
        forms.append((E, E * 2 * Fe, Ft, E * Fe))
    for e, c0, f, o0 in forms:
        a = g[:, c0:c0 + f]
        y = a * torch.sigmoid(a) * g[:, c0 + f:c0 + 2 * f]
        want += weight.double()[:, e:e + 1] * (y @ down.double()[:, o0:o0 + f].T)
    close(got, want, dtype)
    if E:
        dead = (weight[:, :E] == 0).repeat_interleave(Fe, dim=1)
        assert float(act[:, :E * Fe].float().cpu()[dead].abs().max()) == 0.0


# ------------------------------------------------------- window attention

def paged(k, v, page, device, dtype, seed=0):
    """Scatter [n, G, D] keys / values into shuffled pages of a pool."""
    n, G, D = k.shape
    n_pages = -(-n // page)
    perm = (torch.randperm(n_pages + 3, generator=torch.Generator()
                           .manual_seed(seed))[:n_pages] + 1)
    kc = torch.zeros(n_pages + 5, G, page, D, dtype=dtype)
    vc = torch.zeros(n_pages + 5, G, page, v.shape[2], dtype=dtype)
    for j in range(n):
        kc[perm[j // page], :, j % page] = k[j].to(dtype)
        vc[perm[j // page], :, j % page] = v[j].to(dtype)
    return kc.to(device), vc.to(device), perm.to(torch.int32).view(1, -1).to(
        device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,size,page", [
    (4, 2, 32, 32, 36, 16), (6, 3, 64, 64, 33, 16), (3, 1, 24, 20, 7, 4),
    (8, 1, 32, 16, 1, 8), (2, 2, 64, 128, 200, 16)])
def test_window_attention_with_distance_bias(device, dtype, H, G, D, Dv, size,
                                             page):
    """A planted key dominates one query's softmax; the query just inside
    the window must return that key's value, the query one further must
    not see it — as a prompt portion and as single decoded tokens, with the
    planted key on a page border."""
    n = max(3 * size, 70)
    q, k, v = rnd(n, H, D, seed=1), rnd(n, G, D, seed=2), rnd(n, G, Dv, seed=3)
    r1 = rnd(H, seed=4).abs() + 0.25
    r2 = rnd(H, seed=5).abs() + 0.25
    j_star = page * 2 - 1                       # last row of its page
    i_in = j_star + size - 1                    # still sees j_star
    # strong enough to beat the distance penalty at the window's edge
    boost = (12.0 + float(r1.max()) * math.log1p(float(r2.max()) * size)) \
        / (D ** -0.5)
    for i in (i_in, i_in + 1):
        if i < n:
            q[i] = 0.0
            q[i, :, 0] = 1.0
    k[j_star] = 0.0
    k[j_star, :, 0] = boost
    v[j_star] = 5.0
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    want = O.biased_window_softmax(q.double(), k.double(), v.double(),
                                   D ** -0.5, size, r1.double(), r2.double())
    assert float(want[i_in].min()) > 4.0        # the beacon is seen ...
    if size > 1:
        assert float(want[i_in + 1].max()) < 4.0    # ... and then it is gone
    kc, vc, table = paged(k, v, page, device, dtype)
    dist = torch.stack([r1, r2], dim=1).contiguous().to(device)
    i32 = dict(dtype=torch.int32, device=device)
    # a portion that starts mid-window and ends past the edge
    lo, hi = max(0, i_in - 5), min(n, i_in + 4)
    out = torch.empty(hi - lo, H, Dv, device=device, dtype=dtype)
    ops.masked_attention(
        out, q[lo:hi].to(device=device, dtype=dtype), kc, vc, table,
        torch.tensor([hi], **i32), torch.tensor([0], **i32),
        torch.tensor([hi - lo], **i32), D ** -0.5, ops.MASK_WINDOW, size,
        max_qlen=hi - lo, dist_bias=dist)
    close(out, want[lo:hi], dtype, 2e-5)
    # the same positions decoded one by one
    for i in range(lo, hi):
        o1 = torch.empty(1, H, Dv, device=device, dtype=dtype)
        ops.masked_attention(
            o1, q[i:i + 1].to(device=device, dtype=dtype), kc, vc, table,
            torch.tensor([i + 1], **i32), None, None, D ** -0.5,
            ops.MASK_WINDOW, size, dist_bias=dist)
        close(o1[0], want[i], dtype, 2e-5)
    # the whole sequence as one prompt, first tokens included, with a gate
    # per output coordinate (columns of a wider projection)
    gate = rnd(n, H * Dv + 8, seed=6, scale=2.0).to(dtype)
    gated = want * torch.sigmoid(gate[:, :H * Dv].double()).view(n, H, Dv)
    out = torch.empty(n, H, Dv, device=device, dtype=dtype)
    ops.masked_attention(
        out, q.to(device=device, dtype=dtype), kc, vc, table,
        torch.tensor([n], **i32), torch.tensor([0], **i32),
        torch.tensor([n], **i32), D ** -0.5, ops.MASK_WINDOW, size,
        head_gate=gate.to(device)[:, :H * Dv], max_qlen=n, dist_bias=dist)
    close(out, gated, dtype, 2e-5)
    i = n - 1                                   # and decoded
    o1 = torch.empty(1, H, Dv, device=device, dtype=dtype)
    ops.masked_attention(
        o1, q[i:i + 1].to(device=device, dtype=dtype), kc, vc, table,
        torch.tensor([n], **i32), None, None, D ** -0.5, ops.MASK_WINDOW,
        size, head_gate=gate.to(device)[i:i + 1, :H * Dv], dist_bias=dist)
    close(o1[0], gated[i], dtype, 2e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_plain_kv_append_into_pages(device):
    T, G, D, Dv, PS = 7, 2, 6, 10, 4
    k, v = rnd(T, G * D + 5, seed=1), rnd(T, G * Dv, seed=2)
    kc = torch.zeros(5, G, PS, D, device=device)
    vc = torch.zeros(5, G, PS, Dv, device=device)
    slots = torch.tensor([4, 5, 6, 7, 16, -1, 3], device=device)
    ops.head_kv_append(k.to(device)[:, :G * D].view(T, G, D),
                  v.to(device).view(T, G, Dv), kc, vc, slots)
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        assert torch.equal(kc[s // PS, :, s % PS].cpu(),
                           k[t, :G * D].view(G, D))
        assert torch.equal(vc[s // PS, :, s % PS].cpu(), v[t].view(G, Dv))
    assert float(kc.abs().sum()) == float(k[[0, 1, 2, 3, 4, 6], :G * D].abs().sum())


# ------------------------------------------------------- latent attention

@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mixer,far", [
    (O.latent_mixer(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64,
                    scaling={"factor": 4.0, "original": 64, "fast": 8.0,
                             "slow": 1.0}), 300),
    (O.latent_mixer(heads=3, dim=8, rot_dim=6, vdim=20, kv_rank=10,
                    base=50.0), 40),
    (O.latent_mixer(heads=1, dim=16, rot_dim=2, vdim=8, kv_rank=96), 70)])
def test_latent_attention_module_over_paged_pool(device, dtype, mixer, far):
    """The serving module (absorbed key map, re-ordered rotary pairs, pool
    row = latent | rotated key) against the oracle's expanded keys and
    values: a prompt portion, a second portion, then decoded tokens — far
    beyond the first pages, positions large enough for YaRN to matter."""
    from agentainer_amd.models.llama import AttnMetadata
    from agentainer_amd.models.sipelorn import (RotaryLatentAttention,
                                                config_from_dict)

    W, eps, page = 48, 1e-5, 8
    cfg = O.make_config([(mixer, None)], width=W, eps=eps)
    w = O.random_weights(cfg, seed=3)
    mc = config_from_dict(cfg).layers[0].latent
    n = far + 12
    h = rnd(n, W, seed=7)
    want = O.latent_attention(h.double(), {k: t.double() for k, t in w.items()},
                              "l0.mix.", mixer["mixer"], eps)
    mod = RotaryLatentAttention(W, mc, eps, dtype, extra_rows=0).to(device)
    mod.load(lambda name: w["l0.mix." + name].to(device=device, dtype=dtype))
    n_pages = -(-n // page)
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(1)) + 1
    pool = torch.zeros(n_pages + 2, page, mc.padded_rank, device=device,
                       dtype=dtype)
    table = perm.to(torch.int32).view(1, -1).to(device)
    got, at = [], 0
    for step in [far - 3, 9] + [1] * 6:
        pos = torch.arange(at, at + step)
        slots = (perm[pos // page] * page + pos % page).to(device)
        i32 = dict(dtype=torch.int32, device=device)
        md = AttnMetadata(
            page_table=table, seq_lens=torch.tensor([at + step], **i32),
            slot_mapping=slots, positions=pos.to(**i32), is_prefill=step > 1,
            query_starts=torch.tensor([0], **i32),
            query_lens=torch.tensor([step], **i32), max_qlen=step)
        y, _ = mod(h[at:at + step].to(device=device, dtype=dtype), pool, md)
        got.append(y.float().cpu())
        at += step
    got = torch.cat(got)
    tol = 5e-5 if dtype == torch.float32 else 4e-2
    err = float((got.double() - want).abs().max() / want.abs().max())
    assert err < tol, err


@pytest.mark.parametrize("device", DEVICES)
def test_rotary_pair_order_and_yarn_table(device):
    """Interleaved pairs re-ordered to (i, i + half) and rotated with the
    framework's table give the oracle's interleaved rotation, re-ordered."""
    rot = {"base": 300.0, "dims": 8,
           "scaling": {"factor": 3.0, "original": 40, "fast": 6.0,
                       "slow": 0.7}}
    v = rnd(25, 10, seed=1).double()               # 2 coordinates pass
    want = O.rotate_interleaved(v, rot)
    order = list(range(0, 8, 2)) + list(range(1, 8, 2)) + [8, 9]
    freqs, amp = ops.rotary_frequencies(8, 300.0, rot["scaling"],
                                        device=device)
    f_want, a_want = O.yarn_frequencies(8, 300.0, rot["scaling"])
    assert abs(amp - a_want) < 1e-12
    assert torch.allclose(freqs.double().cpu(), torch.tensor(f_want, dtype=F64),
                          rtol=1e-6)
    pos = torch.arange(25, dtype=torch.int32, device=device)
    cs = ops.rotary_table(pos, freqs, amp)
    # rows: one query head of size 10 at offset 0, latent rank 3, key part 10
    proj = torch.zeros(25, 24, device=device)
    proj[:, :10] = v[:, order].float().to(device)
    proj[:, 10:13] = 1.0
    proj[:, 13:23] = v[:, order].float().to(device)
    pool = torch.zeros(8, 4, 32, device=device)
    slots = torch.arange(25, device=device) + 4
    ops.latent_rotary_append(proj, 1, 10, 0, 10, 3, 10, torch.ones(
        3, device=device), 0.0, cs, pool, slots)
    assert torch.allclose(proj[:, :10].double().cpu(), want[:, order],
                          atol=1e-5)
    rows = pool.view(-1, 32)[4:29].double().cpu()
    assert torch.allclose(rows[:, :3], torch.ones(25, 3, dtype=F64), atol=1e-6)
    assert torch.allclose(rows[:, 3:13], want[:, order], atol=1e-5)
    assert float(rows[:, 13:].abs().max()) == 0.0
