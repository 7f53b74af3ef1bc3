"""Every HIP kernel of the recurrent extension against the fp32 reference
op of the same name (GPU only)."""

import pytest
import torch

from agentainer_amd import ops
from agentainer_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _need():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    assert ops.recurrent_available(), "recurrent HIP extension not built"


def _step(lens_new, lens_before, decode=False):
    """seq_lens, query_starts, query_lens for portions of the given sizes."""
    B = len(lens_new)
    seq = torch.tensor([a + b for a, b in zip(lens_before, lens_new)],
                       dtype=torch.int32)
    if decode:
        return seq, None, None
    st, acc = [], 0
    for n in lens_new:
        st.append(acc)
        acc += n
    return (seq, torch.tensor(st, dtype=torch.int32),
            torch.tensor(lens_new, dtype=torch.int32))


def _dev(t):
    return None if t is None else t.to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [96, 130, 1024])
def test_postln_rmsnorm_residual(dtype, W):
    _need()
    g = torch.Generator().manual_seed(W)
    T = 37
    x = torch.randn(T, W, generator=g)
    y = torch.randn(T, W + 8, generator=g).to(dtype)[:, :W]
    y2 = torch.randn(T, W, generator=g).to(dtype)
    ra = torch.rand(T, generator=g)
    w = 1 + 0.1 * torch.randn(W, generator=g)
    for case in range(4):
        xr, xg = x.clone(), x.clone().to(DEV)
        hr = torch.empty(T, W, dtype=dtype)
        hg = torch.empty(T, W, dtype=dtype, device=DEV)
        yy = None if case == 3 else (y.float() if case == 2 else y)
        kw = dict(alpha=1.7 if case != 3 else 1.0, y_scale=0.9,
                  y2=y2 if case == 1 else None, y2_scale=0.6,
                  row_add=ra if case == 2 else None)
        ref.postln_rmsnorm_residual(xr, yy, kw["y_scale"], kw["y2"],
                                    kw["y2_scale"], kw["alpha"],
                                    kw["row_add"], w, 1e-5, hr)
        ops.postln_rmsnorm_residual(
            xg, _dev(yy), w.to(DEV), 1e-5, hg, alpha=kw["alpha"],
            y_scale=kw["y_scale"], y2=_dev(kw["y2"]), y2_scale=kw["y2_scale"],
            row_add=_dev(kw["row_add"]))
        torch.testing.assert_close(xg.cpu(), xr, rtol=2e-5, atol=2e-5)
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        torch.testing.assert_close(hg.cpu().float(), hr.float(), rtol=tol,
                                   atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4])
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("D,extra", [(24, 100), (25, 7), (128, 256), (64, 40)])
def test_short_conv_state(dtype, taps, decode, D, extra):
    """Sizes that take the four-channels-per-lane kernel (8, 16, 32 lanes
    per head) and sizes that do not."""
    _need()
    g = torch.Generator().manual_seed(taps)
    heads = 3
    C = 2 * heads * D + extra
    new = [1, 1, 1] if decode else [5, 1, 2, 9]
    before = [0, 3, 7] if decode else [0, 4, 1, 0]
    seq, qs, ql = _step(new, before, decode)
    T, B = sum(new), len(new)
    u = torch.randn(T, C + 8, generator=g).to(dtype)[:, :C]
    w = torch.randn(taps, C, generator=g)
    tail = torch.randn(6, taps - 1, C, generator=g)
    slots = torch.tensor([4, 0, 2, 5][:B], dtype=torch.long)
    for out_dt, kw in ((torch.float32, dict(silu=True,
                                            norm_channels=2 * heads * D,
                                            head_dim=D,
                                            lead_channels=heads * D,
                                            lead_scale=0.3)),
                       (dtype, dict())):
        tr, tg = tail.clone(), tail.clone().to(DEV)
        outr = torch.empty(T, C, dtype=out_dt)
        outg = torch.empty(T, C, dtype=out_dt, device=DEV)
        ref.short_conv_state(outr, u, w, tr, slots, seq, qs, ql,
                             kw.get("silu", False), kw.get("norm_channels", 0),
                             kw.get("head_dim", 1), kw.get("lead_channels", 0),
                             kw.get("lead_scale", 1.0), 1e-6)
        ops.short_conv_state(outg, u.to(DEV), w.to(DEV), tg, slots.to(DEV),
                             seq.to(DEV), _dev(qs), _dev(ql), **kw)
        tol = 1e-5 if out_dt == torch.float32 else 2e-2
        torch.testing.assert_close(outg.cpu().float(), outr.float(), rtol=tol,
                                   atol=tol)
        torch.testing.assert_close(tg.cpu(), tr, rtol=0, atol=0)


@pytest.mark.parametrize("kind", [ops.SCAN_GLA, ops.SCAN_DELTA,
                                  ops.SCAN_MLSTM])
@pytest.mark.parametrize("D,Dv,H,G", [(32, 48, 4, 2), (48, 40, 3, 3),
                                      (24, 16, 2, 1), (128, 128, 2, 2),
                                      (256, 64, 1, 1), (6, 5, 2, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_memory_scan(kind, D, Dv, H, G, dtype):
    _need()
    if kind != ops.SCAN_DELTA and G != H:
        G = H
    g = torch.Generator().manual_seed(D * 7 + Dv)
    for decode in (False, True):
        new = [1, 1, 1] if decode else [19, 1, 8, 2]
        before = [5, 0, 40] if decode else [0, 3, 11, 0]
        seq, qs, ql = _step(new, before, decode)
        T, B = sum(new), len(new)
        n_slots = 6
        slots = torch.tensor([3, 1, 5, 0][:B], dtype=torch.long)
        q = torch.randn(T, G, D, generator=g).to(dtype)
        k = (torch.randn(T, G, D, generator=g) / D ** 0.5).to(dtype)
        v = torch.randn(T, H, Dv, generator=g).to(dtype)
        if kind == ops.SCAN_MLSTM:
            gate = torch.randn(T, 2 * H, generator=g) * 3
            bias = torch.randn(2 * H, generator=g)
        else:
            gate = torch.randn(T, H * D, generator=g) * 2
            bias = torch.randn(H * D, generator=g)
        rate = torch.randn(H, generator=g) * 0.5
        beta = torch.randn(T, H + 3, generator=g)[:, :H]
        S = torch.randn(n_slots, H, Dv, D, generator=g)
        n_st = torch.randn(n_slots, H, D, generator=g)
        m_st = torch.randn(n_slots, H, generator=g)
        param = {ops.SCAN_GLA: 0.1, ops.SCAN_DELTA: 0.0,
                 ops.SCAN_MLSTM: 9.0}[kind]
        Sr, nr, mr = S.clone(), n_st.clone(), m_st.clone()
        outr = torch.zeros(T, H, Dv)
        ref.matrix_memory_scan(kind, outr, q, k, v, gate, bias, rate, beta,
                               D ** -0.5, param, Sr, nr, mr, slots, seq, qs,
                               ql)
        Sg, ng, mg = S.to(DEV), n_st.to(DEV), m_st.to(DEV)
        outg = torch.zeros(T, H, Dv, device=DEV)
        ops.matrix_memory_scan(kind, outg, q.to(DEV), k.to(DEV), v.to(DEV),
                               gate.to(DEV), bias.to(DEV), rate.to(DEV),
                               beta.to(DEV), D ** -0.5, param, Sg, ng, mg,
                               slots.to(DEV), seq.to(DEV), _dev(qs), _dev(ql))
        torch.testing.assert_close(outg.cpu(), outr, rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(Sg.cpu(), Sr, rtol=2e-4, atol=2e-4)
        if kind == ops.SCAN_MLSTM:
            torch.testing.assert_close(ng.cpu(), nr, rtol=2e-4, atol=2e-4)
            torch.testing.assert_close(mg.cpu(), mr, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Dv,shared", [(64, True), (40, False), (192, True)])
def test_head_rmsnorm_gate(dtype, Dv, shared):
    _need()
    g = torch.Generator().manual_seed(Dv)
    T, H = 21, 3
    o = torch.randn(T, H, Dv, generator=g)
    w = torch.randn(Dv if shared else H * Dv, generator=g)
    for gate in (torch.randn(T, H * Dv + 8, generator=g).to(dtype)[:, :H * Dv],
                 torch.randn(T, H * Dv, generator=g)):
        for silu in (False, True):
            outr = torch.empty(T, H * Dv, dtype=dtype)
            outg = torch.empty(T, H * Dv, dtype=dtype, device=DEV)
            ref.head_rmsnorm_gate(outr, o, w, gate, 1e-5, silu)
            ops.head_rmsnorm_gate(outg, o.to(DEV), w.to(DEV), gate.to(DEV),
                                  1e-5, silu)
            tol = 1e-5 if dtype == torch.float32 else 2e-2
            torch.testing.assert_close(outg.cpu().float(), outr.float(),
                                       rtol=tol, atol=tol)


@pytest.mark.parametrize("E,top,groups,keep", [(24, 5, 3, 1), (8, 2, 4, 2),
                                               (6, 6, 1, 1), (96, 5, 8, 3),
                                               (130, 3, 1, 1), (12, 1, 12, 1)])
def test_grouped_softmax_route(E, top, groups, keep):
    _need()
    g = torch.Generator().manual_seed(E)
    T = 50
    logits = torch.randn(T, E, generator=g) * 2
    corr = torch.randn(E, generator=g) * 0.2 - 0.1
    for c in (corr, None):
        wr = torch.empty(T, E)
        wg = torch.empty(T, E, device=DEV)
        ref.grouped_softmax_route(wr, logits, c, top, groups, keep, 1.75)
        ops.grouped_softmax_route(wg, logits.to(DEV), _dev(c), top, groups,
                                  keep, 1.75)
        torch.testing.assert_close(wg.cpu(), wr, rtol=1e-5, atol=1e-6)
        assert int((wg != 0).sum(-1).min()) == top


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("F_", [32, 30])
def test_routed_clamped_glu(dtype, F_):
    _need()
    g = torch.Generator().manual_seed(F_)
    T, E, I = 33, 5, 2
    gu = (torch.randn(T, E * 2 * F_, generator=g) * 2).to(dtype)
    weight = torch.rand(T, E + I, generator=g)
    weight[torch.rand(T, E + I, generator=g) < 0.5] = 0
    outr = torch.empty(T, E * F_, dtype=dtype)
    outg = torch.empty(T, E * F_, dtype=dtype, device=DEV)
    ref.routed_clamped_glu(outr, gu, weight, E, 1.5, 1.702)
    ops.routed_clamped_glu(outg, gu.to(DEV), weight.to(DEV), E, 1.5, 1.702)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    torch.testing.assert_close(outg.cpu().float(), outr.float(), rtol=tol,
                               atol=tol)


@pytest.mark.parametrize("kind", [ops.SCAN_GLA, ops.SCAN_DELTA,
                                  ops.SCAN_MLSTM])
@pytest.mark.parametrize("D,Dv,H,B", [(32, 256, 16, 64), (64, 128, 16, 64),
                                      (128, 128, 16, 32), (256, 128, 8, 32)])
def test_matrix_memory_scan_many_columns(kind, D, Dv, H, B):
    """Launches with many (sequence, head, column) triples take the
    variant with the fewest lanes per column; a decode step and a step of
    short portions."""
    _need()
    g = torch.Generator().manual_seed(D)
    for decode in (True, False):
        new = [1] * B if decode else [2] * B
        before = [(3 * i) % 5 for i in range(B)]
        seq, qs, ql = _step(new, before, decode)
        T = sum(new)
        slots = torch.randperm(B + 3, generator=g)[:B]
        q = torch.randn(T, H, D, generator=g)
        k = torch.randn(T, H, D, generator=g) / D ** 0.5
        v = torch.randn(T, H, Dv, generator=g)
        if kind == ops.SCAN_MLSTM:
            gate = torch.randn(T, 2 * H, generator=g) * 3
            bias = torch.randn(2 * H, generator=g)
        else:
            gate = torch.randn(T, H * D, generator=g) * 2
            bias = torch.randn(H * D, generator=g)
        rate = torch.randn(H, generator=g) * 0.5
        beta = torch.randn(T, H, generator=g)
        S = torch.randn(B + 3, H, Dv, D, generator=g)
        n_st = torch.randn(B + 3, H, D, generator=g)
        m_st = torch.randn(B + 3, H, generator=g)
        param = {ops.SCAN_GLA: 0.25, ops.SCAN_DELTA: 0.0,
                 ops.SCAN_MLSTM: 9.0}[kind]
        Sr, nr, mr = S.clone(), n_st.clone(), m_st.clone()
        outr = torch.zeros(T, H, Dv)
        ref.matrix_memory_scan(kind, outr, q, k, v, gate, bias, rate, beta,
                               0.5, param, Sr, nr, mr, slots, seq, qs, ql)
        Sg, ng, mg = S.to(DEV), n_st.to(DEV), m_st.to(DEV)
        outg = torch.zeros(T, H, Dv, device=DEV)
        ops.matrix_memory_scan(kind, outg, q.to(DEV), k.to(DEV), v.to(DEV),
                               gate.to(DEV), bias.to(DEV), rate.to(DEV),
                               beta.to(DEV), 0.5, param, Sg, ng, mg,
                               slots.to(DEV), seq.to(DEV), _dev(qs), _dev(ql))
        torch.testing.assert_close(outg.cpu(), outr, rtol=2e-4, atol=2e-4)
        torch.testing.assert_close(Sg.cpu(), Sr, rtol=2e-4, atol=2e-4)
        if kind == ops.SCAN_MLSTM:
            torch.testing.assert_close(ng.cpu(), nr, rtol=2e-4, atol=2e-4)
