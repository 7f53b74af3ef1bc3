"""Pekarax through the serving engine (per-sequence state slots + paged
K/V, varlen + decode paths, scheduler) against the plain float64 oracle.
Every scenario runs on CPU (reference ops) and, marked gpu, on the MI355X
(HIP kernels, captured decode graph). Models are small random ones in
float32 so that a lost state, a tail that is one token off, a slot that was
not started from zero or a dropped identity expert shows far above the
tolerance."""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import pekarax_oracle as O  # noqa: E402

from agentainer_amd.config import load_config  # noqa: E402
from agentainer_amd.engine.llm import GenRequest, LLMEngine  # noqa: E402
from agentainer_amd.store import Store  # noqa: E402

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def make_instance(tmp_path, cfg, weights, device, dtype="float32", page=4,
                  pool_tokens=512, slots=4, **extra):
    path = str(tmp_path / "ckpt")
    O.save_checkpoint(path, cfg, weights)
    conf = load_config(path="/nonexistent.yaml", env={})
    conf.data["store"]["path"] = str(tmp_path / "root")
    e = conf.data["engine"]
    e.update(sync_mode=True, async_decode=False, prefill_stream=False,
             prefix_sharing=False, dtype=dtype, kv_page_size=page,
             kv_pool_tokens=pool_tokens,
             max_seqs=slots + (1 if device == "cuda" else 0),
             max_pages_per_seq=-(-pool_tokens // page),
             max_batch_tokens=1 << 20)
    e.update(extra)
    store = Store(str(tmp_path / "root" / "state"), sync="never")
    if device == "cuda":
        torch.backends.cuda.matmul.allow_tf32 = False
    eng = LLMEngine(store, conf, device=device,
                    state_root=str(tmp_path / "root"))
    return eng, eng._get_instance(path), path


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(3, cfg["vocab"], (n,), generator=g).tolist()


def replay(inst, reqs, schedule):
    """schedule: list of steps, each [(request id, n tokens)]. Every
    position's logits are collected. Returns {id: [T, V] tensor}."""
    at = {i: 0 for i in reqs}
    got = {i: [] for i in reqs}
    for step in schedule:
        entries, want = [], []
        for i, n in step:
            entries.append((i, reqs[i][at[i]:at[i] + n]))
            want.append(list(range(n)))
            at[i] += n
        lg = inst.forward_step(entries, want).float().cpu()
        k = 0
        for i, n in step:
            got[i].append(lg[k:k + n])
            k += n
        for i, _n in step:
            if at[i] == len(reqs[i]):
                inst.release(i)
    return {i: torch.cat(v) for i, v in got.items()}


def check(got, cfg, weights, reqs, tol=3e-4):
    for i, toks in reqs.items():
        want = O.forward(cfg, weights, toks)
        assert got[i].shape == want.shape
        err = float((got[i] - want).abs().max() / want.abs().max())
        assert err < tol, f"request {i}: relative error {err:.3e}"


def cuts(total, sizes):
    out, k = [], 0
    while total > 0:
        n = min(sizes[k % len(sizes)], total)
        out.append(n)
        total -= n
        k += 1
    return out


def small_config(order="dpg", **kw):
    """order: d = channel_delta, p = parallel, g = gla."""
    mk = {"d": O.delta_layer, "p": O.parallel_layer, "g": O.gla_layer}
    return O.make_config([mk[c]() for c in order], **kw)


@pytest.mark.parametrize("device", DEVICES)
def test_layers_match_oracle_residual_trace(tmp_path, device):
    """Layer by layer: the fp32 residual after every layer."""
    cfg = small_config(order="dpgd", no_ff=(2,))
    w = O.random_weights(cfg, seed=1)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    toks = tokens_for(cfg, 19, 1)
    trace = []
    want = O.forward(cfg, w, toks, trace)
    inst.model.residual_trace = []
    got = inst.forward_step([("a", toks)], [list(range(19))]).float().cpu()
    layers = inst.model.residual_trace
    inst.model.residual_trace = None
    assert len(layers) == len(trace) == 4
    for k, (a, b) in enumerate(zip(layers, trace)):
        # engine rows may carry bucket padding past the real tokens
        err = float((a[:19].cpu() - b).abs().max() / b.abs().max())
        assert err < 1e-4, f"layer {k}: {err:.3e}"
    assert float((got - want).abs().max() / want.abs().max()) < 3e-4


@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token_decode(tmp_path, device):
    """Whole prompt in one step == one token per step from the first token
    on (decode path: memories and convolution tails carried in the slots)."""
    cfg = small_config()
    w = O.random_weights(cfg, seed=2)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    reqs = {"a": tokens_for(cfg, 30, 2), "b": tokens_for(cfg, 30, 2)}
    got = replay(inst, {"a": reqs["a"]}, [[("a", 30)]])
    got.update(replay(inst, {"b": reqs["b"]}, [[("b", 1)] for _ in range(30)]))
    check(got, cfg, w, reqs)
    assert float((got["a"] - got["b"]).abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [5, 1, 1, 2], [13, 2]])
def test_portions_of_several_sizes(tmp_path, device, sizes):
    """Portions cut mid-page and shorter than the convolutions' reach
    (taps 4 and 3, portions of 1 and 2 tokens: the tail is shifted, not
    replaced), then a decoded tail."""
    cfg = small_config()
    w = O.random_weights(cfg, seed=3)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    toks = tokens_for(cfg, 41, 3)
    sched = [[("a", n)] for n in cuts(33, sizes)] + [[("a", 1)]] * 8
    check(replay(inst, {"a": toks}, sched), cfg, w, {"a": toks})


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_reuse_of_pages_and_slots(tmp_path, device):
    """Unequal requests side by side — portions beside single tokens — in
    a pool too small for all of them at once: pages and state slots of
    finished requests go to the next ones, which must start from zero
    state although the slot still holds the last owner's memory."""
    cfg = small_config(order="pdg")
    w = O.random_weights(cfg, seed=4)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4,
                                 pool_tokens=112, slots=4)
    reqs = {i: tokens_for(cfg, n, 10 + k) for k, (i, n) in enumerate(
        [("a", 40), ("b", 17), ("c", 3), ("d", 28), ("e", 36)])}
    sched = [
        [("a", 16), ("b", 9)],
        [("a", 16), ("b", 1), ("c", 2)],
        [("a", 1), ("b", 1), ("c", 1)],             # pure decode batch
        [("a", 1), ("b", 6), ("d", 2)],             # c's slot reused by d
        [("a", 6), ("d", 26)],                      # a, b, d finish
        [("e", 30)],                                # reuses pages and a slot
        [("e", 1)], [("e", 1)], [("e", 4)],
    ]
    free0 = inst.kvm.free_pages
    got = replay(inst, reqs, sched)
    check(got, cfg, w, reqs)
    assert inst.kvm.free_pages == free0          # everything given back
    assert len(inst.kvm._free_slots) == 4
    # each request alone gives the same logits as inside the batches
    for i in ("b", "d"):
        alone = replay(inst, {i: reqs[i]}, [[(i, len(reqs[i]))]])
        assert float((alone[i] - got[i]).abs().max()) < 1e-3


@pytest.mark.parametrize("device", DEVICES)
def test_long_sequence_page_borders_long_decode(tmp_path, device):
    """150 tokens: the attention reads keys many pages back, the memories
    accumulate over the whole sequence, half of it decoded token by
    token."""
    cfg = small_config(order="pg")
    w = O.random_weights(cfg, seed=5)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=8,
                                 pool_tokens=256)
    toks = tokens_for(cfg, 150, 5)
    sched = [[("a", 70)], [("a", 9)]] + [[("a", 1)]] * 71
    check(replay(inst, {"a": toks}, sched), cfg, w, {"a": toks})


@pytest.mark.parametrize("device", DEVICES)
def test_state_is_really_carried(tmp_path, device):
    """Dropping the first tokens changes the logits long after every
    convolution has forgotten them: the memories carry them."""
    cfg = small_config(order="gd", no_ff=(0, 1))
    w = O.random_weights(cfg, seed=12)
    toks = tokens_for(cfg, 24, 12)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device)
    got = replay(inst, {"a": toks}, [[("a", 9)]] + [[("a", 1)]] * 15)
    check(got, cfg, w, {"a": toks})
    short = O.forward(cfg, w, toks[6:])
    assert float((got["a"][-1] - short[-1]).abs().max()) > 1e-2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layers,kw", [
    # values that a usual model makes equal (or 1) all differ here
    ([O.delta_layer(heads=6, kv_heads=2, dim=12, vdim=20, conv=2, rank=3,
                    grank=7),
      O.parallel_layer(heads=3, kv_heads=1, dim=24, vdim=8, conv=5,
                       rot_dims=6, base=77.0, scale=1.3, left_scale=0.4,
                       right_scale=1.0, m_heads=3, m_dim=4, m_vdim=28,
                       cap=3.0),
      O.gla_layer(heads=3, dim=20, vdim=4, tau=1.0, rank=9)],
     dict(width=48, alpha=1.0, no_ff=(0,),
          mlp=O.moe(experts=5, identity=0, top=1, ff=12, limit=0.7, groups=1,
                    keep=1, scale=1.0))),
    ([O.gla_layer(heads=1, dim=40, vdim=36, tau=30.0, rank=1),
      O.delta_layer(heads=1, kv_heads=1, dim=36, vdim=40, conv=1, rank=2,
                    grank=1),
      O.parallel_layer(heads=2, kv_heads=2, dim=8, vdim=8, conv=1,
                       rot_dims=8, m_heads=1, m_dim=72, m_vdim=8, cap=20.0)],
     dict(width=32, alpha=3.5, eps=1e-3,
          mlp=O.moe(experts=3, identity=5, top=4, ff=6, limit=9.0, groups=8,
                    keep=5, scale=0.5))),
    ([O.parallel_layer(heads=8, kv_heads=1, dim=4, vdim=12, conv=4,
                       rot_dims=2, m_heads=4, m_dim=12, m_vdim=4)] * 2,
     dict(width=64, alpha=0.5,
          mlp=O.moe(experts=12, identity=4, top=6, ff=20, limit=2.0,
                    groups=4, keep=4, scale=3.0))),
])
def test_other_sizes(tmp_path, device, layers, kw):
    cfg = O.make_config(layers, vocab=300, **kw)
    w = O.random_weights(cfg, seed=6)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    reqs = {"a": tokens_for(cfg, 23, 6), "b": tokens_for(cfg, 9, 7)}
    sched = [[("a", 11), ("b", 2)], [("a", 2), ("b", 1)],
             [("a", 1), ("b", 1)], [("a", 9), ("b", 5)]]
    check(replay(inst, reqs, sched), cfg, w, reqs)


@pytest.mark.parametrize("device", DEVICES)
def test_checkpoint_offload_restore(tmp_path, device):
    """A sequence's pages AND its per-slot state survive offload to host
    and restore into other pages and another slot."""
    cfg = small_config()
    w = O.random_weights(cfg, seed=8)
    eng, inst, _ = make_instance(tmp_path, cfg, w, device, page=4)
    toks = tokens_for(cfg, 30, 8)
    inst.forward_step([("pre", toks[:5])], [[0]])  # takes the first slot
    a = inst.forward_step([("a", toks[:21])], [[20]]).float().cpu()
    ck = inst.kvm.offload("a", free=True)
    assert not inst.kvm.has_seq("a") and ck.state is not None
    inst.release("pre")
    inst.forward_step([("x", toks[:9])], [[0]])    # dirty pages and slots
    inst.forward_step([("y", toks[3:9])], [[0]])
    inst.kvm.restore("a", ck)
    b = inst.forward_step([("a", toks[21:])], [list(range(9))]).float().cpu()
    want = O.forward(cfg, w, toks)
    assert float((a[0] - want[20]).abs().max() / want.abs().max()) < 3e-4
    assert float((b - want[21:]).abs().max() / want.abs().max()) < 3e-4


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(tmp_path, device):
    """Deploy the checkpoint directory as an agent and generate greedily
    through the engine's own scheduler (chunked admission: the step token
    budget is smaller than the prompt), against oracle argmax decoding."""
    from agentainer_amd.registry import Manager

    cfg = small_config(vocab=300)
    w = O.random_weights(cfg, seed=9)
    eng, inst0, path = make_instance(tmp_path, cfg, w, device, page=4,
                                     pool_tokens=400, slots=8,
                                     max_batch_tokens=8)
    conf = load_config(path="/nonexistent.yaml", env={})
    manager = Manager(eng.store, eng, conf)
    agents = [manager.deploy(name=f"g{k}", model=path,
                             sampling={"max_tokens": 12}) for k in range(2)]
    inst = eng._instances[path]
    assert inst.stateful and not inst.async_decode and not inst.prefix_sharing
    reqs = []
    for k, ag in enumerate(agents):
        manager.start(ag.id)
        prompt = tokens_for(cfg, 21 + 6 * k, 20 + k)
        r = GenRequest(agent_id=ag.id, prompt_tokens=prompt, max_new=12,
                       temperature=0.0, top_p=1.0, seed=0)
        b = inst.binding(ag.id)
        with inst._lock:
            b.queue.put(r)
            inst._pump_agent(b)
        reqs.append(r)
    for _ in range(200):
        inst.step()
        if all(r.done.is_set() for r in reqs):
            break
    for r in reqs:
        assert r.done.is_set() and not r.error, r.error
        # the sampler reads bf16 logits: every generated token must be the
        # oracle's argmax up to that rounding, given the tokens before it
        seq = list(r.prompt_tokens)
        assert 1 <= len(r.generated) <= 12
        for k, t in enumerate(r.generated):
            lg = O.forward(cfg, w, seq)[-1]
            assert float(lg[t]) >= float(lg.max()) - 0.01 * float(lg.abs().max()), (k, t)
            seq.append(t)
        assert (len(r.generated) == 12
                or r.generated[-1] == inst.tokenizer.eos_id)


def test_named_random_init_model_is_registered(tmp_path):
    """`deploy tiny-pekarax` resolves through the family registry."""
    from agentainer_amd.models import registry

    assert registry.family_of("tiny-pekarax") == "Pekarax"
    assert registry.build_target("tiny-pekarax") == "masked+recurrent"
    conf = load_config(path="/nonexistent.yaml", env={})
    conf.data["store"]["path"] = str(tmp_path / "root")
    conf.data["engine"].update(sync_mode=True, kv_pool_tokens=128,
                               max_seqs=8)
    eng = LLMEngine(Store(str(tmp_path / "root" / "state"), sync="never"),
                    conf, device="cpu", state_root=str(tmp_path / "root"))
    eng.validate_model("tiny-pekarax")
    inst = eng._get_instance("tiny-pekarax")
    lg = inst.forward_step([("a", [5, 6, 7, 8])], [[3]])
    assert lg.shape == (1, 512) and bool(torch.isfinite(lg).all())


@pytest.mark.gpu
@pytest.mark.parametrize("layers,kw", [
    ([O.delta_layer(heads=4, kv_heads=2, dim=64, vdim=32, conv=4, rank=8,
                    grank=8),
      O.parallel_layer(heads=8, kv_heads=2, dim=64, vdim=64, conv=3,
                       rot_dims=32, scale=0.1, m_heads=2, m_dim=32,
                       m_vdim=64, cap=11.0),
      O.gla_layer(heads=2, dim=128, vdim=64, tau=12.0, rank=8)],
     dict(width=128, mlp=O.moe(experts=8, identity=2, top=3, ff=64,
                               limit=1.8, groups=2, keep=1))),
    # head sizes the attention tile kernel does not take -> row kernel
    ([O.parallel_layer(heads=3, kv_heads=1, dim=24, vdim=20, conv=2,
                       rot_dims=8, m_heads=3, m_dim=40, m_vdim=12),
      O.delta_layer(heads=2, kv_heads=1, dim=20, vdim=36, conv=3)],
     dict(width=72))])
def test_bf16_serving_path_close_to_oracle(tmp_path, layers, kw):
    """bf16 serving precision (captured decode graph): logits stay within
    bf16 rounding of the oracle, and graph replays keep agreeing with it
    step after step."""
    cfg = O.make_config(layers, vocab=300, **kw)
    w = O.random_weights(cfg, seed=11)
    for k in w:
        # peaky routers: near-ties (which bf16 rounding may flip) then sit
        # among experts of small weight
        if k.endswith("mlp.router"):
            w[k] = (w[k] * 4).bfloat16().float()
    eng, inst, _ = make_instance(tmp_path, cfg, w, "cuda", dtype="bfloat16",
                                 page=16, pool_tokens=512)
    reqs = {"a": tokens_for(cfg, 120, 1), "b": tokens_for(cfg, 75, 2)}
    sched = ([[("a", 64), ("b", 3)], [("a", 30), ("b", 50)]]
             + [[("a", 1), ("b", 1)]] * 22 + [[("a", 4)]])
    got = replay(inst, reqs, sched)
    assert inst.use_graph and inst._graphs, "decode graph was not captured"
    for i, toks in reqs.items():
        want = O.forward(cfg, w, toks)
        d = got[i] - want
        d = d - d.mean(-1, keepdim=True)
        rel = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
        # a position where two expert groups score within bf16 rounding of
        # each other may take the other group; its neighbours do not
        assert int((rel > 0.08).sum()) <= 0.05 * rel.numel(), rel
        assert float(rel.median()) < 0.03, float(rel.median())
