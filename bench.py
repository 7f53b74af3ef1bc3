#!/usr/bin/env python3
"""bench.py — concurrent-agent chat throughput on MI355X.

Measures BASELINE.json's headline metric: concurrent-agent chat req/sec
(+ p50 E2E latency) for N stateful agents sharing one model under the
continuous-batching engine, synthetic prompts, random-init weights, greedy
bf16 decode, WAL + history writes included in the timed region (the full
config-3 serving path).

A STEP is one engine iteration: admit+prefill (token-budgeted) then one
batched decode step for every running sequence. The harness keeps every
agent closed-loop (one outstanding chat request each; a completed request
is immediately replaced), so the decode batch stays at the agent count.

Scaling mode is WEAK data parallelism: each rank (GPU) runs its own engine
replica serving its own `--agents` agents (the reference's replica fan-out
semantics); ranks synchronize only at the timing barriers.
Whole-job value = sum of per-rank completed requests / max elapsed.

Launch (driver contract):
  python bench.py --gpus 1 --steps K --warmup W
  python -m torch.distributed.run --nnodes=1 --nproc-per-node N \
      --master-addr 127.0.0.1 bench.py --gpus N --steps K --warmup W

Tensor-parallel mode (BASELINE config 4, Llama-3-70B TP=8 over xGMI):
  python -m torch.distributed.run --nnodes=1 --nproc-per-node 8 \
      --master-addr 127.0.0.1 bench.py --gpus 8 --tp 8 --steps K --warmup W
Rank 0 schedules ONE engine sharded across all ranks (broadcast step
plans, RCCL all-reduce per sub-layer); value = rank 0's completed
requests / barrier-bounded elapsed.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import tempfile
import time

import torch

from agentainer_amd.config import load_config
from agentainer_amd.engine.llm import OP_BARRIER, GenRequest, LLMEngine
from agentainer_amd.registry import Manager
from agentainer_amd.store import Store
from agentainer_amd.wal import RequestManager


def parse_args():
    return _parser().parse_args()


def _parser():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=300)
    p.add_argument("--warmup", type=int, default=60)
    p.add_argument("--agents", type=int, default=64)
    p.add_argument("--tp", type=int, default=1,
                   help="tensor-parallel degree (= world size); default "
                        "model becomes llama3-70b (config 4)")
    p.add_argument("--model", default=None,
                   help="default: llama3-8b on GPU, tiny-llama on CPU "
                        "(llama3-70b / tiny-llama-tp when --tp > 1)")
    p.add_argument("--prompt-len", type=int, default=256)
    p.add_argument("--gen-len", type=int, default=64)
    p.add_argument("--max-batch-tokens", type=int, default=16384)
    p.add_argument("--expert-fp8", action="store_true",
                   help="fp8 MFMA expert decode GEMMs (Mixtral, config 5)")
    p.add_argument("--kv-fp8", action="store_true",
                   help="OCP e4m3 KV cache (half the KV bytes, 2x agents)")
    p.add_argument("--expert-fp4", action="store_true",
                   help="MXFP4 block-scaled expert GEMMs (quarter bytes)")
    p.add_argument("--dense-quant", default="", choices=["", "fp8", "mxfp4"],
                   help="opt-in quantized dense decode projections (turbo; "
                        "NOT the headline dtype)")
    p.add_argument("--arch-compare", action="store_true",
                   help="instead of the headline workload: prefill and decode "
                        "tokens/s of a checkpoint-defined design (see "
                        "--arch-design) at real-layer sizes beside "
                        "Llama/Mixtral stacks of equal size")
    p.add_argument("--arch-sizes", default=None,
                   help="--arch-compare: which size points to run "
                        "(default: all points of the design)")
    p.add_argument("--arch-design", default="lelitar",
                   choices=["lelitar", "volalorn", "pekarax", "sipelorn"],
                   help="--arch-compare: which design to measure")
    return p


def _arch_points():
    """Size points: (name, Lelitar config, reference model config, class).
    A few layers each — throughput per layer is what is compared."""
    from agentainer_amd.models.lelitar import (FeedForwardConfig,
                                               LatentMixerConfig,
                                               LelitarConfig,
                                               LelitarLayerConfig)
    from agentainer_amd.models.llama import LlamaConfig
    from agentainer_amd.models.mixtral import MixtralConfig

    def lel(name, width, heads, q_rank, kv_rank, window, ff, n, moe=None):
        mlp = (FeedForwardConfig("moe", ff, experts=moe[0], top=moe[1])
               if moe else FeedForwardConfig("dense", ff))
        mixer = LatentMixerConfig(heads=heads, dim=128, vdim=128,
                                  q_rank=q_rank, kv_rank=kv_rank,
                                  window=window, scale=128 ** -0.5)
        return LelitarConfig(name=name, vocab_size=32000, hidden_size=width,
                             layers=[LelitarLayerConfig(mixer, mlp)
                                     for _ in range(n)],
                             norm_eps=1e-6, norm_groups=2, residual_mult=0.5)

    pts = {
        "s": ("w2048-ff8192", lel("lelitar-s", 2048, 16, 768, 256, 1024,
                                  8192, 4),
              LlamaConfig(name="llama-s", vocab_size=32000, hidden_size=2048,
                          n_layers=4, n_heads=16, n_kv_heads=4,
                          intermediate_size=8192, tie_embeddings=False), None),
        "l": ("w4096-ff14336", lel("lelitar-l", 4096, 32, 1536, 512, 4096,
                                   14336, 4),
              LlamaConfig(name="llama-l", vocab_size=32000, hidden_size=4096,
                          n_layers=4, n_heads=32, n_kv_heads=8,
                          intermediate_size=14336, tie_embeddings=False),
              None),
        "moe": ("w2048-8x4096-top2", lel("lelitar-moe", 2048, 16, 768, 256,
                                         1024, 4096, 4, moe=(8, 2)),
                MixtralConfig(name="mixtral-s", vocab_size=32000,
                              hidden_size=2048, n_layers=4, n_heads=16,
                              n_kv_heads=4, intermediate_size=4096,
                              n_experts=8, top_k=2, tie_embeddings=False),
                "mixtral"),
    }
    return pts


def _volalorn_points():
    """Volalorn size points beside Llama stacks of equal width, head counts
    and ff: layers alternate the sigmoid/chunk mixer (YaRN rotary on half
    the head) and the softmax/window mixer (8 kept first tokens). Masks are
    sized so that a decode step at the benchmark's context reads about as
    many keys as the Llama stack does."""
    from agentainer_amd import ops
    from agentainer_amd.models.llama import LlamaConfig
    from agentainer_amd.models.volalorn import (MaskedAttentionConfig,
                                                PolyFeedForwardConfig,
                                                VolalornConfig,
                                                VolalornLayerConfig)

    def vol(name, width, heads, kv, chunk, window, ff, n):
        sig = MaskedAttentionConfig(
            heads=heads, kv_heads=kv, dim=128, vdim=128, scale=128 ** -0.5,
            mask_kind=ops.MASK_CHUNK, mask_size=chunk, rot_dims=64,
            rot_base=500000.0, rot_scaling={"factor": 4.0, "original": 8192,
                                            "fast": 16.0, "slow": 2.0},
            softcap=30.0, sigmoid_weights=True, key_bias=True, head_gate=True)
        soft = MaskedAttentionConfig(
            heads=heads, kv_heads=kv, dim=128, vdim=128, scale=128 ** -0.5,
            mask_kind=ops.MASK_WINDOW, mask_size=window, keep_first=8,
            rot_dims=128, rot_base=500000.0, qkv_bias=True, norm_first=True)
        layers = [VolalornLayerConfig(
            "attention" if i % 2 == 0 else "attention_2",
            sig if i % 2 == 0 else soft, PolyFeedForwardConfig(ff))
            for i in range(n)]
        return VolalornConfig(name=name, vocab_size=32000, hidden_size=width,
                              layers=layers, norm_eps=1e-5, logit_scale=0.75)

    return {
        "s": ("w2048-ff8192", vol("volalorn-s", 2048, 16, 4, 2048, 1024,
                                  8192, 4),
              LlamaConfig(name="llama-s", vocab_size=32000, hidden_size=2048,
                          n_layers=4, n_heads=16, n_kv_heads=4,
                          intermediate_size=8192, tie_embeddings=False), None),
        "l": ("w4096-ff14336", vol("volalorn-l", 4096, 32, 8, 8192, 4096,
                                   14336, 4),
              LlamaConfig(name="llama-l", vocab_size=32000, hidden_size=4096,
                          n_layers=4, n_heads=32, n_kv_heads=8,
                          intermediate_size=14336, tie_embeddings=False),
              None),
    }


def _pekarax_points():
    """Pekarax size points beside Mixtral stacks of equal width, attention
    head counts, expert count, expert size and top-k: four layers
    (channel-delta, parallel attention + mLSTM, gated linear attention,
    channel-delta), every one followed by the routed experts (two identity
    experts on top of the weighted ones, two groups of which one is
    kept)."""
    from agentainer_amd import ops
    from agentainer_amd.models.mixtral import MixtralConfig
    from agentainer_amd.models.pekarax import (GroupedExpertsConfig,
                                               MatrixMemoryConfig,
                                               PekaraxConfig,
                                               PekaraxLayerConfig)
    from agentainer_amd.models.volalorn import MaskedAttentionConfig

    def pek(name, width, heads, kv, ff, experts, top):
        ex = GroupedExpertsConfig(experts=experts, identity=2, top=top, ff=ff,
                                  limit=7.0, groups=2, keep_groups=1,
                                  scale=2.0)
        hv = width // 128
        delta = MatrixMemoryConfig(ops.SCAN_DELTA, hv, hv // 2, 128, 128,
                                   conv_taps=4, decay_rank=64, gate_rank=64)
        gla = MatrixMemoryConfig(ops.SCAN_GLA, hv // 2, hv // 2, 128, 256,
                                 decay_rank=64, tau=8.0)
        mlstm = MatrixMemoryConfig(ops.SCAN_MLSTM, hv // 2, hv // 2, 128, 256,
                                   gate_cap=15.0)
        attn = MaskedAttentionConfig(
            heads=heads, kv_heads=kv, dim=128, vdim=128, scale=0.09,
            mask_kind=ops.MASK_CAUSAL, mask_size=0, rot_dims=64,
            rot_base=500000.0, conv_taps=3)
        layers = [PekaraxLayerConfig("channel_delta", memory=delta, mlp=ex),
                  PekaraxLayerConfig("parallel", attn=attn, memory=mlstm,
                                     attn_scale=0.8, memory_scale=0.9, mlp=ex),
                  PekaraxLayerConfig("gla", memory=gla, mlp=ex),
                  PekaraxLayerConfig("channel_delta", memory=delta, mlp=ex)]
        return PekaraxConfig(name=name, vocab_size=32000, hidden_size=width,
                             layers=layers, norm_eps=1e-5, postln_alpha=2.0)

    return {
        "s": ("w2048-8x4096-top2", pek("pekarax-s", 2048, 16, 4, 4096, 8, 2),
              MixtralConfig(name="mixtral-s", vocab_size=32000,
                            hidden_size=2048, n_layers=4, n_heads=16,
                            n_kv_heads=4, intermediate_size=4096,
                            n_experts=8, top_k=2, tie_embeddings=False),
              "mixtral"),
        "l": ("w4096-8x7168-top2", pek("pekarax-l", 4096, 32, 8, 7168, 8, 2),
              MixtralConfig(name="mixtral-l", vocab_size=32000,
                            hidden_size=4096, n_layers=4, n_heads=32,
                            n_kv_heads=8, intermediate_size=7168,
                            n_experts=8, top_k=2, tie_embeddings=False),
              "mixtral"),
    }


def _sipelorn_points():
    """Sipelorn size points beside Mixtral stacks of equal width, attention
    head counts, expert count, expert size and top-k: four layers (latent
    attention, window attention, window attention on the previous layer's
    keys and values, latent attention); three are followed by the routed
    experts (two groups of which one is kept, plus a shared expert of a
    quarter of an expert's size), the last by a dense xIELU feed-forward of
    twice an expert's size. Bigram table, per-layer token inputs of 256
    values and gated residuals as the design has them. The latent pool row
    (latent + rotated key part) is 256 wide at width 2048 and 512 at 4096."""
    from agentainer_amd import ops
    from agentainer_amd.models.mixtral import MixtralConfig
    from agentainer_amd.models.sipelorn import (RotaryLatentConfig,
                                                SipelornConfig,
                                                SipelornFeedForwardConfig,
                                                SipelornLayerConfig)
    from agentainer_amd.models.volalorn import MaskedAttentionConfig

    def sip(name, width, heads, kv, ff, experts, top, rank, window):
        moe = SipelornFeedForwardConfig("moe", ff, experts=experts, top=top,
                                        groups=2, keep_groups=1,
                                        shared_ff=ff // 4)
        latent = RotaryLatentConfig(
            heads=heads, dim=128, rot_dim=64, vdim=128, kv_rank=rank,
            scale=192 ** -0.5, rot_dims=64, rot_base=1e6,
            rot_scaling={"factor": 4.0, "original": 4096, "fast": 16.0,
                         "slow": 2.0})

        def attn(src=None):
            return MaskedAttentionConfig(
                heads=heads, kv_heads=kv, dim=128, vdim=128, scale=0.09,
                mask_kind=ops.MASK_WINDOW, mask_size=window, qkv_bias=True,
                conv_taps=4, plain_qk=True, dist_bias=True, elem_gate=True,
                kv_from=src)

        layers = [
            SipelornLayerConfig("latent_attention", latent=latent, mlp=moe),
            SipelornLayerConfig("attention", attn=attn(), mlp=moe),
            SipelornLayerConfig("attention", attn=attn(1), mlp=moe),
            SipelornLayerConfig("latent_attention", latent=latent,
                                mlp=SipelornFeedForwardConfig("dense",
                                                              2 * ff))]
        return SipelornConfig(name=name, vocab_size=32000, hidden_size=width,
                              layers=layers, norm_eps=1e-5, embed_scale=8.0,
                              bigram_buckets=65521, bigram_mul_prev=36313,
                              bigram_mul_cur=27191, side_dim=256)

    return {
        "s": ("w2048-8x4096-top2",
              sip("sipelorn-s", 2048, 16, 4, 4096, 8, 2, 192, 1024),
              MixtralConfig(name="mixtral-s", vocab_size=32000,
                            hidden_size=2048, n_layers=4, n_heads=16,
                            n_kv_heads=4, intermediate_size=4096,
                            n_experts=8, top_k=2, tie_embeddings=False),
              "mixtral"),
        "l": ("w4096-8x7168-top2",
              sip("sipelorn-l", 4096, 32, 8, 7168, 8, 2, 448, 4096),
              MixtralConfig(name="mixtral-l", vocab_size=32000,
                            hidden_size=4096, n_layers=4, n_heads=32,
                            n_kv_heads=8, intermediate_size=7168,
                            n_experts=8, top_k=2, tie_embeddings=False),
              "mixtral"),
    }


def run_arch_compare(args):
    """Prefill (8 x 1024-token prompts per step) and decode (64 sequences at
    1024 tokens of context, captured graph) throughput, through the
    engine's own varlen and decode step functions."""
    from agentainer_amd.engine.llm import ModelInstance
    from agentainer_amd.models.lelitar import LelitarForCausalLM
    from agentainer_amd.models.mixtral import MixtralForCausalLM
    from agentainer_amd.models.pekarax import PekaraxForCausalLM
    from agentainer_amd.models.sipelorn import SipelornForCausalLM
    from agentainer_amd.models.volalorn import VolalornForCausalLM

    dev = "cuda" if torch.cuda.is_available() else "cpu"
    small = dev == "cpu"
    n_pf, pf_len, n_dec, ctx = (2, 64, 4, 64) if small else (8, 1024, 64, 1024)
    steps = max(3, min(args.steps, 20))
    ecfg = {"sync_mode": True, "async_decode": False, "prefill_stream": False,
            "prefix_sharing": False, "kv_page_size": 16,
            "kv_pool_tokens": (n_dec + n_pf) * (ctx + 256) + 4096,
            "max_seqs": n_dec + n_pf + 2, "max_batch_tokens": 1 << 20,
            "max_decode_batch": n_dec}

    def sync():
        if dev == "cuda":
            torch.cuda.synchronize()

    def measure(name, cfg, cls):
        inst = ModelInstance(name, cfg, dev, ecfg, model_cls=cls)
        g = torch.Generator().manual_seed(0)

        def toks(n):
            return torch.randint(3, cfg.vocab_size, (n,), generator=g).tolist()

        # prefill: fresh sequences every step
        pf_ms = []
        for it in range(steps + 2):
            plan = [(f"p{i}", toks(pf_len), False, None) for i in range(n_pf)]
            sync()
            t0 = time.time()
            inst._prefill_exec(plan)
            sync()
            if it >= 2:
                pf_ms.append((time.time() - t0) * 1e3)
            for i in range(n_pf):
                inst.kvm.free_seq(f"p{i}")
        # decode: n_dec sequences with ctx tokens of context
        for i in range(0, n_dec, 8):
            inst._prefill_exec([(f"d{j}", toks(ctx), False, None)
                                for j in range(i, min(i + 8, n_dec))])
        plan = [(f"d{j}", 5) for j in range(n_dec)]
        dec_ms = []
        for it in range(steps * 4 + 4):
            sync()
            t0 = time.time()
            inst._decode_exec(plan)
            sync()
            if it >= 4:
                dec_ms.append((time.time() - t0) * 1e3)
        del inst
        if dev == "cuda":
            torch.cuda.empty_cache()
        pf = statistics.median(pf_ms)
        dc = statistics.median(dec_ms)
        return {"prefill_ms": round(pf, 3),
                "prefill_tok_s": round(n_pf * pf_len / pf * 1e3),
                "decode_ms": round(dc, 3),
                "decode_tok_s": round(n_dec / dc * 1e3)}

    design = args.arch_design
    pts = {"volalorn": _volalorn_points, "pekarax": _pekarax_points,
           "sipelorn": _sipelorn_points, "lelitar": _arch_points}[design]()
    ours_cls = {"volalorn": VolalornForCausalLM,
                "pekarax": PekaraxForCausalLM,
                "sipelorn": SipelornForCausalLM,
                "lelitar": LelitarForCausalLM}[design]
    for key in (args.arch_sizes or ",".join(pts)).split(","):
        label, lcfg, rcfg, kind = pts[key.strip()]
        if small:  # CPU dry run: shrink to something that finishes
            continue
        ours = measure(lcfg.name, lcfg, ours_cls)
        theirs = measure(rcfg.name, rcfg,
                         MixtralForCausalLM if kind == "mixtral" else None)
        print(json.dumps({
            "metric": "arch_compare", "point": label, "layers": rcfg.n_layers,
            "prefill": f"{n_pf}x{pf_len}", "decode": f"{n_dec}@{ctx}",
            "dtype": "bf16", "data": "synthetic", design: ours,
            "reference_model": rcfg.name, "reference": theirs,
            "prefill_ratio": round(ours["prefill_tok_s"]
                                   / theirs["prefill_tok_s"], 3),
            "decode_ratio": round(ours["decode_tok_s"]
                                  / theirs["decode_tok_s"], 3)}), flush=True)


class ClosedLoopClient:
    """One agent's closed loop: WAL append -> submit -> on completion WAL
    ack + history write -> next request."""

    def __init__(self, agent, inst, store, wal, prompt_len, gen_len, seed):
        self.agent = agent
        self.inst = inst
        self.store = store
        self.wal = wal
        self.prompt_len = prompt_len
        self.gen_len = gen_len
        self.rng = torch.Generator().manual_seed(seed)
        self.active = None
        self.active_wal = None
        self.completed = []  # (t_submit, t_done)

    def _prompt_tokens(self):
        v = self.inst.cfg.vocab_size
        return torch.randint(3, v, (self.prompt_len,), generator=self.rng).tolist()

    def submit(self):
        toks = self._prompt_tokens()
        wal_req = self.wal.store_request(self.agent.id, "POST", "/chat",
                                         body={"tokens": self.prompt_len})
        req = GenRequest(agent_id=self.agent.id, prompt_tokens=toks,
                         max_new=self.gen_len, temperature=0.0, top_p=1.0, seed=0)
        b = self.inst.binding(self.agent.id)
        with self.inst._lock:
            b.queue.put(req)
            self.inst._pump_agent(b)
        self.active = req
        self.active_wal = wal_req

    def poll(self, record: bool):
        if self.active is not None and self.active.done.is_set():
            req = self.active
            self.wal.store_response(self.agent.id, self.active_wal.id,
                                    {"tokens": len(req.generated)})
            hist = f"agent:{self.agent.id}:conversations"
            self.store.rpush(hist, {"user": "bench", "tokens": len(req.generated),
                                    "ts": req.fin_t})
            if self.store.llen(hist) > 50:
                self.store.ltrim(hist, -50, -1)
            if record:
                self.completed.append((req.enq_t, req.fin_t))
            # KV hygiene: schedule a conversation reset so seq length stays
            # bounded. pending_reset is applied AT ADMISSION inside the
            # engine (plan-mirrored), so TP workers reset in lockstep and
            # no pages are freed under an in-flight speculative step.
            b = self.inst.binding(self.agent.id)
            if b is not None:
                b.pending_reset = True
            self.submit()


def main():
    args = parse_args()
    if args.arch_compare:
        run_arch_compare(args)
        return
    rank = int(os.environ.get("RANK", "0"))
    world = int(os.environ.get("WORLD_SIZE", "1"))
    has_gpu = torch.cuda.is_available()
    device = "cuda" if has_gpu else "cpu"
    if has_gpu:
        local_rank = int(os.environ.get("LOCAL_RANK", "0"))
        torch.cuda.set_device(local_rank)
    dist = None
    if world > 1:
        import torch.distributed as dist_mod
        dist = dist_mod
        dist.init_process_group(backend="nccl" if has_gpu else "gloo")

    tp = max(args.tp, 1)
    if tp > 1 and world != tp:
        raise SystemExit(f"--tp {tp} requires a torchrun world of {tp} "
                         f"(got WORLD_SIZE={world})")
    if tp > 1:
        model_name = args.model or ("llama3-70b" if has_gpu else "tiny-llama-tp")
    else:
        model_name = args.model or ("llama3-8b" if has_gpu else "tiny-llama")
    if not has_gpu and args.model is None:
        # CPU fallback sizes so the no-GPU smoke run finishes in seconds
        args.agents = min(args.agents, 4)
        args.prompt_len = min(args.prompt_len, 32)
        args.gen_len = min(args.gen_len, 8)
        args.steps = min(args.steps, 40)
        args.warmup = min(args.warmup, 8)
    # any driver-chosen --steps must complete requests INSIDE the timed
    # region (a gen_len longer than the window yields a vacuous 0 req/s):
    # cap generation length at half the timed steps
    args.gen_len = max(1, min(args.gen_len, max(args.steps // 2, 1)))

    tmp = tempfile.mkdtemp(prefix=f"bench-rank{rank}-")
    cfg = load_config(path="/nonexistent.yaml", env={})
    cfg.data["store"]["path"] = tmp
    cfg.data["engine"]["sync_mode"] = True
    cfg.data["engine"]["max_batch_tokens"] = args.max_batch_tokens
    cfg.data["engine"]["max_decode_batch"] = max(args.agents, 1)
    cfg.data["engine"]["expert_fp8"] = bool(args.expert_fp8)
    cfg.data["engine"]["expert_fp4"] = bool(args.expert_fp4)
    cfg.data["engine"]["dense_quant"] = args.dense_quant
    if args.kv_fp8:
        cfg.data["engine"]["kv_dtype"] = "fp8"
    if tp > 1:
        cfg.data["engine"]["tp_degree"] = tp
    store = Store(os.path.join(tmp, "state"), sync="interval")
    engine = LLMEngine(store, cfg, device=device, state_root=tmp)
    if tp > 1 and rank != 0:
        # SPMD worker: execute rank 0's broadcast step plans (incl. the
        # "barrier" timing fences) until shutdown
        engine.run_worker()
        dist.destroy_process_group()
        return
    manager = Manager(store, engine, cfg)
    wal = RequestManager(store)

    def fence():
        """Synchronize + barrier on every rank (TP: via the plan channel)."""
        if tp > 1:
            import agentainer_amd.parallel as par
            par.send_ints([OP_BARRIER])
        if has_gpu:
            torch.cuda.synchronize()
        if dist:
            dist.barrier()

    t_load0 = time.time()
    agents = []
    for i in range(args.agents):
        a = manager.deploy(name=f"bench-{i}", model=model_name,
                           sampling={"max_tokens": args.gen_len})
        manager.start(a.id)
        agents.append(a)
    inst = engine._instances[model_name]
    if rank == 0:
        print(f"# model={model_name} load+attach {time.time()-t_load0:.1f}s "
              f"pages={inst.kvm.n_pages}", file=sys.stderr)

    clients = [ClosedLoopClient(a, inst, store, wal, args.prompt_len,
                                args.gen_len, seed=1000 * rank + i)
               for i, a in enumerate(agents)]
    for c in clients:
        c.submit()

    def run_steps(n, record):
        for _ in range(n):
            inst.step()
            for c in clients:
                c.poll(record)

    # warmup
    run_steps(args.warmup, record=False)
    for c in clients:
        c.completed.clear()

    # timed region
    fence()
    t0 = time.time()
    run_steps(args.steps, record=True)
    fence()
    t1 = time.time()

    elapsed = t1 - t0
    n_done = sum(len(c.completed) for c in clients)
    e2es = sorted(d - s for c in clients for (s, d) in c.completed)
    decode_tokens = inst.decode_tokens
    prefill_tokens = inst.prefill_tokens

    if dist and tp == 1:
        # weak DP: whole-job aggregate = sum of completions / MAX elapsed,
        # with the e2e populations of EVERY rank merged so p50/p99 are
        # whole-job too (not rank-0-only)
        dd = device if has_gpu else "cpu"
        stats = torch.tensor([elapsed, float(n_done)],
                             dtype=torch.float64, device=dd)
        gathered = [torch.zeros_like(stats) for _ in range(world)]
        dist.all_gather(gathered, stats)
        elapsed = max(float(g[0]) for g in gathered)  # MAX over ranks
        n_done = sum(float(g[1]) for g in gathered)
        n = torch.tensor([len(e2es)], dtype=torch.int64, device=dd)
        ns = [torch.zeros_like(n) for _ in range(world)]
        dist.all_gather(ns, n)
        width = max(int(x.item()) for x in ns)
        if width > 0:
            buf = torch.full((width,), float("nan"), dtype=torch.float64,
                             device=dd)
            if e2es:
                buf[: len(e2es)] = torch.tensor(e2es, dtype=torch.float64,
                                                device=dd)
            bufs = [torch.zeros_like(buf) for _ in range(world)]
            dist.all_gather(bufs, buf)
            e2es = sorted(v for b in bufs for v in b.tolist() if v == v)

    if rank == 0:
        p50 = statistics.median(e2es) if e2es else None
        p99 = (e2es[min(len(e2es) - 1, int(0.99 * len(e2es)))] if e2es else None)
        out = {
            "metric": "concurrent_agent_chat_req_per_s",
            "value": round(n_done / elapsed, 3),
            "unit": "req/s",
            "n_gpus": world if has_gpu else 0,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(elapsed / args.steps * 1000, 3),
            "higher_is_better": True,
            "scaling": "strong" if tp > 1 else "weak",
            "vs_baseline": None,  # reference publishes no number
            "dtype": (f"bf16+{args.dense_quant}w" if args.dense_quant else
                      "bf16+fp4exp" if args.expert_fp4 else
                      "bf16+fp8exp" if args.expert_fp8 else
                      "bf16+fp8kv" if args.kv_fp8 else "bf16"),
            "data": "synthetic",
            "config": {
                "model": model_name,
                "agents_per_gpu": args.agents if tp == 1 else None,
                "agents": args.agents * (max(world, 1) if tp == 1 else 1),
                "global_batch": args.agents * (max(world, 1) if tp == 1 else 1),
                "prompt_len": args.prompt_len,
                "gen_len": args.gen_len,
                "seq_len": args.prompt_len + args.gen_len,
                "parallelism": (f"tp{world}" if tp > 1 else f"dp{max(world,1)}"),
                "p50_e2e_s": round(p50, 4) if p50 is not None else None,
                "p99_e2e_s": round(p99, 4) if p99 is not None else None,
                "decode_tokens_rank0": decode_tokens,
                "prefill_tokens_rank0": prefill_tokens,
            },
        }
        print(json.dumps(out))
    if tp > 1:
        engine.shutdown()  # broadcasts shutdown so workers exit run_worker
    if dist:
        dist.destroy_process_group()


if __name__ == "__main__":
    main()
