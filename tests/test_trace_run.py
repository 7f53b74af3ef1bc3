"""bin/trace_run as a program: JSON steps in, logits files and 'done'
lines out, against the plain oracle (CPU engine path)."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import lelitar_oracle as O  # noqa: E402
import pekarax_oracle as PO  # noqa: E402
import sipelorn_oracle as SO  # noqa: E402
import volalorn_oracle as VO  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "bin", "trace_run")


def _run(model, out, steps, dtype="float32", max_tokens=128):
    p = subprocess.run(
        [sys.executable, TOOL, "--model", model, "--dtype", dtype, "--out",
         out, "--max-tokens", str(max_tokens), "--device", "cpu"],
        input="".join(json.dumps(s) + "\n" for s in steps), text=True,
        capture_output=True, timeout=300)
    return p


def _lelitar_case():
    cfg = O.random_config(vocab=120, window=6, kinds=("moe", "dense", None))
    return O, cfg, O.random_weights(cfg, seed=21)


def _volalorn_case():
    cfg = VO.make_config(
        [VO.sigmoid_mixer(chunk=5), VO.softmax_mixer(window=6, keep_first=2),
         VO.sigmoid_mixer(chunk=16, softcap=None)], vocab=120, no_ff=(1,))
    return VO, cfg, VO.random_weights(cfg, seed=22)


def _pekarax_case():
    cfg = PO.make_config([PO.delta_layer(), PO.parallel_layer(),
                          PO.gla_layer()], vocab=120, no_ff=(1,))
    return PO, cfg, PO.random_weights(cfg, seed=23)


class _SipelornOracle:
    """The Sipelorn oracle behind the other oracles' call signature."""
    save_checkpoint = staticmethod(SO.save_checkpoint)

    @staticmethod
    def forward(cfg, w, tokens):
        return SO.forward(tokens, w, cfg).float()


def _sipelorn_case():
    cfg = SO.make_config(
        [(SO.latent_mixer(), SO.moe_mlp()),
         (SO.window_mixer(window=6), SO.dense_mlp()),
         (SO.window_mixer(window=9, kv_from=1), None)], vocab=120)
    return _SipelornOracle, cfg, SO.random_weights(cfg, seed=24)


@pytest.mark.parametrize("case", [_lelitar_case, _volalorn_case,
                                  _pekarax_case, _sipelorn_case])
def test_trace_run_mixed_steps_match_oracle(tmp_path, case):
    O, cfg, w = case()
    model = str(tmp_path / "ckpt")
    O.save_checkpoint(model, cfg, w)
    g = torch.Generator().manual_seed(3)
    a = torch.randint(0, 120, (37,), generator=g).tolist()
    b = torch.randint(0, 120, (20,), generator=g).tolist()
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}],
         "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]},
                                {"id": "b", "tokens": b[:9], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[9:], "want": [10]}],
         "end": ["b"]},                      # a sits this step out
        {"step": 3, "entries": [{"id": "a", "tokens": a[18:], "want": [5, 18]}],
         "end": ["a"]},
        {"step": 4, "entries": [{"id": "c", "tokens": b[:2], "want": [1]}],
         "end": ["c"]},                      # pages and slot of b again
    ]
    out = str(tmp_path / "out")
    p = _run(model, out, steps)
    assert p.returncode == 0, p.stderr[-2000:]
    done = [ln for ln in p.stdout.splitlines() if ln.startswith("done ")]
    assert done == [f"done {i}" for i in range(5)]
    la, lb = O.forward(cfg, w, a), O.forward(cfg, w, b)
    want = {0: la[[0, 16]], 1: la[[17]], 2: lb[[19]], 3: la[[23, 36]],
            4: lb[[1]]}
    V = cfg["vocab"]
    for n, ref in want.items():
        got = torch.from_numpy(
            np.fromfile(os.path.join(out, f"{n}.f32"), dtype="<f4")
            .reshape(-1, V))
        assert got.shape == ref.shape
        assert float((got - ref).abs().max() / ref.abs().max()) < 3e-4, n


def test_trace_run_refuses_float32_for_bf16_only_family(tmp_path):
    d = tmp_path / "llama"
    d.mkdir()
    (d / "config.json").write_text(json.dumps({
        "model_type": "llama", "num_attention_heads": 4, "hidden_size": 512,
        "vocab_size": 512, "num_hidden_layers": 1, "num_key_value_heads": 1,
        "intermediate_size": 256}))
    p = _run(str(d), str(tmp_path / "o"), [], dtype="float32")
    assert p.returncode == 3
