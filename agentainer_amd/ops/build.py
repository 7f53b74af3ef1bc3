"""In-tree build of the gfx950 HIP extension.

Drives hipcc directly (no hipify, no CUDA shims): every .hip/.cpp under
csrc/ is compiled for --offload-arch=gfx950 and linked into
agentainer_amd/ops/_hip_ops.so. Built in-tree so the .so travels with the
gpurun snapshot (a JIT cache under ~/.cache would not).

hipcc cross-compiles on a GPU-less box, so `python -m agentainer_amd.ops.build`
doubles as the does-it-build check.
"""

from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

import torch
from torch.utils import cpp_extension

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
# AGENTAINER_ASAN=1 builds a host-AddressSanitized variant (SURVEY.md §5
# race-detection row): the C++ binding layer (all torch interop, tensor
# lifetime, host bookkeeping) compiles with -fsanitize=address; device
# .hip kernels stay unsanitized (device ASAN needs xnack+, not a serving
# config). Run it with LD_PRELOAD=$(clang -print-file-name=libclang_rt.asan-x86_64.so).
ASAN = os.environ.get("AGENTAINER_ASAN", "") == "1"
OUT = os.path.join(HERE, "_hip_ops_asan.so" if ASAN else "_hip_ops.so")
OBJ_DIR = os.path.join(HERE, "_build_asan" if ASAN else "_build")
ARCH = os.environ.get("PYTORCH_ROCM_ARCH", "gfx950")

# the latent-attention family's kernels build into their own module so a
# deployment that serves only that family compiles only these
LATENT_SOURCES = [
    "latent_bindings.cpp",
    "grouped_norm.hip",
    "latent_attn.hip",
    "routed_ffn.hip",
]

# scalar-gain norms, PolyNorm, rotary + q/k norm + append, masked attention
MASKED_SOURCES = [
    "masked_bindings.cpp",
    "scalar_norm.hip",
    "rotary_norm.hip",
    "masked_attn.hip",
]

# post-norm residual, short convolutions with state, matrix-memory scans,
# head norm + gate, group-limited routing, clamped gated experts
RECURRENT_SOURCES = [
    "recurrent_bindings.cpp",
    "postln_norm.hip",
    "short_conv.hip",
    "matrix_memory.hip",
    "matrix_memory_gla.hip",
    "matrix_memory_delta.hip",
    "matrix_memory_mlstm.hip",
    "grouped_route.hip",
]

# hashed bigram embedding, gated residual + layer norm, xIELU, sigmoid
# group routing, output-weighted gated experts, latent rotary append
GATED_SOURCES = [
    "gated_bindings.cpp",
    "gated_norm.hip",
    "bigram_embed.hip",
    "sigmoid_route.hip",
    "latent_rotary.hip",
]

SOURCES = [
    "bindings.cpp",
    "rmsnorm.hip",
    "elementwise.hip",
    "rope.hip",
    "kvcache.hip",
    "decode_attn.hip",
    "prefill_attn.hip",
    "sampling.hip",
    "skinny_gemm.hip",
]


def _newest(paths):
    return max(os.path.getmtime(p) for p in paths if os.path.exists(p))


def _target(target: str):
    """(output .so, object dir, sources, module name) of a build target."""
    if target == "latent":
        sfx = "_asan" if ASAN else ""
        return (os.path.join(HERE, f"_hip_latent{sfx}.so"),
                os.path.join(HERE, "_build_latent" + sfx), LATENT_SOURCES,
                "_hip_latent")
    if target == "masked":
        sfx = "_asan" if ASAN else ""
        return (os.path.join(HERE, f"_hip_masked{sfx}.so"),
                os.path.join(HERE, "_build_masked" + sfx), MASKED_SOURCES,
                "_hip_masked")
    if target == "recurrent":
        sfx = "_asan" if ASAN else ""
        return (os.path.join(HERE, f"_hip_recurrent{sfx}.so"),
                os.path.join(HERE, "_build_recurrent" + sfx),
                RECURRENT_SOURCES, "_hip_recurrent")
    if target == "gated":
        sfx = "_asan" if ASAN else ""
        return (os.path.join(HERE, f"_hip_gated{sfx}.so"),
                os.path.join(HERE, "_build_gated" + sfx), GATED_SOURCES,
                "_hip_gated")
    if target != "core":
        raise ValueError(f"unknown build target {target!r}")
    return OUT, OBJ_DIR, SOURCES, "_hip_ops"


def needs_build(target: str = "core") -> bool:
    OUT, _obj, SOURCES, _name = _target(target)
    if not os.path.exists(OUT):
        return True
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    srcs.append(os.path.join(CSRC, "common.h"))
    srcs.append(os.path.join(CSRC, "latent_common.h"))
    srcs.append(os.path.join(CSRC, "matrix_memory_kernel.h"))
    srcs.append(os.path.abspath(__file__))
    return _newest(srcs) > os.path.getmtime(OUT)


def build(verbose: bool = True, force: bool = False,
          target: str = "core") -> str:
    if target == "all":
        target = "core+latent+masked+recurrent+gated"
    if "+" in target:
        out = ""
        for t in target.split("+"):
            out = build(verbose, force, t)
        return out
    OUT, OBJ_DIR, SOURCES, modname = _target(target)
    if not force and not needs_build(target):
        return OUT
    os.makedirs(OBJ_DIR, exist_ok=True)
    torch_inc = cpp_extension.include_paths()
    torch_lib = cpp_extension.library_paths()[0]
    py_inc = sysconfig.get_paths()["include"]
    inc_flags = [f"-I{p}" for p in torch_inc + [py_inc, CSRC]]
    cxx_flags = [
        "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        f"-DTORCH_EXTENSION_NAME={modname}",
        # packed-fp32 VALU forms are kept out of generated code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-D_GLIBCXX_USE_CXX11_ABI=1",
        "-fno-gpu-rdc",
        "-Wno-unused-result",
    ]
    objs = []
    procs = []
    for src in SOURCES:
        src_path = os.path.join(CSRC, src)
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        objs.append(obj)
        if (os.path.exists(obj)
                and os.path.getmtime(obj) > _newest(
                    [src_path, os.path.join(CSRC, "common.h"),
                     os.path.join(CSRC, "latent_common.h"),
                     os.path.join(CSRC, "matrix_memory_kernel.h")])
                and not force):
            continue
        san = (["-fsanitize=address", "-shared-libsan"]
               if ASAN and src.endswith(".cpp") else [])
        cmd = (["hipcc", "-c", src_path, "-o", obj] + cxx_flags + san
               + inc_flags + (["-x", "hip"] if src.endswith(".cpp") else []))
        if verbose:
            print("[ops.build]", " ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                            stderr=subprocess.STDOUT)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        if p.returncode != 0:
            failed = True
            print(f"[ops.build] FAILED {src}:\n{out.decode()}", file=sys.stderr)
    if failed:
        raise RuntimeError("HIP extension build failed")
    link = (["hipcc", "-shared", "-fPIC", "-o", OUT] + objs
            + (["-fsanitize=address", "-shared-libsan"] if ASAN else [])
            + [f"-L{torch_lib}", "-ltorch", "-ltorch_python", "-lc10",
               "-ltorch_hip", "-lc10_hip", f"-Wl,-rpath,{torch_lib}"])
    if verbose:
        print("[ops.build]", " ".join(link), flush=True)
    tmp_out = OUT + f".tmp{os.getpid()}"
    link[link.index(OUT)] = tmp_out
    res = subprocess.run(link, capture_output=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout.decode()}\n{res.stderr.decode()}")
    os.replace(tmp_out, OUT)
    return OUT


if __name__ == "__main__":
    targets = [a for a in sys.argv[1:] if not a.startswith("-")] or ["all"]
    for t in targets:
        print("built", build(force="--force" in sys.argv, target=t))
