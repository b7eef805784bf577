"""Builds libfta.so (the C-ABI library) in-tree with hipcc for gfx950.

Run as `python -m flash_tree_attn_amd.build`. hipcc cross-compiles, so no GPU is
needed to build. The library is written next to this file and loaded by ctypes.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_PATH = os.path.join(HERE, "libfta.so")
SOURCES = ["fta_host.cpp", "stage1_shuffle.hip", "stage1_mfma.hip", "stage1_mfma_wide.hip", "stage1_mfma_splitkeys.hip", "stage2_merge.hip", "append_kv.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # NaN-agnostic min/max (no canonicalising v_max x,x,x); infinities stay honoured,
    # the kernels use -inf as the "masked" logit.
    "-fno-honor-nans",
    "-I", INCLUDE, "-I", CSRC,
] + os.environ.get("FTA_EXTRA_FLAGS", "").split()


def _compile(src: str) -> str:
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def _link(objs, path: str) -> None:
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", path]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")


def _generate() -> None:
    """Rewrites csrc/wide_loop_asm.inc from its generator (deterministic; the file is committed)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("gen_wide_loop", os.path.join(CSRC, "gen_wide_loop.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    text = mod.render()
    path = os.path.join(CSRC, "wide_loop_asm.inc")
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as f:
            f.write(text)


def build(verbose: bool = True) -> str:
    """Compiles every HIP source of the library and links it."""
    _generate()
    with ThreadPoolExecutor(max_workers=min(6, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    _link(objs, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build()
