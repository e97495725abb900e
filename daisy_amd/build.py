"""Builds ``libdaisy_hip.so`` (the gfx950 kernels + C ABI) in-tree with hipcc.

Run as ``python -m daisy_amd.build``.  hipcc cross-compiles for gfx950 without
a GPU, so this works on a CPU-only machine; the resulting library sits next to
the sources so that it travels with the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_NAME = "libdaisy_hip.so"
LIB_PATH = os.path.join(CSRC, LIB_NAME)
SOURCES = ["abi.hip", "decode.hip", "prefill.hip", "kda.hip", "kda_step.hip", "prep.hip", "kimi.hip", "linear.hip", "layer_step.hip"]
# Diagnostic kernels of the benchmark (matrix-pipe and read-stream ceilings): not part of the product.  Their source
# sits next to bench.py at the repository root and is built into a library of its own there, which only bench.py loads.
ROOT = os.path.dirname(os.path.dirname(CSRC))
PROBE_LIB_NAME = "libdaisy_bench_probe.so"
PROBE_LIB_PATH = os.path.join(ROOT, PROBE_LIB_NAME)
PROBE_SOURCE = os.path.join(ROOT, "bench_probe.hip")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # Keep the compiler from forming packed-fp32 instructions from scalar code.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")
    return exe


def _compile(src: str, verbose: bool) -> str:
    path = src if os.path.isabs(src) else os.path.join(CSRC, src)
    obj = os.path.splitext(path)[0] + ".o"
    cmd = [_hipcc(), *HIPCC_FLAGS, "-I", ROOT, "-c", path, "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    if verbose and r.stderr.strip():
        # The host pass warns that it does not know the packed-fp32 feature; harmless.
        lines = [ln for ln in r.stderr.splitlines() if "packed-fp32-ops" not in ln]
        if lines:
            print("\n".join(lines), flush=True)
    return obj


def _link(objs, out: str, verbose: bool) -> None:
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")


def build(verbose: bool = True, sources=None) -> str:
    """Compiles every source and links the product library (and the benchmark's probe library);
    returns the product library's path."""
    srcs = list(sources or SOURCES)
    every = srcs + ([PROBE_SOURCE] if os.path.exists(PROBE_SOURCE) else [])
    if "abi.hip" not in every:
        every.append("abi.hip")
    with ThreadPoolExecutor(max_workers=min(4, len(every))) as ex:
        objs = dict(zip(every, ex.map(lambda s: _compile(s, verbose), every)))
    _link([objs[s] for s in srcs], LIB_PATH, verbose)
    if PROBE_SOURCE in objs:
        _link([objs["abi.hip"], objs[PROBE_SOURCE]], PROBE_LIB_PATH, verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-q" not in sys.argv))
