"""Builds libminivllm_amd.so (gfx950) in-tree with hipcc.

``python -m minivllm_amd._build`` or ``build_library()``.  The library is
written next to the sources' package (minivllm_amd/libminivllm_amd.so).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libminivllm_amd.so")
PROBE_LIB_PATH = os.path.join(PKG_DIR, "libmvllm_probe.so")      # measurement support for bench.py, not an operator
PROBE_SOURCES = ["mfma_probe.hip"]
SOURCES = ["capi.hip", "store_kvcache.hip", "paged_decode.hip", "prefill_varlen.hip", "prefill_other_dims.hip", "prefill_half_step_dims.hip", "prefill_pingpong.hip", "prefill_staged.hip", "prefill_split.hip", "prefill_f32.hip", "qk_norm_rope_store.hip", "sampler.hip",
           "rms_norm.hip", "activation.hip", "linear_small.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fhip-fp32-correctly-rounded-divide-sqrt",   # INT8 scales/codes must match IEEE division
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libminivllm_amd.so")
    return exe


def build_library(verbose: bool = True, jobs: int = 4) -> str:
    hipcc = _hipcc()
    obj_dir = os.path.join(PKG_DIR, "build")
    os.makedirs(obj_dir, exist_ok=True)

    def compile_one(src, extra=(), suffix=""):
        obj = os.path.join(obj_dir, src.replace(".hip", suffix + ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        # the probe library also holds the decode kernels built as "loads only" (the access pattern's ceiling)
        probe_decode = pool.submit(compile_one, "paged_decode.hip", ("-DMVLLM_DECODE_LOADS_ONLY=1",), "_loads_only")
        # ... and the two-group prefill kernel with its per-tile clock stamps
        probe_prefill = pool.submit(compile_one, "prefill_pingpong.hip", ("-DMVLLM_PP_TIMELINE=1",), "_timeline")
        objs = list(pool.map(compile_one, SOURCES + PROBE_SOURCES))
        objs.append(probe_decode.result())
        objs.append(probe_prefill.result())
    for lib, members in ((LIB_PATH, objs[:len(SOURCES)]), (PROBE_LIB_PATH, objs[len(SOURCES):])):
        cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *members]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
