"""Builds libet_hip.so (the C-ABI library of include/et_hip.h) for gfx950 with hipcc.

Usage: ``python build.py`` from anywhere. The library lands next to this file
as ``lib/libet_hip.so``; it is what the tests, the smoke check and the
benchmark load. hipcc cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(LIB_DIR, "libet_hip.so")

# Packed-FP32 instructions are switched off for all device code.
COMMON = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", CSRC, "-I", INCLUDE,
]
# dequant.hip must round every multiply and subtract separately (bit-exact decode).
SOURCES = {
    "dequant.hip": ["-ffp-contract=off"],
    "gemv_limb.hip": [],
    "gemv_mma.hip": [],
    "lds_handover.cpp": [],
    "gemv_generic.hip": [],
    "quantize_act.hip": ["-ffp-contract=off"],
    "gemm_i8.hip": [],
    "gemm_h16.hip": [],
    "kv_attention.hip": [],
    "decode_ops.hip": ["-ffp-contract=off"],
    # matrix-core results straight into VGPRs, as in the batch kernels (no accumulation-register moves)
    "calibrate.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "quantized.cpp": [],
    "static_workspace.cpp": [],
    "kv_cache.cpp": [],
    "decode_host.cpp": [],
    "gguf.cpp": [],
    "c_api.cpp": [],
}


def _compile(item):
    name, extra = item
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ_DIR, name + ".o")
    cmd = ["hipcc", "-c", src, "-o", obj] + COMMON + extra
    if name.endswith(".cpp"):
        cmd = ["hipcc", "-x", "hip", "-c", src, "-o", obj] + COMMON + extra
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature: harmless.
    noise = ("is not a recognized feature for this target", "1 warning generated", "warning generated")
    log = "\n".join(l for l in (proc.stderr or "").splitlines() if not any(n in l for n in noise))
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {name}:\n{proc.stderr}")
    return name, obj, log


def build(verbose: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        results = list(pool.map(_compile, SOURCES.items()))
    for name, _, log in results:
        if verbose and log.strip():
            print(f"[{name}]\n{log}", file=sys.stderr)
    objs = [obj for _, obj, _ in results]
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    proc = subprocess.run(link, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
