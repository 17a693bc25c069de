"""Builds libet_hip.so (the C-ABI library of include/et_hip.h) and libet_hip_calibrate.so (the
measurement aids of include/et_hip_calibrate.h) for gfx950 with hipcc.

Usage: ``python build.py`` from anywhere. The libraries land next to this file
under ``lib/``; the first is what the tests, the smoke check and the benchmark
load, the second only the benchmark's ``calibrate_*`` workloads and the tests of
those aids. hipcc cross-compiles, so no GPU is needed to build.
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
CALIBRATE_LIB_PATH = os.path.join(LIB_DIR, "libet_hip_calibrate.so")

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
    "quantized.cpp": [],
    "static_workspace.cpp": [],
    "kv_cache.cpp": [],
    "decode_host.cpp": [],
    "gguf.cpp": [],
    "c_api.cpp": [],
}
# The measurement library: its own kernels, and the batched Q4_K kernel once more with the template
# instantiations that leave one part of it out (gemm_h16_probe; the rest of that file it takes from
# its own copy, so the operators' library carries no probe).
CALIBRATE_SOURCES = {
    # matrix-core results straight into VGPRs, as in the batch kernels (no accumulation-register moves)
    "calibrate.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
    "gemm_h16.hip": ["-DET_HIP_CALIBRATE"],
    "c_api_calibrate.cpp": [],
}


def _compile(item):
    name, extra = item
    src = os.path.join(CSRC, name)
    obj = os.path.join(OBJ_DIR, name + (".calibrate.o" if "-DET_HIP_CALIBRATE" in extra else ".o"))
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
    items = list(SOURCES.items()) + list(CALIBRATE_SOURCES.items())
    with ThreadPoolExecutor(max_workers=8) as pool:
        results = list(pool.map(_compile, items))
    for name, _, log in results:
        if verbose and log.strip():
            print(f"[{name}]\n{log}", file=sys.stderr)
    objs = [obj for _, obj, _ in results[:len(SOURCES)]]
    calibrate_objs = [obj for _, obj, _ in results[len(SOURCES):]]
    for path, members, extra in ((LIB_PATH, objs, []),
                                 # what the probe's copy of gemm_h16 shares with the operators (the reduction
                                 # kernels' launchers) comes from their library, found next to this one
                                 (CALIBRATE_LIB_PATH, calibrate_objs, ["-L", LIB_DIR, "-let_hip", "-Wl,-rpath,$ORIGIN"])):
        link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", path] + members + extra
        proc = subprocess.run(link, capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"link failed:\n{proc.stderr}")
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
