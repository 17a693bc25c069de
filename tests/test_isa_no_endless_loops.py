"""The kernels whose waves wait for each other through LDS words bound every such wait, so that a launch
always ends. What the bound cannot guard against is a loop the compiler makes itself: an instantiation
of such a kernel has been seen to compile into a loop with an empty body that branches onto its own label
(the lanes of a wave that a transformation of the row loop had parked there never left it). This test
compiles those sources to gfx950 ISA and looks for that shape: a label followed, with nothing but
register moves and no-ops in between, by a branch back to the same label.
"""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "effect-torch_amd", "csrc")
SOURCES = ["gemv_limb.hip", "gemv_mma.hip"]

LABEL = re.compile(r"^(\.LBB\d+_\d+):")
BRANCH = re.compile(r"^\s+s_(?:branch|cbranch_\w+)\s+(\.LBB\d+_\d+)\s*$")
IDLE = re.compile(r"^\s+(?:s_mov_b(?:32|64)|s_nop|v_mov_b32\w*|s_and_b64\s+vcc,\s*exec,\s*0)\b")


def endless_loops(text):
    """Labels whose block does nothing but move registers and then branches back to itself."""
    found = []
    lines = text.splitlines()
    for i, line in enumerate(lines):
        match = LABEL.match(line)
        if not match:
            continue
        label = match.group(1)
        for follower in lines[i + 1:i + 6]:
            if follower.strip().startswith(";") or not follower.strip():
                continue
            branch = BRANCH.match(follower)
            if branch:
                if branch.group(1) == label:
                    found.append(label)
                break
            if not IDLE.match(follower):
                break
    return found


def test_the_detector_sees_the_shape():
    bad = ".LBB0_50:\n\ts_mov_b64 vcc, vcc\n\ts_cbranch_vccz .LBB0_50\n.LBB0_51:\n\ts_endpgm\n"
    assert endless_loops(bad) == [".LBB0_50"]
    polling = ".LBB0_7:\n\tds_read_b32 v1, v2\n\ts_waitcnt lgkmcnt(0)\n\ts_cbranch_vccnz .LBB0_7\n"
    assert endless_loops(polling) == []


@pytest.fixture(scope="module")
def listings():
    """The ISA of every source, compiled side by side (one compiler process each)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc here")
    with tempfile.TemporaryDirectory() as scratch:
        running = {}
        for source in SOURCES:
            out = os.path.join(scratch, source + ".s")
            command = [hipcc, "-S", "-o", out, os.path.join(CSRC, source), "--offload-arch=gfx950", "-O3", "-std=c++17",
                       "-fPIC", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-I", CSRC,
                       "-I", os.path.join(ROOT, "include"), "--cuda-device-only"]
            running[source] = (subprocess.Popen(command, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL), out)
        texts = {}
        for source, (process, out) in running.items():
            assert process.wait(timeout=900) == 0, f"hipcc failed on {source}"
            with open(out) as listing:
                texts[source] = listing.read()
    return texts


@pytest.mark.parametrize("source", SOURCES)
def test_no_loop_without_a_body(listings, source):
    text = listings[source]
    assert "s_endpgm" in text  # a listing of kernels, not an empty file
    assert endless_loops(text) == []
