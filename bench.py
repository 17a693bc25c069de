#!/usr/bin/env python3
"""Benchmark of the quantized-GGUF matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--vectors M]

A "step" is one pass of the hot path over one batch of synthetic input: one
``quantized_linear`` of the chosen workload, enqueued through the C ABI. The
default workload is the headline one: Q4_K dequant-GEMV, W 14336 x 4096, one
activation vector (M = 1). Inputs are resident in HBM before the timed region.

Cold HBM, not cache: the packed weight of every workload here fits the 256 MB
Infinity Cache, so consecutive steps rotate over enough distinct weight copies
(> 512 MiB in total) that no step can find its weight in a cache. ``--hot``
times the same buffer over and over instead (labelled, never the headline).

The K timed steps are captured once into a HIP graph (the launches go through
the C ABI on the capturing stream) and replayed, so the device sees K kernels
back to back without host launch gaps; HIP events on that stream bracket the
replay. One JSON line is printed at the end.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0        # MI355X dense int8 MFMA, published (5.0 POP/s)
F16_PEAK_TFLOPS = 2500.0       # MI355X dense fp16 MFMA, published (2.5 PFLOP/s)
ROTATE_BYTES = 640 << 20       # > 2x the 256 MB Infinity Cache

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by the same
# counters' reading for a plain copy of known size. The counters cannot be collected from inside
# this script, so each figure is tied to the kernel it was taken from: the kernel's name as the
# planner reports it and the SHA-256 of the source file that defines it at the time of the profile.
# When either differs from what runs now, `roofline.traffic` is null until the profile is re-taken.
MEASURED_TRAFFIC = {
    ("q4_k_gemv_14336x4096", 1, "f32"): {
        "bytes": 33283900, "kernel": "gemv_limb_dma", "source": "gemv_limb.hip",
        "sha256": "4fa7d816114655dcc55c2445c3543c2c2a4ee75ef28d65d3e37a1ac4883848cb",
        "profile": "profiles/gemv_limb_q4k_14336x4096_m1_hbm_traffic.md"},
    ("q4_0_gemv_11008x4096", 1, "f32"): {
        "bytes": 25614000, "kernel": "gemv_limb_dma", "source": "gemv_limb.hip",
        "sha256": "4fa7d816114655dcc55c2445c3543c2c2a4ee75ef28d65d3e37a1ac4883848cb",
        "profile": "profiles/gemv_limb_q4k_14336x4096_m1_hbm_traffic.md"},
    ("q4_k_gemv_14336x4096", 4, "f32"): {
        "bytes": 33895200, "kernel": "gemv_mma", "source": "gemv_mma.hip",
        "sha256": "f3bf93df89988bc17bec99050bd1b47eecb979a5c848917aad42700dfb58aba2",
        "profile": "profiles/gemv_mma_small_batch_2_to_8_vectors.md"},
    ("q4_k_gemv_14336x4096", 8, "f32"): {
        "bytes": 34754600, "kernel": "gemv_mma", "source": "gemv_mma.hip",
        "sha256": "f3bf93df89988bc17bec99050bd1b47eecb979a5c848917aad42700dfb58aba2",
        "profile": "profiles/gemv_mma_small_batch_2_to_8_vectors.md"},
    ("kv_attention_decode", 2048): {
        "bytes": 270024900, "kernel": "kv_attend", "source": "kv_attention.hip",
        "sha256": "590105a686a613206e4bfe632266890d8f03aa1f6a00829b1aa81122a1f041fd",
        "profile": "profiles/kv_attend_decode_32slots_ctx2048_f16.md"},
}


def measured_traffic(key, kernel_name):
    """The profiled HBM bytes per launch of `key`, or None when the kernel that runs now is not the
    one that was profiled (another kernel name, or its source file has changed since)."""
    import hashlib

    entry = MEASURED_TRAFFIC.get(key)
    if entry is None or not str(kernel_name).startswith(entry["kernel"]):
        return None
    path = os.path.join(ROOT, "effect-torch_amd", "csrc", entry["source"])
    try:
        with open(path, "rb") as source:
            digest = hashlib.sha256(source.read()).hexdigest()
    except OSError:
        return None
    return entry["bytes"] if digest == entry["sha256"] else None


def cpu_model():
    try:
        with open("/proc/cpuinfo") as info:
            for line in info:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


class pinned_to_one_core:
    """Pins this process to one host core for the CPU baseline (the reference's loop is single
    threaded) and restores the affinity afterwards."""

    def __enter__(self):
        self.before = None
        self.core = None
        try:
            self.before = os.sched_getaffinity(0)
            self.core = max(self.before)  # the highest allowed core: least likely to serve interrupts
            os.sched_setaffinity(0, {self.core})
        except (AttributeError, OSError):
            self.before = None
        return self

    def __exit__(self, *exc):
        if self.before is not None:
            try:
                os.sched_setaffinity(0, self.before)
            except OSError:
                pass
        return False

    def describe(self):
        where = f"pinned to core {self.core}" if self.before is not None else "not pinned"
        return f"{where} of {cpu_model()}"


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=None, help="timed steps (default 2000; llama3_8b_batched_decode: 128)")
    p.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default 200; "
                   "llama3_8b_batched_decode: 2)")
    p.add_argument("--workload", default="q4_k_gemv_14336x4096",
                   help="one of effect_torch_amd.synth.CONFIGS, calibrate_read, calibrate_copy, calibrate_mfma_{i8,i8_scaled,i8_scaled_bf16,i8_biased,i8_biased_matrix_only,i8_biased_valu_only,f16,f16_16x16}, calibrate_contraction, "
                        "kv_attention_decode")
    p.add_argument("--vectors", type=int, default=None, help="activation vectors M (default: first of the workload)")
    p.add_argument("--mode", choices=["f32", "int8"], default=None)
    p.add_argument("--kv-dtype", choices=["f16", "bf16", "u8", "f32"], default="f16",
                   help="kv_attention_decode / llama3_8b_batched_decode: element type of the key/value slabs "
                        "(u8 = the int8-quantized tier with one f32 scale per row and head)")
    p.add_argument("--codec", default="q4_k", help="quantized_embedding_vocab: the table's codec (q2_k ... q6_k, q4_0, q8_0)")
    p.add_argument("--context", type=int, default=2048, help="kv_attention_decode / llama3_8b_batched_decode: "
                   "positions per slot")
    p.add_argument("--unfused", action="store_true", help="llama3_8b_batched_decode: one launch sequence per "
                   "operator (no shared quantisation, separate residual sums)")
    p.add_argument("--layers", type=int, default=32, help="llama3_8b_batched_decode: transformer layers")
    p.add_argument("--hot", action="store_true", help="reuse one weight buffer (cache-resident; not the headline)")
    p.add_argument("--no-graph", action="store_true", help="enqueue the steps one by one instead of replaying a HIP graph")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-decode", action="store_true", help="headline workload: skip the batched-decode leg that fills "
                                                            "the line's `decode` object")
    p.add_argument("--cpu-seconds", type=float, default=10.0)
    p.add_argument("--waves-per-simd", type=int, default=2, help="calibrate_mfma_*: resident waves per SIMD (one workgroup of "
                   "four waves per compute unit each)")
    p.add_argument("--sizes-mib", default=None, help="calibrate_read_sweep: comma-separated sizes in MiB instead of "
                   "8 ... 1024 (the headline weight's size is always measured as well)")
    args = p.parse_args()
    decode = args.workload == "llama3_8b_batched_decode"
    if args.steps is None:
        args.steps = 128 if decode else 2000
    if args.warmup is None:
        args.warmup = 2 if decode else 200
    return args


def cpu_baseline(cfg, vectors, mode, weight, x, seconds, algorithmic_bytes):
    """Times the CPU oracle (a C restatement of the reference's scalar loop,
    crates/runtime-cpu/src/quantized.rs:447-498) on one host core over a bounded
    sample of the same workload."""
    import numpy as np
    import oracle

    rows, columns, codec = cfg["rows"], cfg["columns"], cfg["codec"]
    # Size the sample from a small probe: whole calls if one fits the budget, else a row range.
    probe_rows = min(rows, 64)
    t0 = time.perf_counter()
    oracle.linear_rows(codec, rows, columns, x[:1], weight, None, 0, probe_rows)
    per_row_vector = max((time.perf_counter() - t0) / probe_rows, 1e-9)
    full_call = per_row_vector * rows * vectors
    if full_call <= seconds:
        sample_rows, calls = rows, max(1, int(seconds / full_call))
    else:
        sample_rows, calls = max(16, int(seconds / (per_row_vector * vectors))), 1
        sample_rows = min(sample_rows, rows)
    y = np.zeros((vectors, rows), dtype=np.float32)
    with pinned_to_one_core() as pin:
        t0 = time.perf_counter()
        for _ in range(calls):
            oracle.linear_rows(codec, rows, columns, x, weight, None, 0, sample_rows, out=y)
        elapsed = time.perf_counter() - t0
        pinned = pin.describe()
    seconds_per_call = elapsed / calls * (rows / sample_rows)
    what = (f"{calls} full call(s) of the same workload" if sample_rows == rows else
            f"rows 0..{sample_rows} of {rows} of one call, scaled by {rows / sample_rows:.1f}")
    return {
        "value": round(algorithmic_bytes / seconds_per_call / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": f"{what}; {elapsed:.1f} s of CPU work; f32 activations, scalar C restatement of the "
                  f"reference's single-threaded loop ({seconds_per_call * 1e3:.1f} ms per call); {pinned}",
    }


MIN_GRAPH_STEPS = 400     # a graph of fewer kernels pays its launch (about 15 us) per step: see time_steps
MAX_GRAPH_STEPS = 2000    # ... and one of up to this many when the steps are short (a replay of about 15 ms)
GRAPH_WINDOW_MS = 15.0
MIN_REPETITIONS = 5       # timed replays of the K steps; the median is reported
TIMED_WINDOW_MS = 20.0    # short replays are repeated until about this much device time is covered
MAX_REPETITIONS = 400
LAST_TIMING = {}


def time_steps(step, steps, warmup, use_graph):
    """Warm up, then time `steps` calls of step(i) on torch's current stream (one HIP graph of the K
    steps unless disabled), repeated: every repetition is bracketed by its own pair of HIP events on
    that stream, the repetitions run back to back, and the MEDIAN over them is reported. A K-step
    replay shorter than the timed window is repeated more often (at least MIN_REPETITIONS times), so
    that a short run is not one sample taken while the device clocks still ramp. A graph of few
    kernels would charge its own launch to them (about 15 us per replay: 0.75 us per step of a
    20-step graph, none of it kernel time), so the K steps are captured `cycles` times over in one
    graph until it holds MIN_GRAPH_STEPS of them - more, up to MAX_GRAPH_STEPS, while a replay stays
    under about GRAPH_WINDOW_MS (judged by the warm-up steps' own time): a run with K = 20 then times
    the same kind of replay as one with K = 2000; a repetition times cycles * K steps and the time per
    step is the replay time over that count.
    Returns (ms per step, graph used, wall seconds); LAST_TIMING holds repetitions / min / max."""
    import torch

    stream = torch.cuda.current_stream()
    warm = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
    warm[0].record(stream)
    for i in range(warmup):
        step(i)
    warm[1].record(stream)
    torch.cuda.synchronize()
    graph = None
    # an upper estimate of a step (plain enqueues carry their launch time): how many fit the window
    estimate_ms = warm[0].elapsed_time(warm[1]) / warmup if warmup > 0 else GRAPH_WINDOW_MS
    wanted = int(min(MAX_GRAPH_STEPS, max(MIN_GRAPH_STEPS, GRAPH_WINDOW_MS / max(estimate_ms, 1e-4))))
    cycles = max(1, -(-wanted // steps)) if use_graph else 1
    if use_graph:
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(steps * cycles):
                    step(i)
            graph.replay()  # one untimed replay
            torch.cuda.synchronize()
        except Exception as exc:  # noqa: BLE001 - report and fall back to plain enqueues
            print(f"HIP graph capture failed ({exc}); timing plain enqueues", file=sys.stderr)
            graph = None
            cycles = 1
            torch.cuda.synchronize()

    def run_once():
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                step(i)

    def timed(repetitions):
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                  for _ in range(repetitions)]
        torch.cuda.synchronize()
        for start, stop in events:
            start.record(stream)
            run_once()
            stop.record(stream)
        torch.cuda.synchronize()
        return [start.elapsed_time(stop) for start, stop in events]

    probe = timed(1)[0]
    repetitions = int(min(MAX_REPETITIONS, max(MIN_REPETITIONS, -(-TIMED_WINDOW_MS // max(probe, 1e-3)))))
    wall0 = time.perf_counter()
    samples = sorted(timed(repetitions))
    wall = time.perf_counter() - wall0
    median = samples[len(samples) // 2] if len(samples) % 2 else 0.5 * (samples[len(samples) // 2 - 1] +
                                                                         samples[len(samples) // 2])
    timed_steps = steps * cycles
    LAST_TIMING.clear()
    LAST_TIMING.update({"repetitions": repetitions, "ms_per_step_min": round(samples[0] / timed_steps, 6),
                        "ms_per_step_max": round(samples[-1] / timed_steps, 6),
                        "timing": f"median of {repetitions} timed replays, one HIP event pair each, of a graph that holds "
                                  f"the {steps} steps {cycles} time(s) over ({timed_steps} launches per replay)"})
    return median / timed_steps, graph is not None, wall


def with_timing(result):
    """Adds the repetition record of the last time_steps() call to a result line."""
    for key in ("repetitions", "ms_per_step_min", "ms_per_step_max"):
        result[key] = LAST_TIMING.get(key)
    result.setdefault("config", {})["timing"] = LAST_TIMING.get("timing")
    return result


def calibrate(args, et):
    """Plain streaming read / copy of the headline weight's size: the bandwidth the device
    delivers to a kernel of that footprint, and the reference for counter calibration."""
    import torch

    device = torch.device("cuda:0")
    nbytes = 14336 * 2304  # the packed Q4_K 14336 x 4096 weight
    copies = 1 if args.hot else -(-ROTATE_BYTES // nbytes)
    buffers = [torch.randint(0, 255, (nbytes,), dtype=torch.uint8, device=device) for _ in range(copies)]
    workgroups = 512
    sink = torch.zeros(4 * workgroups, dtype=torch.int32, device=device)
    dst = torch.empty(nbytes, dtype=torch.uint8, device=device)
    if args.workload == "calibrate_read":
        step = lambda i: et.calibration_read(buffers[i % copies], sink, workgroups)  # noqa: E731
        moved = nbytes
    else:
        step = lambda i: et.calibration_copy(buffers[i % copies], dst)  # noqa: E731
        moved = 2 * nbytes
    ms, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
    gbs = moved / (ms * 1e-3) / 1e9
    print(json.dumps(with_timing({
        "metric": f"{args.workload} GB/s", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": f"{args.workload} of {nbytes} bytes ({'hot' if args.hot else 'cold, %d buffers' % copies})",
                   "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": moved, "avg_launch_us": round(ms * 1e3, 3)},
    })))


def calibrate_read_sweep(args, et):
    """Workload ``calibrate_read_sweep``: plain reads of 8 MiB ... 1 GiB by different read kernels
    (``et_hip_calibration_read_variant``), cold (the buffers of a size rotate through a 2.25 GiB pool),
    each as a HIP-graph replay timed like every other workload; per kernel the launch times are fitted
    to t = t0 + bytes / BW. What this answers: how long a read of the headline weight's 33 MB takes on
    this device whatever kernel does it - the fixed cost t0 of a launch in a dependent chain plus the
    transfer at the rate large reads sustain."""
    import numpy as np
    import torch

    device = torch.device("cuda:0")
    pool_bytes = 2304 << 20
    pool = torch.randint(0, 255, (pool_bytes,), dtype=torch.uint8, device=device)
    sink = torch.zeros(4 * 4096, dtype=torch.int32, device=device)
    headline = 14336 * 2304
    sizes = [8 << 20, 16 << 20, headline, 64 << 20, 128 << 20, 256 << 20, 512 << 20, 1024 << 20]
    if args.sizes_mib:
        sizes = sorted({int(float(m) * (1 << 20)) for m in args.sizes_mib.split(",")} | {headline})
    at_headline = sizes.index(headline)
    # (variant, workgroups): the LDS kernels hold a whole compute unit's LDS, one workgroup each
    kernels = [("plain", 512), ("plain", 2048), ("deep", 512), ("deep", 1024), ("streaming", 1024), ("lds4", 256),
               ("lds8", 256), ("lds8_nt", 256), ("lds8_nt_shallow", 256), ("lds8_nt_ranges", 256),
               ("lds8_nt_ranges_shallow", 256)]
    table, fits = [], []
    for variant, workgroups in kernels:
        times = []
        for size in sizes:
            size -= size % 1024
            copies = max(1, min(pool_bytes // size, -(-ROTATE_BYTES // size)))
            views = [pool[i * size:(i + 1) * size] for i in range(copies)]
            step = lambda i: et.calibration_read_variant(variant, views[i % copies], sink, workgroups)  # noqa: E731
            steps = int(max(copies, min(args.steps, 4e-3 / (size / 4e12))))
            ms, graphed, _ = time_steps(step, steps, min(args.warmup, 2 * copies), not args.no_graph)
            times.append(ms * 1e-3)
            table.append({"kernel": f"{variant} x{workgroups}", "bytes": size, "us": round(ms * 1e3, 3),
                          "GBps": round(size / (ms * 1e-3) / 1e9, 1), "steps": steps, "copies": copies,
                          "repetitions": LAST_TIMING.get("repetitions")})
            print(json.dumps(table[-1]), file=sys.stderr, flush=True)
        slope, t0 = np.polyfit(np.array(sizes, dtype=np.float64), np.array(times), 1)
        fits.append({"kernel": f"{variant} x{workgroups}", "t0_us": round(t0 * 1e6, 3),
                     "BW_GBps": round(1.0 / slope / 1e9, 1),
                     "predicted_us_at_headline_bytes": round((t0 + headline * slope) * 1e6, 3),
                     "measured_us_at_headline_bytes": round(times[at_headline] * 1e6, 3)})
    best = min(fits, key=lambda f: f["measured_us_at_headline_bytes"])
    gbs = headline / (best["measured_us_at_headline_bytes"] * 1e-6) / 1e9
    print(json.dumps({
        "metric": "calibrate_read_sweep GB/s at the headline weight's size", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(best["measured_us_at_headline_bytes"] * 1e-3, 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "calibrate_read_sweep: plain reads of 8 MiB ... 1 GiB by read kernels of eleven launch shapes, cold, "
                               "graph replay; fit t = t0 + bytes / BW per kernel",
                   "best_kernel_at_headline_bytes": best["kernel"], "fits": fits, "table": table},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
    }))


def calibrate_contraction(args, et, synth):
    """Workload ``calibrate_contraction``: the batched Q4_K contraction at 14336 x 4096 (``--vectors`` 32 by
    default, or 7 ... 32) as the operator path launches it, then with its consumers' arithmetic left out,
    with its copies left out, with the weight or the activation copies alone left out, and with only
    the weight or only the activation copies (no arithmetic) - the same waves, waits and barriers every time. Says what bounds the kernel: the path into LDS or the
    instruction stream. ``value`` is the whole kernel's rate."""
    import numpy as np
    import torch

    device = torch.device("cuda:0")
    rows, columns = 14336, 4096
    vectors = args.vectors or 32
    rng = np.random.default_rng(11)
    base = torch.from_numpy(synth.random_weight(synth.Q4_K, rows, columns, rng)).to(device)
    copies = 1 if args.hot else -(-ROTATE_BYTES // base.numel())
    weights = [base] + [torch.roll(base, i, 0).contiguous() for i in range(1, copies)]
    plan = et.RawLinear(et.GgmlQuant.Q4_K, rows, columns, vectors)
    x = torch.randn(vectors, columns, device=device)
    prepared = torch.empty(plan.prepared_input_bytes, dtype=torch.uint8, device=device)
    plan.prepare_input(x, prepared)
    y = torch.empty(vectors, rows, device=device)
    want = torch.empty_like(y)
    plan.enqueue_prepared(prepared, weights[0], None, want, torch.empty(16, dtype=torch.uint8, device=device))
    et.calibration_contraction("whole", plan, weights[0], prepared, y)
    torch.cuda.synchronize()
    assert torch.equal(y, want), "the probe's whole kernel is the operator path's"
    table = {}
    for probe in et.CONTRACTION_PROBES:
        step = lambda i: et.calibration_contraction(probe, plan, weights[i % copies], prepared, y)  # noqa: E731
        ms, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
        table[probe] = round(ms * 1e3, 2)
    moved = base.numel() + vectors * (columns + rows) * 4
    gbs = moved / (table["whole"] * 1e-6) / 1e9
    print(json.dumps(with_timing({
        "metric": "calibrate_contraction GB/s of the whole kernel", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(table["whole"] * 1e-3, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"calibrate_contraction: Q4_K {rows}x{columns}, {vectors} vectors, contraction kernel alone "
                               f"({'hot' if args.hot else 'cold, %d weight buffers' % copies}); us per launch by probe",
                   "us_per_launch": table,
                   "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": moved, "avg_launch_us": table["whole"]},
    })))


def calibrate_mfma(args, et):
    """Loops of one matrix-core instruction that touch no memory (``calibrate_mfma_i8``, ``_i8_scaled``,
    ``_i8_scaled_bf16``, ``_f16``, ``_f16_16x16``): what the matrix cores of this device sustain, next to the published peak.
    ``_i8_scaled`` adds the f32 epilogue of a contraction whose operands both carry a scale per 32
    columns: the ceiling of that arithmetic whatever feeds it. ``_i8_biased`` is the step of the int8
    batch kernel as it runs now; ``_i8_biased_matrix_only`` / ``_i8_biased_valu_only`` are its matrix and
    its VALU instructions alone (rates quoted as if each were the whole step)."""
    import torch

    kind = args.workload[len("calibrate_mfma_"):]
    if kind not in et.MFMA_OPERATIONS:
        sys.exit(f"unknown workload {args.workload}; kinds: {sorted(et.MFMA_OPERATIONS)}")
    device = torch.device("cuda:0")
    # one workgroup of four waves per compute unit and resident wave per SIMD (two by default)
    workgroups, iterations = 256 * max(1, args.waves_per_simd), 2000
    sink = torch.zeros(256 * workgroups, dtype=torch.float32, device=device)
    step = lambda i: et.calibration_mfma(kind, iterations, sink)  # noqa: E731
    ms, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
    torch.cuda.synchronize()
    if kind == "i8_biased_valu_only":  # the sums stay at their starting bits: every element adds 0
        expected = 0.0
    elif kind == "i8_biased_matrix_only":  # only the last step's results are summed: 16 elements of 32 * 0.5
        expected = 256.0
    else:
        expected = {"i8": 32.0, "i8_scaled": 16.0, "i8_scaled_bf16": 16.0, "i8_biased": 16.0, "f16": 16.0,
                    "f16_16x16": 32.0}[kind] * iterations * (16 if kind == "f16_16x16" else 64)
    assert torch.all(sink == expected), (float(sink[0]), expected)
    operations = et.MFMA_OPERATIONS[kind] * 4 * iterations * 4 * workgroups
    tops = operations / (ms * 1e-3) / 1e12
    peak = INT8_PEAK_TOPS if kind.startswith("i8") else F16_PEAK_TFLOPS
    print(json.dumps(with_timing({
        "metric": f"{args.workload} TOP/s", "value": round(tops, 1), "unit": "TOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8" if kind.startswith("i8") else "f16", "data": "synthetic",
        "config": {"workload": f"{args.workload}: {workgroups} workgroups of four waves ({workgroups // 256} per SIMD), {iterations} rounds of four "
                               "independent instructions per wave, no memory traffic",
                   "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues"},
        "roofline": {"bound": "mfma", "achieved": round(tops, 1), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(tops / peak, 4), "traffic": None},
    })))


def make_kv_slabs(torch, kv_dtype, max_tokens, kv_heads, width, device):
    """Random key / value slabs of the given tier: (k_slab, v_slab, k_scales, v_scales, bytes per cached row of a head)."""
    if kv_dtype == "u8":
        slabs = [torch.randint(1, 256, (max_tokens, kv_heads, width), device=device, dtype=torch.uint8) for _ in range(2)]
        scales = [torch.rand(max_tokens, kv_heads, device=device) * 0.02 + 0.005 for _ in range(2)]
        return slabs[0], slabs[1], scales[0], scales[1], width + 4
    dtype = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[kv_dtype]
    slabs = [torch.randn(max_tokens, kv_heads, width, device=device, dtype=dtype) for _ in range(2)]
    return slabs[0], slabs[1], None, None, width * slabs[0].element_size()


def kv_slabs_to_host(np, torch, layer):
    """numpy views of a layer's slabs for the oracle (bfloat16 as its bits)."""
    def host(t):
        return t.view(torch.int16).cpu().numpy().view(np.uint16) if t.dtype == torch.bfloat16 else t.cpu().numpy()
    scales = [t.cpu().numpy() if t is not None else None for t in (layer.k_scales, layer.v_scales)]
    return host(layer.k_slab), host(layer.v_slab), scales[0], scales[1]


def kv_decode(args, et):
    """Workload ``kv_attention_decode``: one decode step of paged key/value-cache attention for a
    Llama-3-8B-shaped layer - 32 slots, 32 query heads over 8 kv heads of width 128, f16 slabs in
    blocks of 16 tokens, 2047 cached positions plus the new one per slot. A step appends the new
    K / V rows and attends (write + attend + merge kernels); the K and V rows every slot reads
    are the algorithmic bytes. Two layers' slabs (2 x 268 MB) alternate so that no step finds its
    rows in the 256 MB Infinity Cache."""
    import numpy as np
    import torch

    device = torch.device("cuda:0")
    torch.manual_seed(7)
    slots, query_heads, kv_heads, width, block, context = 32, 32, 8, 128, 16, args.context
    layers = 1 if args.hot else 2
    rng = np.random.default_rng(7)
    blocks_per_slot = -(-context // block)
    total_blocks = slots * blocks_per_slot
    max_tokens = total_blocks * block
    table_host = rng.permutation(total_blocks).reshape(slots, blocks_per_slot).astype(np.int32)
    cursors_host = np.full(slots, context - 1, dtype=np.int32)
    advances_host = np.ones(slots, dtype=np.int32)
    q_host = rng.standard_normal((slots, query_heads, 1, width)).astype(np.float32)
    k_host = rng.standard_normal((slots, kv_heads, 1, width)).astype(np.float32)
    v_host = rng.standard_normal((slots, kv_heads, 1, width)).astype(np.float32)
    scale = 1.0 / float(np.sqrt(width))
    table = torch.from_numpy(table_host).to(device)
    cursors, advances = torch.from_numpy(cursors_host).to(device), torch.from_numpy(advances_host).to(device)
    q, k, v = (torch.from_numpy(a).to(device) for a in (q_host, k_host, v_host))
    states = []
    for _ in range(layers):
        k_slab, v_slab, k_scales, v_scales, row_bytes = make_kv_slabs(torch, args.kv_dtype, max_tokens, kv_heads,
                                                                      width, device)
        states.append(et.KvLayer(k_slab, v_slab, block, table, cursors, advances, context, k_scales=k_scales,
                                 v_scales=v_scales))
    out = torch.empty_like(q)
    workspace = et.kv_attention_workspace(states[0], query_heads, 1)
    statuses = []

    def step(i):
        statuses.append(et.kv_attention_into(states[i % layers], q, k, v, scale, None, out, workspace=workspace,
                                             synchronize=False))
        if len(statuses) > 4:
            statuses.pop(0)

    # Parity gate before any timing: the first slots against the CPU oracle.
    import oracle
    step(0)
    torch.cuda.synchronize()
    et.kv_attention_status_check(states[0], 1, statuses[-1])
    check = 2
    k_ref, v_ref, ks_ref, vs_ref = kv_slabs_to_host(np, torch, states[0])
    want = oracle.kv_attention(k_ref, v_ref, block, table_host[:check].view(np.uint32),
                               cursors_host[:check].view(np.uint32), advances_host[:check].view(np.uint32),
                               q_host[:check], k_host[:check], v_host[:check], scale, k_scales=ks_ref, v_scales=vs_ref)
    err = float(np.abs(out.cpu().numpy()[:check] - want).max())
    assert err <= 1e-4, f"parity gate failed: max |err| {err:.4g}"

    ms, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
    seconds = ms * 1e-3
    slab_bytes = 2 * slots * context * kv_heads * row_bytes         # K and V rows (and scales) read
    small = 4 * (2 * q.numel() + 2 * k.numel()) + 2 * slots * kv_heads * row_bytes  # q, out, new k / v in, new rows out
    algorithmic = slab_bytes + small
    gbs = algorithmic / seconds / 1e9
    tokens_per_s = slots / seconds
    result = {
        "metric": "kv_attention_decode GB/s", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": f"{args.kv_dtype} slabs, f32 arithmetic", "data": "synthetic",
        "config": {
            "workload": f"kv_attention_decode: {slots} slots x {query_heads} query heads / {kv_heads} kv heads x "
                        f"width {width}, context {context}, {args.kv_dtype} slabs, block {block}",
            "slabs": "hot: one layer" if args.hot else f"cold: alternating over {layers} layers "
                                                       f"({layers * slab_bytes >> 20} MiB)",
            "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues",
            "layer_steps_per_s": round(1.0 / seconds, 1),
            "slot_tokens_per_s_per_layer": round(tokens_per_s, 1),
            "host_wall_ms": round(wall * 1e3, 3),
        },
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic(("kv_attention_decode", context),
                                                 et.kv_attention_kernel(states[0], query_heads, 1))
                     if args.kv_dtype == "f16" else None,
                     "kernel": et.kv_attention_kernel(states[0], query_heads, 1),
                     "algorithmic_bytes_per_launch": algorithmic, "avg_launch_us": round(ms * 1e3, 3)},
    }
    if not args.no_cpu:
        sample = 4
        with pinned_to_one_core() as pin:
            calls, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < args.cpu_seconds or calls == 0:
                oracle.kv_attention(k_ref, v_ref, block, table_host[:sample].view(np.uint32),
                                    cursors_host[:sample].view(np.uint32), advances_host[:sample].view(np.uint32),
                                    q_host[:sample], k_host[:sample], v_host[:sample], scale, k_scales=ks_ref,
                                    v_scales=vs_ref)
                calls += 1
            elapsed = time.perf_counter() - t0
            where = pin.describe()
        per_step = elapsed / calls * (slots / sample)
        result["cpu_baseline"] = {
            "value": round(algorithmic / per_step / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{calls} call(s) over {sample} of the {slots} slots, scaled by {slots // sample}; "
                      f"{elapsed:.1f} s of CPU work; scalar C restatement of the reference's f64 three-pass loop "
                      f"({per_step * 1e3:.0f} ms per step); {where}"}
    print(json.dumps(with_timing(result)))


DECODE_OPS = ("rms_norm_decode", "rotary_decode", "silu_mul_decode", "greedy_decode", "embedding_gather_decode")


def decode_op(args, et):
    """The small operators of one Llama-3-8B-shaped decode step for 32 slots, one launch per step:
    RMS norm of [32, 4096], rotary of q [32, 32, 1, 128] at the slots' cursors, SiLU(gate) * up of
    [32, 14336], greedy tokens of [32, 128256] logits, 32 rows of the f16 [128256, 4096] embedding
    table. Inputs rotate over enough copies to stay out of the caches."""
    import numpy as np
    import torch
    import oracle

    device = torch.device("cuda:0")
    rng = np.random.default_rng(11)
    name = args.workload
    slots = 32

    def copies_for(nbytes):
        return 1 if args.hot else max(2, -(-ROTATE_BYTES // max(nbytes, 1)))

    if name == "rms_norm_decode":
        x = rng.standard_normal((slots, 4096)).astype(np.float32)
        w = rng.standard_normal(4096).astype(np.float32)
        n = min(copies_for(x.nbytes), 64)
        xs = [torch.from_numpy(np.roll(x, i, axis=1)).to(device) for i in range(n)]
        wd, out = torch.from_numpy(w).to(device), torch.empty(slots, 4096, device=device)
        step = lambda i: et.rms_norm_into(xs[i % n], wd, 1e-5, out)  # noqa: E731
        check = lambda: np.abs(out.cpu().numpy() - oracle.rms_norm(np.roll(x, 0, axis=1), w, 1e-5)).max() <= 1e-6  # noqa: E731
        algorithmic = 2 * x.nbytes + w.nbytes
        cpu = lambda: oracle.rms_norm(x, w, 1e-5)  # noqa: E731
        shape = "x [32, 4096] f32, weight [4096]"
    elif name == "rotary_decode":
        x = rng.standard_normal((slots, 32, 1, 128)).astype(np.float32)
        cursors = rng.integers(0, 8192, slots).astype(np.int32)
        n = min(copies_for(x.nbytes), 64)
        xs = [torch.from_numpy(np.roll(x, i, axis=3)).to(device) for i in range(n)]
        od, out = torch.from_numpy(cursors).to(device), torch.empty(x.shape, device=device)
        step = lambda i: et.rotary_into(xs[i % n], od, 500000.0, 1.0, et.RotaryLayout.HALF_SPLIT, out)  # noqa: E731
        check = lambda: np.abs(out.cpu().numpy() - oracle.rotary(x, cursors, 500000.0)).max() <= 1e-6  # noqa: E731
        algorithmic = 2 * x.nbytes + cursors.nbytes
        cpu = lambda: oracle.rotary(x, cursors, 500000.0)  # noqa: E731
        shape = "q [32, 32, 1, 128] f32, theta 5e5, half-split pairs, per-slot offsets"
    elif name == "silu_mul_decode":
        gate = (rng.standard_normal((slots, 14336)) * 3).astype(np.float32)
        up = rng.standard_normal((slots, 14336)).astype(np.float32)
        n = min(copies_for(2 * gate.nbytes), 64)
        gs = [torch.from_numpy(np.roll(gate, i, axis=1)).to(device) for i in range(n)]
        us = [torch.from_numpy(np.roll(up, i, axis=1)).to(device) for i in range(n)]
        out = torch.empty(gate.shape, device=device)
        step = lambda i: et.silu_mul_into(gs[i % n], us[i % n], out)  # noqa: E731
        check = lambda: np.allclose(out.cpu().numpy(), oracle.silu_mul(gate, up), rtol=1e-6, atol=1e-6)  # noqa: E731
        algorithmic = 3 * gate.nbytes
        cpu = lambda: oracle.silu_mul(gate, up)  # noqa: E731
        shape = "gate, up [32, 14336] f32"
    elif name == "greedy_decode":
        logits = rng.standard_normal((slots, 128256)).astype(np.float32)
        n = min(copies_for(logits.nbytes), 48)
        ls = [torch.from_numpy(np.roll(logits, 1000 * i, axis=1)).to(device) for i in range(n)]
        tokens = torch.empty(slots, dtype=torch.int32, device=device)
        status = torch.empty(4 * slots, dtype=torch.uint8, device=device)
        from effect_torch_amd import _native
        from effect_torch_amd.quantized import _Desc
        descs = [_Desc(t) for t in ls]
        scratch = torch.empty(et.greedy_workspace_bytes(slots, 128256), dtype=torch.uint8, device=device)

        def step(i):
            code = _native.lib().et_hip_greedy_tokens_into(descs[i % n].ref, tokens.data_ptr(), scratch.data_ptr(),
                                                           scratch.numel(), status.data_ptr(),
                                                           torch.cuda.current_stream().cuda_stream)
            assert code == 0, _native.last_error()
        check = lambda: np.array_equal(tokens.cpu().numpy(), oracle.argmax_rows(logits).astype(np.int32))  # noqa: E731
        algorithmic = logits.nbytes + 8 * slots
        cpu = lambda: oracle.argmax_rows(logits)  # noqa: E731
        shape = "logits [32, 128256] f32"
    else:
        table = rng.standard_normal((128256, 4096)).astype(np.float16)
        td = torch.from_numpy(table).to(device)
        n = 64
        ids_host = [rng.integers(0, 128256, slots) for _ in range(n)]
        ids = [torch.from_numpy(a.astype(np.int32)).to(device).view(torch.uint32) for a in ids_host]
        out = torch.empty((slots, 4096), dtype=torch.float16, device=device)
        keep = []

        def step(i):
            keep.append(et.gather_rows_into(td, ids[i % n], out, synchronize=False))
            if len(keep) > 4:
                keep.pop(0)
        check = lambda: np.array_equal(out.cpu().numpy().view(np.uint16),  # noqa: E731
                                       oracle.gather_rows(table, ids_host[0]).view(np.uint16))
        algorithmic = 2 * slots * 4096 * 2 + 4 * slots + 8 * slots
        cpu = lambda: oracle.gather_rows(table, ids_host[0])  # noqa: E731
        shape = "32 rows of the f16 [128256, 4096] table"

    step(0)
    torch.cuda.synchronize()
    assert check(), f"parity gate failed for {name}"
    ms, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
    seconds = ms * 1e-3
    gbs = algorithmic / seconds / 1e9
    result = {
        "metric": f"{name} GB/s", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 6), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16" if name == "embedding_gather_decode" else "f32", "data": "synthetic",
        "config": {"workload": f"{name}: {shape}", "inputs": "hot" if args.hot else f"rotating over {n} copies",
                   "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues",
                   "host_wall_ms": round(wall * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": algorithmic, "avg_launch_us": round(ms * 1e3, 3)},
    }
    if not args.no_cpu:
        with pinned_to_one_core() as pin:
            calls, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < min(args.cpu_seconds, 3.0) or calls == 0:
                cpu()
                calls += 1
            elapsed = time.perf_counter() - t0
            where = pin.describe()
        result["cpu_baseline"] = {"value": round(algorithmic / (elapsed / calls) / 1e9, 4), "unit": "GB/s", "cores": 1,
                                  "kind": "port", "sample": f"{calls} full call(s) of the same workload, "
                                  f"{elapsed:.1f} s of CPU work ({elapsed / calls * 1e6:.0f} us per call); {where}"}
    print(json.dumps(with_timing(result)))


def quantized_embedding(args, et):
    """Workload ``quantized_embedding_vocab``: ``embedding_into`` on a vocabulary-sized packed table
    ([128256, 4096] in Q4_K, Q6_K with ``--codec q6_k`` ...): ``--vectors`` token ids (default 8192, a
    prefill chunk of 4 sequences x 2048) are gathered and decoded bit-exactly to f32 rows. The bytes
    that must move: the ids, every selected packed row once, every f32 output row once (the stores
    dominate: 16 384 B written per 2 304 B read for Q4_K)."""
    import numpy as np
    import torch
    import oracle
    from effect_torch_amd import synth

    device = torch.device("cuda:0")
    codec = et.GgmlQuant.from_name(args.codec.upper())
    assert codec is not None, f"unknown codec {args.codec}"
    rows, columns = 128256, 4096
    tokens = args.vectors if args.vectors is not None else 8192
    rng = np.random.default_rng(0xE77C0DE9)
    base_rows = 8192  # distinct random rows; the table repeats them rolled by one row per repeat
    block = synth.random_weight(int(codec), base_rows, columns, rng)
    table_host = np.concatenate([np.roll(block, r, axis=0) for r in range(-(-rows // base_rows))])[:rows]
    table = torch.from_numpy(table_host).to(device)
    n = 1 if args.hot else 8
    ids_host = [rng.integers(0, rows, tokens).astype(np.int64) for _ in range(n)]
    ids = [torch.from_numpy(a).to(device) for a in ids_host]
    outs = [torch.empty((tokens, columns), dtype=torch.float32, device=device) for _ in range(2)]
    plan = et.embedding_requirements(ids[0], table, codec, (rows, columns))
    keep = []

    def step(i):
        keep.append(et.embedding_into(ids[i % n], table, codec, outs[i % 2], plan, synchronize=False))
        if len(keep) > 4:
            keep.pop(0)

    step(0)
    torch.cuda.synchronize()
    et.embedding_status_check(plan, keep[-1])
    sample = min(tokens, 256)
    want = oracle.embedding_into(int(codec), rows, columns, ids_host[0][:sample], table_host)
    got = outs[0][:sample].cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "parity gate failed: decoded rows differ"
    ms, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
    row_bytes = codec.encoded_row_bytes(columns)
    algorithmic = tokens * (8 + row_bytes + 4 * columns)
    gbs = algorithmic / (ms * 1e-3) / 1e9
    result = {
        "metric": "quantized embedding GB/s", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 6), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"quantized_embedding_vocab: {tokens} i64 ids into the {codec.ggml_name} "
                               f"[{rows}, {columns}] table -> f32 [{tokens}, {columns}]",
                   "inputs": "hot" if args.hot else f"rotating over {n} id sets and 2 outputs",
                   "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues",
                   "host_wall_ms": round(wall * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": algorithmic, "avg_launch_us": round(ms * 1e3, 3)},
    }
    if not args.no_cpu:
        cpu_tokens = min(tokens, 512)
        with pinned_to_one_core() as pin:
            calls, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < min(args.cpu_seconds, 5.0) or calls == 0:
                oracle.embedding_into(int(codec), rows, columns, ids_host[0][:cpu_tokens], table_host)
                calls += 1
            elapsed = time.perf_counter() - t0
            where = pin.describe()
        per_token = elapsed / calls / cpu_tokens
        result["cpu_baseline"] = {"value": round((8 + row_bytes + 4 * columns) / per_token / 1e9, 4), "unit": "GB/s",
                                  "cores": 1, "kind": "port",
                                  "sample": f"{calls} call(s) on the first {cpu_tokens} ids, {elapsed:.1f} s of CPU "
                                            f"work ({per_token * 1e6:.1f} us per row); scalar C restatement; {where}"}
    print(json.dumps(with_timing(result)))


def llama_decode(args, et, emit=True):
    """Workload ``llama3_8b_batched_decode`` (the end-to-end batched-decode configuration): greedy decode of
    ``--steps`` tokens (default 128) for 32 sequences of a Llama-3-8B-shaped model from a prefilled context
    of ``--context`` positions (default 2048), every operator through the C ABI (effect_torch_amd.LlamaDecoder):
    per step the lookup of the sequences' tokens in the half-float embedding table, per layer RMS norm (half-
    float weights), the q / k / v / o and gate / up / down contractions on Q4_K weights (M = 32, f32
    activations), rotary on q and k at the sequences' cursors, paged key/value-cache attention over half-float
    slabs in blocks of 16, SiLU * up and the two residual sums; then the final norm, the Q4_K output projection
    to 128256 logits, greedy selection INTO the token buffer the next step reads, and the cursors' advance on
    the device. One step is captured as one HIP graph; the timed region replays it ``--steps`` times - every
    replay is another step, the context grows by one position per step - and the repetitions start from the
    same state. Weights are synthetic (one random matrix per shape, rolled by layer into distinct buffers), the
    prefilled cache is random."""
    import numpy as np
    import torch
    import oracle
    from effect_torch_amd import synth

    device = torch.device("cuda:0")
    torch.manual_seed(0x11A3A)
    steps, warmup = args.steps, min(args.warmup, 8)
    shape = et.LlamaShape(layers=args.layers)
    hidden, heads, kv_heads, width, ffn, vocab = shape.hidden, shape.heads, shape.kv_heads, shape.head_dim, shape.ffn, shape.vocab
    layers, slots, context, block = args.layers, 32, args.context, 16
    max_context = context + max(steps, warmup)
    mode = et.ActivationMode.INT8 if args.mode == "int8" else et.ActivationMode.F32
    rng = np.random.default_rng(0x11A3A)

    shapes = shape.linear_shapes()
    host = {name: synth.random_weight(synth.Q4_K, rows, columns, rng) for name, (rows, columns) in shapes.items()}
    base = {name: torch.from_numpy(w).to(device) for name, w in host.items()}
    weights = [{name: (base[name] if layer == 0 else torch.roll(base[name], layer, 0).contiguous())
                for name in shapes if name != "head"} for layer in range(layers)]
    # random-init norms around 1/16 keep the residual stream of these (far from trained) weights inside the
    # half floats of the slabs over 32 layers; half floats, widened on use
    norms_host = [((1.0 + 0.1 * rng.standard_normal((2, hidden))) / 16.0).astype(np.float16) for _ in range(layers)]
    norms = [torch.from_numpy(n).to(device) for n in norms_host]
    final_norm = torch.from_numpy(((1.0 + 0.1 * rng.standard_normal(hidden)) / 16.0).astype(np.float16)).to(device)
    embedding_base = rng.standard_normal((8192, hidden)).astype(np.float16)  # row t of the table = base[t % 8192]
    embedding = torch.from_numpy(embedding_base).to(device).repeat(-(-vocab // 8192), 1)[:vocab].contiguous()

    blocks_per_slot = -(-max_context // block)
    total_blocks = slots * blocks_per_slot
    table_host = rng.permutation(total_blocks).reshape(slots, blocks_per_slot).astype(np.int32)
    cursors_host = np.full(slots, context, dtype=np.int32)   # `context` positions are cached; the step adds one
    tokens_host = rng.integers(0, vocab, slots).astype(np.int32)
    table, cursors, tokens = (torch.from_numpy(a).to(device) for a in (table_host, cursors_host, tokens_host))
    advances = torch.ones(slots, dtype=torch.int32, device=device)
    kv = []
    for _ in range(layers):
        k_slab, v_slab, k_scales, v_scales, kv_row_bytes = make_kv_slabs(torch, args.kv_dtype, total_blocks * block,
                                                                         kv_heads, width, device)
        kv.append(et.KvLayer(k_slab, v_slab, block, table, cursors, advances, max_context, k_scales=k_scales,
                             v_scales=v_scales))
    decoder = et.LlamaDecoder(shape, et.GgmlQuant.Q4_K, slots, weights, base["head"], norms, final_norm, embedding, kv,
                              tokens, mode=mode, fused=not args.unfused)
    start_cursors, start_tokens = cursors.clone(), tokens.clone()

    def restart():
        """The state every repetition starts from. (The rows the steps append lie behind the prefilled
        context and are written before they are read, so the slabs need no restoring.)"""
        cursors.copy_(start_cursors)
        tokens.copy_(start_tokens)

    # Parity gate: the embedding rows exactly, then layer 0 for two slots against the CPU oracle chained the same way.
    decoder.embed()
    torch.cuda.synchronize()
    x0 = decoder.x.cpu().numpy()[:2].copy()
    assert np.array_equal(x0.view(np.uint32), embedding_base[tokens_host[:2] % 8192].astype(np.float32).view(np.uint32)), \
        "parity gate failed: embedding rows differ"
    decoder.layer_step(0)
    torch.cuda.synchronize()
    et.kv_attention_status_check(kv[0], 1, decoder.status[-1])
    got = decoder.x.cpu().numpy()[:2]
    lin = lambda name, act: oracle.linear_rows(synth.Q4_K, shapes[name][0], shapes[name][1], act, host[name], None, 0,  # noqa: E731
                                               shapes[name][0])
    if args.mode == "int8":
        def lin(name, act):  # noqa: F811
            qa, sa, ta = oracle.quantize_q8(np.ascontiguousarray(act))
            return oracle.linear_q8_rows(synth.Q4_K, shapes[name][0], shapes[name][1], qa, sa, ta, host[name], None, 0,
                                         shapes[name][0])
    norm0 = norms_host[0].astype(np.float32)
    scale = 1.0 / float(np.sqrt(width))
    hh = oracle.rms_norm(x0, norm0[0], 1e-5)
    q_ref = oracle.rotary(lin("wq", hh).reshape(2, heads, 1, width), cursors_host[:2], 500000.0)
    k_ref = oracle.rotary(lin("wk", hh).reshape(2, kv_heads, 1, width), cursors_host[:2], 500000.0)
    v_ref = lin("wv", hh).reshape(2, kv_heads, 1, width)
    # the slabs already hold the rows this very step appended; the oracle writes the same values again
    slabs_host = kv_slabs_to_host(np, torch, kv[0])
    ones = np.ones(2, np.uint32)
    att = oracle.kv_attention(slabs_host[0], slabs_host[1], block, table_host[:2].view(np.uint32),
                              cursors_host[:2].view(np.uint32), ones, q_ref, k_ref, v_ref, scale,
                              k_scales=slabs_host[2], v_scales=slabs_host[3])
    x1 = oracle.add(x0, lin("wo", att.reshape(2, hidden)))
    hh = oracle.rms_norm(x1, norm0[1], 1e-5)
    want = oracle.add(x1, lin("down", oracle.silu_mul(lin("gate", hh), lin("up", hh))))
    relative = float(np.linalg.norm(got - want) / np.linalg.norm(want))
    assert relative <= (2e-2 if args.mode == "int8" else 1e-3), f"parity gate failed: relative L2 error {relative:.3g}"

    restart()
    for _ in range(max(warmup, 1)):
        decoder.step()
    torch.cuda.synchronize()
    et.greedy_status_check(decoder.status[-1])
    restart()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        decoder.step()
    stream = torch.cuda.current_stream()
    repetitions = max(MIN_REPETITIONS, 1)
    samples, finals = [], []
    wall0 = time.perf_counter()
    for _ in range(repetitions + 1):  # the first repetition is not counted
        restart()
        torch.cuda.synchronize()
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(steps):
            graph.replay()
        stop.record(stream)
        torch.cuda.synchronize()
        samples.append(start.elapsed_time(stop))
        finals.append((tokens.cpu().numpy().copy(), cursors.cpu().numpy().copy()))
    wall = time.perf_counter() - wall0
    samples = sorted(samples[1:])
    et.greedy_status_check(decoder.status[-1])
    # every repetition is the same decode: the same last tokens, every cursor at context + steps
    for final_tokens, final_cursors in finals:
        assert np.array_equal(final_cursors, cursors_host + steps), "the cursors did not advance one position per step"
        assert np.array_equal(final_tokens, finals[0][0]), "repetitions of the same decode chose different tokens"
    ms_total = samples[len(samples) // 2]
    ms = ms_total / steps
    seconds = ms * 1e-3
    mean_context = context + (steps - 1) / 2.0 + 1.0  # positions a step attends to, averaged over the steps
    parts = et.algorithmic_bytes_per_step(shape, et.GgmlQuant.Q4_K, slots, layers, 1, kv_row_bytes)
    weight_bytes, logits_bytes = parts["weights"], parts["logits"]
    kv_bytes = int(parts["kv"] * mean_context)
    algorithmic = weight_bytes + kv_bytes + logits_bytes
    gbs = algorithmic / seconds / 1e9
    fused = not args.unfused
    result = {
        "metric": "batched decode tok/s", "value": round(slots / seconds, 1), "unit": "tok/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8" if args.mode == "int8" else "f32", "data": "synthetic",
        "repetitions": repetitions, "ms_per_step_min": round(samples[0] / steps, 4), "ms_per_step_max": round(samples[-1] / steps, 4),
        "config": {"workload": f"llama3_8b_batched_decode: {steps} greedy steps, context {context}->{context + steps - 1} cached "
                               f"positions per sequence, {slots} sequences; {layers} layers, hidden {hidden}, {heads}/{kv_heads} "
                               f"heads x {width}, ffn {ffn}, vocab {vocab}; Q4_K weights, f16 embedding table and norm "
                               f"weights, {args.kv_dtype} kv slabs in blocks of {block}; "
                               f"{'int8' if args.mode == 'int8' else 'f32'} activations",
                   "launch": f"one HIP graph of a whole step, replayed {steps} times per repetition; the chosen tokens and the "
                             "advanced cursors stay on the device between steps",
                   "timing": f"median of {repetitions} repetitions of the whole {steps}-step decode, one HIP event pair each, "
                             "after one uncounted repetition",
                   "operators": "one quantisation per distinct input, residual sums in the contraction epilogues"
                                if fused else "one launch sequence per operator",
                   "weight_bytes": weight_bytes, "kv_bytes_read_per_step_mean": kv_bytes,
                   "layer0_relative_l2_error": relative, "host_wall_ms": round(wall * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": algorithmic, "avg_launch_us": round(ms * 1e3, 1)},
    }
    if not args.no_cpu:
        # one layer for one slot and 2048 rows of the output projection on one core, scaled to the step
        with pinned_to_one_core() as pin:
            t0 = time.perf_counter()
            one = x0[:1]
            hh = oracle.rms_norm(one, norm0[0], 1e-5)
            q1 = oracle.rotary(lin("wq", hh).reshape(1, heads, 1, width), cursors_host[:1], 500000.0)
            k1 = oracle.rotary(lin("wk", hh).reshape(1, kv_heads, 1, width), cursors_host[:1], 500000.0)
            v1 = lin("wv", hh).reshape(1, kv_heads, 1, width)
            a1 = oracle.kv_attention(slabs_host[0], slabs_host[1], block,
                                     table_host[:1].view(np.uint32), cursors_host[:1].view(np.uint32),
                                     ones[:1], q1, k1, v1, scale, k_scales=slabs_host[2], v_scales=slabs_host[3])
            y1 = oracle.add(one, lin("wo", a1.reshape(1, hidden)))
            hh = oracle.rms_norm(y1, norm0[1], 1e-5)
            oracle.add(y1, lin("down", oracle.silu_mul(lin("gate", hh), lin("up", hh))))
            t1 = time.perf_counter()
            oracle.linear_rows(synth.Q4_K, vocab, hidden, hh, host["head"], None, 0, 2048)
            t2 = time.perf_counter()
            pinned = pin.describe()
        per_token = (t1 - t0) * layers + (t2 - t1) * vocab / 2048
        result["cpu_baseline"] = {"value": round(1.0 / per_token, 4), "unit": "tok/s", "cores": 1, "kind": "port",
                                  "sample": f"one layer for one slot at context {context} ({t1 - t0:.2f} s) x {layers} "
                                            f"layers + 2048 of {vocab} output rows ({t2 - t1:.2f} s) scaled; scalar C "
                                            f"restatement of the reference's loops ({per_token:.1f} s per token); {pinned}"}
    if emit:
        print(json.dumps(result))
    return result


def decode_leg(args, et):
    """The metric's second half next to the headline: the 128-step greedy batched decode of ``llama_decode`` run
    in the same process (its own parity gate first, no CPU leg), reduced to the figures of one object."""
    import gc
    import torch
    leg = argparse.Namespace(**vars(args))
    leg.steps, leg.warmup, leg.mode, leg.no_cpu, leg.unfused = 128, 8, "f32", True, False
    leg.layers, leg.context, leg.kv_dtype = 32, 2048, "f16"
    t0 = time.perf_counter()
    try:
        full = llama_decode(leg, et, emit=False)
    except Exception as error:  # the headline line is printed whatever happens here
        return {"error": f"{type(error).__name__}: {error}"}
    finally:
        gc.collect()
        torch.cuda.empty_cache()
    roofline = full["roofline"]
    return {"metric": full["metric"], "value": full["value"], "unit": full["unit"], "steps": full["steps"],
            "ms_per_step": full["ms_per_step"], "ms_per_step_min": full["ms_per_step_min"],
            "ms_per_step_max": full["ms_per_step_max"], "repetitions": full["repetitions"], "dtype": full["dtype"],
            "algorithmic_bytes": roofline["algorithmic_bytes_per_launch"], "achieved_gbs": roofline["achieved"],
            "frac": roofline["frac"], "workload": full["config"]["workload"], "launch": full["config"]["launch"],
            "timing": full["config"]["timing"],
            "layer0_relative_l2_error": full["config"]["layer0_relative_l2_error"],
            "leg_wall_s": round(time.perf_counter() - t0, 1)}


BASELINE_CONFIGS = [
    # (BASELINE.json config, arguments after `python bench.py`)
    ("0: Q8_0 4096x4096, M=1", ["--workload", "q8_0_gemv_4096x4096", "--vectors", "1"]),
    ("1: Q4_0 11008x4096, M=1", ["--workload", "q4_0_gemv_11008x4096", "--vectors", "1"]),
    ("1: Q4_0 11008x4096, M=4", ["--workload", "q4_0_gemv_11008x4096", "--vectors", "4"]),
    ("1: Q4_0 11008x4096, M=8", ["--workload", "q4_0_gemv_11008x4096", "--vectors", "8"]),
    ("2: Q4_K 14336x4096, M=1 (headline)", ["--workload", "q4_k_gemv_14336x4096", "--vectors", "1"]),
    ("2: Q4_K 14336x4096, M=16", ["--workload", "q4_k_gemv_14336x4096", "--vectors", "16"]),
    ("2: Q4_K 14336x4096, M=64", ["--workload", "q4_k_gemv_14336x4096", "--vectors", "64"]),
    ("3: Q8_0 4096x14336, M=512, int8 activations", ["--workload", "q8_0_gemm_i8_512x14336x4096", "--vectors", "512"]),
    ("4: Llama-3-8B-shaped batched decode, 32 x 2048, 128 steps", ["--workload", "llama3_8b_batched_decode"]),
    ("f-1: paged KV attention, 32 slots, context 2048, f16", ["--workload", "kv_attention_decode"]),
]


def baseline_configs(args):
    """Workload ``baseline_configs``: every BASELINE configuration (and the attention kernel) as the driver
    would run it - one ``python bench.py ... --steps 20 --warmup 5 --no-cpu`` process each, one after the
    other - gathered into one markdown table (stdout) with the JSON lines behind it; what
    ``profiles/baseline_configs.md`` is made from."""
    import hashlib
    import subprocess

    lines, table = [], []
    for label, extra in BASELINE_CONFIGS:
        decode = "llama3" in extra[1]
        command = [sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--no-cpu", "--no-decode"] + extra
        if not decode:
            command += ["--steps", "20", "--warmup", "5"]
        done = subprocess.run(command, capture_output=True, text=True, timeout=600)
        text = [line for line in done.stdout.splitlines() if line.startswith("{")]
        if done.returncode != 0 or not text:
            table.append(f"| {label} | failed (exit {done.returncode}) | | | | |")
            continue
        result = json.loads(text[-1])
        lines.append(text[-1])
        roofline = result["roofline"]
        unit = roofline.get("unit", "")
        kernel = roofline.get("kernel", "")
        table.append(f"| {label} | `{' '.join(extra)}` | {kernel} | {result['ms_per_step'] * 1e3:.2f} "
                     f"({(result.get('ms_per_step_min') or 0) * 1e3:.2f} - {(result.get('ms_per_step_max') or 0) * 1e3:.2f}) | "
                     f"{result['value']} {result['unit']} | {roofline['achieved']} {unit} = {roofline['frac']:.4f} of {roofline['peak']:g} |")
    sources = sorted(name for name in os.listdir(os.path.join(ROOT, "effect-torch_amd", "csrc")) if name.endswith(".hip"))
    digest = hashlib.sha256()
    for name in sources:
        with open(os.path.join(ROOT, "effect-torch_amd", "csrc", name), "rb") as source:
            digest.update(source.read())
    print("| BASELINE config | arguments (after `python bench.py --gpus 1 --no-cpu --no-decode`, plus `--steps 20 --warmup 5`) | kernel | us per step (min - max of the timed replays) | value | roofline |")
    print("|---|---|---|---|---|---|")
    print("\n".join(table))
    print(f"\nSHA-256 over the kernel sources (effect-torch_amd/csrc/*.hip, in name order): {digest.hexdigest()}; {cpu_model()}\n")
    for line in lines:
        print(line)


def gguf_upload(args, et):
    """Workload ``gguf_upload``: a synthetic GGUF v3 file with the tensor catalog of a Llama-3-8B Q4_K
    model (291 tensors; ``--layers`` of them carry payloads, the default 4 make a 0.5 GB file) is
    written to a temporary directory, parsed, and every tensor is uploaded into device memory. A step
    = the upload of the whole file; the parse is timed separately. Bound by the host side (page cache
    read + pinned staging + PCIe), not by HBM."""
    import struct
    import tempfile
    import numpy as np
    import torch
    from effect_torch_amd import synth

    device = torch.device("cuda:0")
    layers = min(args.layers, 32)
    rng = np.random.default_rng(5)
    hidden, kv, ffn, vocab = 4096, 1024, 14336, 128256

    def gstr(text):
        raw = text.encode()
        return struct.pack("<Q", len(raw)) + raw

    catalog = [("token_embd.weight", (hidden, vocab), 12)]
    for i in range(layers):
        catalog += [(f"blk.{i}.attn_norm.weight", (hidden,), 0), (f"blk.{i}.attn_q.weight", (hidden, hidden), 12),
                    (f"blk.{i}.attn_k.weight", (hidden, kv), 12), (f"blk.{i}.attn_v.weight", (hidden, kv), 12),
                    (f"blk.{i}.attn_output.weight", (hidden, hidden), 12), (f"blk.{i}.ffn_norm.weight", (hidden,), 0),
                    (f"blk.{i}.ffn_gate.weight", (hidden, ffn), 12), (f"blk.{i}.ffn_up.weight", (hidden, ffn), 12),
                    (f"blk.{i}.ffn_down.weight", (ffn, hidden), 12)]
    catalog += [("output_norm.weight", (hidden,), 0)]
    sizes = [(int(np.prod(d)) * 4 if code == 0 else int(np.prod(d)) // 256 * 144) for _, d, code in catalog]
    offsets, cursor = [], 0
    for size in sizes:
        offsets.append(cursor)
        cursor = -(-(cursor + size) // 32) * 32
    vocabulary = [f"token{i}" for i in range(vocab)]
    meta = [gstr("general.architecture") + struct.pack("<I", 8) + gstr("llama"),
            gstr("general.quantization_version") + struct.pack("<II", 4, 2),
            gstr("llama.block_count") + struct.pack("<II", 4, layers),
            gstr("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, vocab) + b"".join(gstr(t) for t in vocabulary)]
    head = b"GGUF" + struct.pack("<IQQ", 3, len(catalog), len(meta)) + b"".join(meta)
    for (name, dims, code), offset in zip(catalog, offsets):
        head += gstr(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", code, offset)
    head += b"\0" * (-len(head) % 32)
    block = rng.integers(0, 256, 64 << 20, dtype=np.uint8).tobytes()
    with tempfile.TemporaryDirectory() as folder:
        path = os.path.join(folder, "model.gguf")
        with open(path, "wb") as out:
            out.write(head)
            written = 0
            while written < cursor:
                piece = block[: min(len(block), cursor - written)]
                out.write(piece)
                written += len(piece)
        file_bytes = len(head) + cursor
        import ctypes
        from effect_torch_amd import _native
        handle = ctypes.c_void_p()
        t0 = time.perf_counter()
        assert _native.lib().et_hip_gguf_open(path.encode(), None, ctypes.byref(handle)) == 0, _native.last_error()
        parse_seconds = time.perf_counter() - t0
        _native.lib().et_hip_gguf_close(handle)
        model = et.GgufFile.open(path)
        assert len(model.tensors) == len(catalog) and model.get("tokenizer.ggml.tokens").value[5] == "token5"
        buffers = {t.name: torch.empty(t.physical_shape if t.format else t.logical_shape,
                                       dtype=torch.uint8 if t.format else torch.float32, device=device)
                   for t in model.tensors}

        def step():
            for t in model.tensors:
                model.upload_tensor(t.name, device, buffers[t.name])

        step()
        probe = model.tensors[2]
        assert np.array_equal(buffers[probe.name].cpu().numpy().reshape(-1),
                              np.frombuffer(model.read_tensor(probe.name).tobytes(), dtype=np.uint8))
        for _ in range(max(args.warmup, 0)):
            step()
        torch.cuda.synchronize()
        steps = max(1, min(args.steps, 5))
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        seconds = (time.perf_counter() - t0) / steps
        t0 = time.perf_counter()
        host = np.empty(max(sizes), dtype=np.uint8)
        for t in model.tensors:
            model.read_tensor(t.name, host[: t.byte_len])
        read_seconds = time.perf_counter() - t0
        model.close()
    gbs = cursor / seconds / 1e9
    print(json.dumps({
        "metric": "gguf_upload GB/s", "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": steps,
        "warmup": args.warmup, "ms_per_step": round(seconds * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": f"gguf_upload: {len(catalog)} tensors of a Llama-3-8B Q4_K catalog ({layers} layers), "
                               f"{file_bytes} file bytes, vocabulary of {vocab} strings in the metadata",
                   "parse_ms": round(parse_seconds * 1e3, 3), "host_read_GBps": round(cursor / read_seconds / 1e9, 2),
                   "path": "page cache -> 2 x 8 MiB pinned staging -> hipMemcpyAsync -> HBM"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 5), "traffic": None,
                     "note": "bound by the host link and the file read, not by HBM",
                     "algorithmic_bytes_per_launch": cursor, "avg_launch_us": round(seconds * 1e6, 1)},
        "cpu_baseline": {"value": round(cursor / read_seconds / 1e9, 2), "unit": "GB/s", "cores": 1, "kind": "port",
                         "sample": "the same tensors read into host memory (read_gguf_tensor_into), one pass"},
    }))


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)

    if args.workload == "baseline_configs":
        return baseline_configs(args)

    import numpy as np
    import torch
    import __graft_entry__ as entry

    et = entry.load_package()
    from effect_torch_amd import synth

    if args.workload in ("calibrate_read", "calibrate_copy"):
        return calibrate(args, et)
    if args.workload == "calibrate_read_sweep":
        return calibrate_read_sweep(args, et)
    if args.workload.startswith("calibrate_mfma_"):
        return calibrate_mfma(args, et)
    if args.workload == "calibrate_contraction":
        return calibrate_contraction(args, et, synth)
    if args.workload in DECODE_OPS:
        assert torch.cuda.is_available() and et.is_available(), "bench.py needs a gfx950 GPU"
        return decode_op(args, et)
    if args.workload == "gguf_upload":
        assert torch.cuda.is_available() and et.is_available(), "bench.py needs a gfx950 GPU"
        if args.layers == 32:
            args.layers = 4
        return gguf_upload(args, et)
    if args.workload == "llama3_8b_batched_decode":
        assert torch.cuda.is_available() and et.is_available(), "bench.py needs a gfx950 GPU"
        return llama_decode(args, et)
    if args.workload == "kv_attention_decode":
        assert torch.cuda.is_available() and et.is_available(), "bench.py needs a gfx950 GPU"
        return kv_decode(args, et)
    if args.workload == "quantized_embedding_vocab":
        assert torch.cuda.is_available() and et.is_available(), "bench.py needs a gfx950 GPU"
        return quantized_embedding(args, et)
    if args.workload not in synth.CONFIGS:
        sys.exit(f"unknown workload {args.workload}; choose from {sorted(synth.CONFIGS)} "
                 "or calibrate_read / calibrate_copy / kv_attention_decode / llama3_8b_batched_decode / gguf_upload / "
                 "quantized_embedding_vocab / " + " / ".join(DECODE_OPS))
    cfg = synth.CONFIGS[args.workload]
    vectors = args.vectors if args.vectors is not None else cfg["vectors"][0]
    mode_name = args.mode or ("int8" if "i8" in args.workload else "f32")
    mode = et.ActivationMode.INT8 if mode_name == "int8" else et.ActivationMode.F32
    codec = et.GgmlQuant(cfg["codec"])
    rows, columns = cfg["rows"], cfg["columns"]

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    assert et.is_available(), "the visible GPU is not gfx950"
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    rng = np.random.default_rng(cfg["seed"])
    weight_host = synth.random_weight(cfg["codec"], rows, columns, rng)
    x_host = synth.random_activations(vectors, columns, rng, cfg["x_scale"])
    weight_bytes = weight_host.size

    copies = 1 if args.hot else max(2, -(-ROTATE_BYTES // weight_bytes))
    base = torch.from_numpy(weight_host).to(device)
    weights = [base]
    for i in range(1, copies):
        # Distinct buffers with distinct contents (rows rolled by i), same distribution.
        weights.append(torch.roll(base, shifts=i, dims=0).contiguous())
    x = torch.from_numpy(x_host).to(device)
    ys = [torch.empty((vectors, rows), dtype=torch.float32, device=device) for _ in range(min(copies, 4))]

    linear = et.RawLinear(codec, rows, columns, vectors, False, mode)
    req = linear.requirements
    workspace = (torch.empty(req.workspace_bytes, dtype=torch.uint8, device=device)
                 if req.workspace_bytes else None)
    algorithmic_bytes = req.algorithmic_bytes

    def step(i):
        linear.enqueue(x, weights[i % copies], None, ys[i % len(ys)], workspace)

    # Parity gate before any timing: the first buffer against the CPU oracle on a row range.
    import oracle
    step(0)
    torch.cuda.synchronize()
    check_rows = min(rows, 256)
    got = ys[0].cpu().numpy()[:, :check_rows]
    if mode_name == "int8":
        q, s, t = oracle.quantize_q8(x_host)
        want = oracle.linear_q8_rows(cfg["codec"], rows, columns, q, s, t, weight_host, None, 0, check_rows)
    else:
        want = oracle.linear_rows(cfg["codec"], rows, columns, x_host, weight_host, None, 0, check_rows)
    want = want[:, :check_rows]
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    err = np.abs(got.astype(np.float64) - want)
    assert np.all(err <= 1e-3 * np.maximum(np.abs(want), 1.0) + 4e-5 * rms), \
        f"parity gate failed: max |err| {err.max():.4g}"

    ms_per_step, graphed, wall = time_steps(step, args.steps, args.warmup, not args.no_graph)
    seconds_per_step = ms_per_step * 1e-3

    gbs = algorithmic_bytes / seconds_per_step / 1e9
    ops = 2.0 * vectors * rows * columns
    if mode_name == "int8" and vectors >= 256:
        roofline = {"bound": "mfma", "achieved": round(ops / seconds_per_step / 1e12, 3),
                    "peak": INT8_PEAK_TOPS, "unit": "TFLOP/s",
                    "frac": round(ops / seconds_per_step / 1e12 / INT8_PEAK_TOPS, 4), "traffic": None}
    else:
        roofline = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None}
    roofline["traffic"] = measured_traffic((args.workload, vectors, mode_name), req.kernel)
    roofline["kernel"] = req.kernel
    roofline["algorithmic_bytes_per_launch"] = algorithmic_bytes
    roofline["avg_launch_us"] = round(ms_per_step * 1e3, 3)

    result = {
        "metric": "Q4_K dequant-GEMV HBM GB/s (% peak) at 14336x4096; batched decode tok/s"
                  if args.workload == "q4_k_gemv_14336x4096" else f"{args.workload} GB/s",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if mode_name == "int8" else "f32",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload} M={vectors} ({codec.ggml_name} W {rows}x{columns}, {mode_name} activations)",
            "weights": "hot: one buffer, cache resident" if args.hot else
                       f"cold: rotating over {copies} distinct weight buffers ({copies * weight_bytes >> 20} MiB)",
            "launch": "hipgraph replay of the K steps" if graphed else "K plain enqueues",
            "percent_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
            "host_wall_ms": round(wall * 1e3, 3),
        },
        "roofline": roofline,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg, vectors, mode_name, weight_host, x_host,
                                              args.cpu_seconds, algorithmic_bytes)
    result = with_timing(result)
    if args.workload == "q4_k_gemv_14336x4096" and vectors == 1 and mode_name == "f32" and not args.hot and not args.no_decode:
        # "...; batched decode tok/s": the end-to-end configuration, measured after the headline with its buffers freed
        del weights, base, ys, x, workspace
        torch.cuda.empty_cache()
        result["decode"] = decode_leg(args, et)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
