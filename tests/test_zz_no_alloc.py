"""The entry point that allocates nothing: et_hip_linear_enqueue_static_workspace against
et_hip_linear_enqueue, through the C ABI.

The batch kernels need scratch memory (activation tiles, K-share partials); the existing entry point
takes it from the caller, the new one from a device array inside the library. Same kernels, same
bytes: the results must be bit-identical. Two calls in a row, the second with a smaller input, so
that what the first call left in the array cannot show in the second one's result.
"""
import numpy as np
import pytest
import torch

import oracle
from effect_torch_amd import synth
from test_gpu_parity import close

pytestmark = pytest.mark.gpu


def both_ways(et, device, codec, rows, columns, vectors, mode, rng, with_bias):
    weight_host = synth.random_weight(codec, rows, columns, rng)
    x_host = synth.random_activations(vectors, columns, rng, 0.5)
    bias_host = rng.standard_normal(rows).astype(np.float32) if with_bias else None
    weight = torch.from_numpy(weight_host).to(device)
    x = torch.from_numpy(x_host).to(device)
    bias = torch.from_numpy(bias_host).to(device) if with_bias else None
    plan = et.RawLinear(et.GgmlQuant(codec), rows, columns, vectors, with_bias, mode)
    need = plan.requirements.workspace_bytes
    assert 0 < need <= et.STATIC_WORKSPACE_BYTES, need  # a kernel with a scratch buffer, inside the limit
    workspace = torch.empty(need, dtype=torch.uint8, device=device)
    mine = torch.full((vectors, rows), float("nan"), device=device)
    theirs = torch.full((vectors, rows), float("nan"), device=device)
    plan.enqueue(x, weight, bias, theirs, workspace)
    plan.enqueue_static_workspace(x, weight, bias, mine)
    torch.cuda.synchronize()
    assert torch.equal(mine, theirs), "the static workspace changed the result"
    return mine.cpu().numpy(), x_host, weight_host, bias_host


def test_static_workspace_entry_point_matches_the_workspace_one(et, device):
    rng = np.random.default_rng(20)
    F32, INT8 = et.ActivationMode.F32, et.ActivationMode.INT8
    # first a large call (K shares, 2 MiB of tiles and partials), then a smaller one of another shape
    got, x, w, b = both_ways(et, device, oracle.Q4_K, 4096, 14336, 32, F32, rng, False)
    want = oracle.linear_rows(oracle.Q4_K, 4096, 14336, x, w, b, 0, 128)[:, :128]
    close(got[:, :128], want)
    got, x, w, b = both_ways(et, device, oracle.Q4_K, 1000, 1024, 9, F32, rng, True)
    close(got, oracle.linear_into(oracle.Q4_K, 1000, 1024, x, w, b))
    # the int8-activation mode and a 32-wide codec, smaller again
    got, x, w, b = both_ways(et, device, oracle.Q8_0, 200, 512, 40, INT8, rng, True)
    q, scale, total = oracle.quantize_q8(x)
    close(got, oracle.linear_q8_rows(oracle.Q8_0, 200, 512, q, scale, total, w, b))
    # and the first shape once more: the array now holds the leftovers of three other calls
    both_ways(et, device, oracle.Q4_K, 4096, 14336, 32, F32, rng, False)


def test_static_workspace_entry_point_under_stream_capture(et, device):
    # What the entry point is for: a caller that records the call into a graph. The plan is made before the
    # capture (that is when the library looks up the array's device address); the recorded call then
    # allocates nothing - device memory in use is the same after it - and every replay, with eager work
    # and synchronisations in between, gives the eager result.
    rng = np.random.default_rng(22)
    codec, rows, columns, vectors = oracle.Q4_K, 4096, 4096, 32
    weight = torch.from_numpy(synth.random_weight(codec, rows, columns, rng)).to(device)
    x = torch.from_numpy(synth.random_activations(vectors, columns, rng)).to(device)
    plan = et.RawLinear(et.GgmlQuant(codec), rows, columns, vectors)
    assert 0 < plan.requirements.workspace_bytes <= et.STATIC_WORKSPACE_BYTES
    eager = torch.empty((vectors, rows), device=device)
    plan.enqueue_static_workspace(x, weight, None, eager)  # warm-up, and the result to compare with
    torch.cuda.synchronize()
    out = torch.full((vectors, rows), float("nan"), device=device)
    free_before = torch.cuda.mem_get_info()[0]
    plan.enqueue_static_workspace(x, weight, None, out)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # nothing was allocated
    assert torch.equal(out, eager)
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            plan.enqueue_static_workspace(x, weight, None, out)
    for replay in range(3):
        out.fill_(float("nan"))
        other = torch.empty((9, 1000), device=device)  # eager work in between, on the same array
        small = et.RawLinear(et.GgmlQuant(codec), 1000, columns, 9)
        small.enqueue_static_workspace(x[:9], weight[:1000], None, other)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"


def test_static_workspace_entry_point_refuses_what_does_not_fit(et, device):
    # 2048 vectors of 14336 columns need 120 MiB of tiles: more than the array holds
    plan = et.RawLinear(et.GgmlQuant.Q4_K, 256, 14336, 2048)
    assert plan.requirements.workspace_bytes > et.STATIC_WORKSPACE_BYTES
    x = torch.zeros((2048, 14336), device=device)
    weight = torch.zeros((256, 8064), dtype=torch.uint8, device=device)
    y = torch.zeros((2048, 256), device=device)
    with pytest.raises(et.QuantizedError, match="the static workspace holds 16777216"):
        plan.enqueue_static_workspace(x, weight, None, y)
    # a GEMV plan (whose only scratch is the dense copy of strided input rows) runs through it just the same
    small = et.RawLinear(et.GgmlQuant.Q4_K, 300, 512, 1)
    assert small.requirements.kernel.startswith("gemv")
    rng = np.random.default_rng(21)
    w = synth.random_weight(oracle.Q4_K, 300, 512, rng)
    xs = synth.random_activations(1, 512, rng)
    out = torch.empty((1, 300), device=device)
    small.enqueue_static_workspace(torch.from_numpy(xs).to(device), torch.from_numpy(w).to(device), None, out)
    close(out.cpu().numpy(), oracle.linear_into(oracle.Q4_K, 300, 512, xs, w))
