"""Streams and HIP-graph capture: every entry point enqueues on the stream it is given and is capturable
(the reference tests both for its launcher: test/test_stream.py:28-37, test/test_cudagraph.py:17-63)."""
import numpy as np
import pytest
import torch

from mxutil import oracle_matmul, randn_operand
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu


def _mm(ct, a, b, **kw):
    return ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, a_format=a.fmt_kw,
                                  b_format=b.fmt_kw, **kw)


@pytest.mark.parametrize("kernel", ["mfma128", "pingpong", "generic"])
def test_launch_on_a_side_stream(ct, dev, kernel):
    """The work goes to the current stream, not the null stream: three calls are enqueued on a side stream and
    the result is read after synchronising that stream alone."""
    a = randn_operand(512, 1024, O.E4M3, 201, dev)
    b = randn_operand(768, 1024, O.E4M3, 202, dev)
    want = _mm(ct, a, b, kernel=kernel)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)
    c = torch.zeros_like(want)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for _ in range(3):
            _mm(ct, a, b, kernel=kernel, C=c)
    side.synchronize()
    assert torch.equal(c, want)
    err = O.rel_fro(c.cpu(), oracle_matmul(a, b))
    assert err <= 1e-3


@pytest.mark.parametrize("shape,kernel,fa,fb", [((512, 768, 1024), "mfma128", O.E4M3, O.E4M3),
                                               ((3072, 3072, 1024), "pingpong", O.E4M3, O.E4M3),
                                               ((3072, 3072, 1024), "auto", O.E2M1, O.E2M1),
                                               ((32, 1024, 4096), "auto", O.E4M3, O.E2M1),
                                               ((64, 256, 8192), "auto", O.E4M3, O.E4M3)])
def test_graph_capture_and_replay(ct, dev, shape, kernel, fa, fb):
    """test/test_cudagraph.py:40-63: capture one call with a preallocated output (scale re-layout, split-K
    partials and the decode kernel included), replay it three times with eager work of the same library and
    synchronisations in between, and compare every replay bit for bit with the eager result.  The inputs
    change between replays (same buffers, new contents), so a replay that did not run would be caught."""
    M, N, K = shape
    a = randn_operand(M, K, fa, 211, dev)
    b = randn_operand(N, K, fb, 212, dev)
    c = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    _mm(ct, a, b, kernel=kernel, C=c)          # warm-up outside the capture (kernel attributes, workspace)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _mm(ct, a, b, kernel=kernel, C=c)
    for rep in range(3):
        a2 = randn_operand(M, K, fa, 300 + rep, dev)
        a.storage.copy_(a2.storage)
        a.scale_t.copy_(a2.scale_t)
        want = _mm(ct, a, b, kernel=kernel, out_dtype=torch.bfloat16)     # eager, between the replays
        other = randn_operand(256, 512, O.E4M3, 400 + rep, dev)
        _mm(ct, other, other)                                             # eager work that uses the cached workspace
        torch.cuda.synchronize()
        c.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(c.view(torch.int16), want.view(torch.int16)), f"replay {rep}"
        if rep == 0:
            ref = O.reference_matmul(a2.codes, a2.scales, np.ascontiguousarray(b.codes.T),
                                     np.ascontiguousarray(b.scales.T), fa, fb)
            assert O.rel_fro(c.float().cpu(), ref) <= 8e-3


def test_bench_entry_point(ct, dev):
    """mx_bench_gemm (the counterpart of the reference launcher's _benchmark, cext/tile_kernel.cpp:3921-4042):
    per-call durations are positive and plausible, operand sets rotate, results are the ordinary ones."""
    sets = []
    for i in range(3):
        a = randn_operand(1024, 1024, O.E4M3, 500 + i, dev)
        b = randn_operand(1024, 1024, O.E4M3, 510 + i, dev)
        sets.append((a, b, torch.zeros((1024, 1024), dtype=torch.float32, device=dev)))
    times = ct.bench_block_scaled_matmul([(a.storage, a.scale_t, b.storage.T, b.scale_t.T, c) for a, b, c in sets],
                                         warmup=2, iters=9)
    assert len(times) == 9 and all(0.001 < t < 50.0 for t in times), times
    for a, b, c in sets:
        assert torch.equal(c, _mm(ct, a, b))
