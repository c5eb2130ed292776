"""mx_gemm_static, the entry point that allocates nothing: its results against mx_gemm's (caller-owned
workspace) through the C ABI, bit for bit, on calls in a row that share the library's static scratch buffer."""
import ctypes

import pytest
import torch

from cutile_amd import _lib as L
from cutile_amd.ops import _gemm_descs, _opts
from mxutil import oracle_matmul, randn_operand
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu


def _both(ct, dev, a, b, out_dtype, kernel="auto", split_k=0, fill=None):
    """(result of mx_gemm_static, result of mx_gemm) for A [M, K] x B [N, K]^T, both called through ctypes."""
    lib = ct.lib()
    stream = L.stream_ptr(dev)
    outs = []
    for static in (True, False):
        c = torch.full((a.rows, b.rows), float("nan"), dtype=out_dtype, device=dev)
        a_pd = 1 if a.fmt == O.E2M1 else -1
        b_pd = 0 if b.fmt == O.E2M1 else -1
        descs, (la, lb), (M, N, K) = _gemm_descs(a.storage, a.fmt, a_pd, a.scale_t, b.storage.T, b.fmt, b_pd,
                                                 b.scale_t.T, c, 32)
        o = _opts(False, la, lb, kernel, 32, split_k)
        refs = [ctypes.byref(d) for d in descs]
        if static:
            if fill is not None:          # the scratch keeps the previous call's contents: make them hostile
                fill()
            rc = lib.mx_gemm_static(*refs, ctypes.byref(o), stream)
        else:
            need = lib.mx_gemm_workspace_bytes(M, N, K, ctypes.byref(o))
            ws = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
            rc = lib.mx_gemm(*refs, ctypes.byref(o), ws.data_ptr(), need, stream)
        assert rc == 0, L.last_error()
        torch.cuda.synchronize()
        outs.append(c)
    return outs


def _hostile_scratch(ct, dev):
    """Leaves NaN everywhere a later call could read the static scratch: static calls whose scale bytes are all
    0xFF (re-laid scales of 0xFF, then split-K partial products that are NaN)."""
    def nan_operand(rows, K):
        q = torch.zeros((rows, K), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
        s = torch.full((rows, K // 32), 0xFF, dtype=torch.uint8, device=dev).view(torch.float8_e8m0fnu)
        return q, s
    for (m, n, k), split in (((4096, 4096, 4096), 0), ((64, 256, 8192), 4)):
        a_q, a_s = nan_operand(m, k)
        b_q, b_s = nan_operand(n, k)
        c = ct.block_scaled_matmul(a_q, a_s, b_q.T, b_s.T, static_scratch=True, split_k=split)
        assert torch.isnan(c).all()


def test_static_scratch_matches_workspace_entry_point(ct, dev):
    assert ct.lib().mx_static_scratch_bytes() == 8 << 20
    hostile = lambda: _hostile_scratch(ct, dev)
    # first call: 4 x 4 tiles of 256 x 256 ... a large re-layout that fills a good part of the scratch
    a1 = randn_operand(3072, 2048, O.E4M3, 601, dev)
    b1 = randn_operand(3072, 2048, O.E4M3, 602, dev)
    s1, w1 = _both(ct, dev, a1, b1, torch.bfloat16, fill=hostile)
    assert torch.equal(s1.view(torch.int16), w1.view(torch.int16))
    # second call, smaller and ragged, right behind it on the same scratch
    a2 = randn_operand(300, 160, O.E4M3, 603, dev)
    b2 = randn_operand(200, 160, O.E2M1, 604, dev)
    s2, w2 = _both(ct, dev, a2, b2, torch.float32)
    assert torch.equal(s2, w2)
    assert O.rel_fro(s2.cpu(), oracle_matmul(a2, b2)) <= 1e-3
    # third: split-K (per-slice scales and fp32 partial products in the scratch), then the first shape again
    a3 = randn_operand(64, 8192, O.E4M3, 605, dev)
    b3 = randn_operand(256, 8192, O.E4M3, 606, dev)
    s3, w3 = _both(ct, dev, a3, b3, torch.float32, fill=hostile)
    assert torch.equal(s3, w3)
    assert O.rel_fro(s3.cpu(), oracle_matmul(a3, b3)) <= 1e-3
    s1b, _ = _both(ct, dev, a1, b1, torch.bfloat16, fill=hostile)
    assert torch.equal(s1b.view(torch.int16), w1.view(torch.int16))
    assert O.rel_fro(s1b[:64].float().cpu(), oracle_matmul(a1, b1)[:64]) <= 8e-3


def test_static_scratch_python_wrapper_and_limit(ct, dev):
    a = randn_operand(512, 1024, O.E4M3, 611, dev)
    b = randn_operand(384, 1024, O.E4M3, 612, dev)
    c = torch.empty((512, 384), dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, C=c, static_scratch=True)
    assert torch.cuda.memory_allocated(dev) == before
    want = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T)
    assert torch.equal(c, want)
    # beyond the limit: refused before anything is launched (descriptors only; the buffers are never touched)
    lib = ct.lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=dev)

    def d(dtype, shape, stride):
        t = L.MxTensor()
        t.ptr, t.dtype, t.ndim, t.packed_dim = buf.data_ptr(), dtype, 2, -1
        t.shape[0], t.shape[1], t.stride[0], t.stride[1] = *shape, *stride
        return t
    M = N = 32768
    K = 8192
    rc = lib.mx_gemm_static(ctypes.byref(d(L.MX_E4M3, (M, K), (K, 1))), ctypes.byref(d(L.MX_E8M0, (M, K // 32), (K // 32, 1))),
                            ctypes.byref(d(L.MX_E4M3, (K, N), (1, K))), ctypes.byref(d(L.MX_E8M0, (K // 32, N), (1, K // 32))),
                            ctypes.byref(d(L.MX_F32, (M, N), (N, 1))), None, L.stream_ptr(dev))
    assert rc == L.MX_ERR_WORKSPACE and "static buffer" in L.last_error()
