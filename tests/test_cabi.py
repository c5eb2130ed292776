"""CPU-only checks of the C ABI: the library loads, exports every symbol the header declares, and its
argument validation (which runs before any HIP call) returns the documented codes."""
import ctypes
import pathlib
import re

import pytest
import torch

import cutile_amd
from cutile_amd import _lib as L

ROOT = pathlib.Path(__file__).resolve().parent.parent


def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "mxgemm.h").read_text()
    declared = set(re.findall(r"MX_API\s+[\w\s\*]+?\b(mx_\w+)\s*\(", header))
    assert declared == set(L.SYMBOLS), declared ^ set(L.SYMBOLS)
    h = ctypes.CDLL(str(cutile_amd.LIB_PATH))
    for name in declared:
        assert hasattr(h, name), name
    assert cutile_amd.lib().mx_version() == int(re.search(r"#define MXGEMM_VERSION (\d+)", header).group(1))


def test_header_enums_match_python_constants():
    header = (ROOT / "include" / "mxgemm.h").read_text()
    for name in ["MX_E4M3", "MX_E5M2", "MX_E2M1", "MX_E8M0", "MX_F32", "MX_BF16", "MX_F16", "MX_I32",
                 "MX_SCALE_2D", "MX_SCALE_SWIZZLE_32_4_4", "MX_SCALE_NATIVE", "MX_SCALE_NATIVE32", "MX_OPERAND_A",
                 "MX_OPERAND_B", "MX_KERNEL_AUTO", "MX_KERNEL_GENERIC",
                 "MX_KERNEL_MFMA_128x128", "MX_KERNEL_MFMA_256x256", "MX_KERNEL_MFMA_256x256_W4", "MX_KERNEL_DECODE", "MX_KERNEL_MFMA_PINGPONG", "MX_KERNEL_MFMA_PINGPONG32", "MX_KERNEL_MFMA_W4_PERSISTENT",
                 "MX_ERR_INVALID", "MX_ERR_SHAPE", "MX_ERR_DTYPE", "MX_ERR_LAYOUT", "MX_ERR_WORKSPACE",
                 "MX_ERR_DEVICE", "MX_ERR_LAUNCH"]:
        m = re.search(rf"\b{name}\s*=\s*(-?\d+)", header)
        assert m and int(m.group(1)) == getattr(L, name), name
    assert ctypes.sizeof(L.MxTensor) == 8 + 4 + 4 + 32 + 32 + 8
    assert ctypes.sizeof(L.MxGemmOpts) == 32


def test_pure_size_functions():
    lib = cutile_amd.lib()
    # [rows/64][K/512][64 lanes][4] dwords, rows padded to 64, K to 512
    assert lib.mx_packed_scale_bytes(8192, 8192) == 8192 * 8192 // 32
    assert lib.mx_packed_scale_bytes(1, 32) == 1024
    assert lib.mx_packed_scale_bytes(65, 544) == 2 * 2 * 1024
    assert lib.mx_gemm_workspace_bytes(8192, 8192, 8192, None) == 2 * 8192 * 8192 // 32
    assert lib.mx_moe_align_max_slots(8192, 8, 256) == (8192 + 8 * 255) // 256 * 256
    assert lib.mx_moe_align_max_slots(3, 64, 16) == 3 * 16
    assert lib.mx_moe_align_max_slots(0, 8, 16) == 0


def _desc(ptr, dtype, shape, stride, packed=-1):
    d = L.MxTensor()
    d.ptr, d.dtype, d.ndim, d.packed_dim = ptr, dtype, len(shape), packed
    for i, (s, st) in enumerate(zip(shape, stride)):
        d.shape[i], d.stride[i] = s, st
    return d


def test_validation_codes_without_gpu():
    lib = cutile_amd.lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8)
    p = buf.data_ptr()
    A = _desc(p, L.MX_E4M3, (64, 128), (128, 1))
    As = _desc(p, L.MX_E8M0, (64, 4), (4, 1))
    B = _desc(p, L.MX_E4M3, (128, 32), (1, 128))
    Bs = _desc(p, L.MX_E8M0, (4, 32), (1, 4))
    C = _desc(p, L.MX_F32, (64, 32), (32, 1))
    call = lambda a, as_, b, bs, c: lib.mx_gemm(ctypes.byref(a), ctypes.byref(as_), ctypes.byref(b), ctypes.byref(bs),
                                                ctypes.byref(c), None, None, 0, None)
    Bbad = _desc(p, L.MX_E4M3, (96, 32), (1, 96))
    assert call(A, As, Bbad, Bs, C) == L.MX_ERR_SHAPE
    assert "K dimension of A (128) must match K dimension of B (96)" in L.last_error()
    assert call(_desc(p, L.MX_F16, (64, 128), (128, 1)), As, B, Bs, C) == L.MX_ERR_DTYPE
    assert call(A, _desc(p, L.MX_E8M0, (32, 4), (4, 1)), B, Bs, C) == L.MX_ERR_SHAPE
    assert call(A, As, B, Bs, _desc(p, L.MX_F32, (64, 16), (16, 1))) == L.MX_ERR_SHAPE
    assert call(A, As, B, Bs, _desc(p, L.MX_F16, (64, 32), (32, 1))) == L.MX_ERR_DTYPE
    assert call(_desc(None, L.MX_E4M3, (64, 128), (128, 1)), As, B, Bs, C) == L.MX_ERR_INVALID
    assert call(_desc(p, L.MX_E4M3, (64, 128), (-128, 1)), As, B, Bs, C) == L.MX_ERR_LAYOUT
    # MFMA path without a workspace for the scale re-layout
    assert call(A, As, B, Bs, C) == L.MX_ERR_WORKSPACE
    # explicit MFMA kernel with a layout it cannot take
    o = L.MxGemmOpts(struct_size=32, kernel=L.MX_KERNEL_MFMA_128x128, block_size=32)
    Brm = _desc(p, L.MX_E4M3, (128, 32), (32, 1))
    rc = lib.mx_gemm(ctypes.byref(A), ctypes.byref(As), ctypes.byref(Brm), ctypes.byref(Bs), ctypes.byref(C),
                     ctypes.byref(o), None, 0, None)
    assert rc == L.MX_ERR_LAYOUT and "K axis is not contiguous" in L.last_error()
    # the general kernel validates a swizzle_32_4_4 descriptor before it indexes through it
    o = L.MxGemmOpts(struct_size=32, kernel=L.MX_KERNEL_GENERIC, block_size=32,
                     a_scale_layout=L.MX_SCALE_SWIZZLE_32_4_4)
    A128 = _desc(p, L.MX_E4M3, (128, 128), (128, 1))
    C128 = _desc(p, L.MX_F32, (128, 32), (32, 1))
    for bad in (_desc(p, L.MX_E8M0, (128, 4), (4, 1)), _desc(p, L.MX_E8M0, (2, 1, 32, 16), (512, 512, 16, 1)),
                _desc(p, L.MX_E8M0, (1, 1, 32, 16), (512, 512, 32, 2))):
        rc = lib.mx_gemm(ctypes.byref(A128), ctypes.byref(bad), ctypes.byref(B), ctypes.byref(Bs), ctypes.byref(C128),
                         ctypes.byref(o), None, 0, None)
        assert rc in (L.MX_ERR_SHAPE, L.MX_ERR_LAYOUT), (rc, L.last_error())
    # moe_align: scratch for more than one chunk of ids is required
    assert lib.mx_moe_align_workspace_bytes(1024, 8) == 0
    assert lib.mx_moe_align_workspace_bytes(8192, 8) == 8 * 8 * 4
    assert lib.mx_moe_align(p, 8192, 8, 256, p, p, None, None, 0, None) == L.MX_ERR_WORKSPACE
    # quantiser argument checks
    x = _desc(p, L.MX_F32, (4, 16), (16, 1))
    xq = _desc(p, L.MX_E4M3, (4, 32), (32, 1))
    sc = _desc(p, L.MX_E8M0, (4, 1), (1, 1))
    assert lib.mx_quantize(ctypes.byref(x), ctypes.byref(xq), ctypes.byref(sc), 0, None) == L.MX_ERR_SHAPE
    assert "larger than the inner most dimension" in L.last_error()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(L, "LIB_PATH", tmp_path / "libmxgemm.so")
    monkeypatch.setattr(L, "_lib", None)
    with pytest.raises(L.MXLibraryError, match="no CPU or PyTorch fallback"):
        L.lib()
