"""Host-side argument rules of mma_scaled / block_scaled_matmul with the reference's messages
(test/test_mma_scaled.py:250-333, samples/BlockScaledMatMul.py:258-264).  Runs on CPU tensors: every
rule is checked before anything touches the device."""
from dataclasses import dataclass

import pytest
import torch

import cutile_amd as ct

f8e4m3fn, f8e5m2, f8e8m0fnu = torch.float8_e4m3fn, torch.float8_e5m2, torch.float8_e8m0fnu
f32, f16, bf16 = torch.float32, torch.float16, torch.bfloat16


@dataclass
class DTC:
    x: torch.dtype
    y: torch.dtype
    xs: torch.dtype
    ys: torch.dtype
    acc: torch.dtype
    message: str


dtype_error_cases = [
    DTC(f8e4m3fn, f8e5m2, f8e8m0fnu, f8e8m0fnu, f32, "x and y must have the same dtype"),
    DTC(f8e4m3fn, f8e4m3fn, f8e8m0fnu, f8e4m3fn, f32, "x_scale and y_scale must have the same dtype"),
    DTC(f16, f16, f8e8m0fnu, f8e8m0fnu, f32, "Unsupported input dtype"),
    DTC(f8e4m3fn, f8e4m3fn, bf16, bf16, f32, "Unsupported scale dtype"),
    DTC(f8e4m3fn, f8e4m3fn, f8e8m0fnu, f8e8m0fnu, f16, "Unsupported acc dtype"),
]


@pytest.mark.parametrize("case", dtype_error_cases, ids=lambda c: c.message)
def test_mma_scaled_dtype_error(case):
    m, n, k, ks = 16, 16, 64, 2
    X = torch.randn((m, k)).to(case.x)
    Xs = torch.randn((m, ks)).to(case.xs)
    Y = torch.randn((k, n)).to(case.y)
    Ys = torch.randn((ks, n)).to(case.ys)
    Z = torch.zeros((m, n)).to(case.acc)
    with pytest.raises(ct.TileTypeError, match=case.message):
        ct.mma_scaled(X, Xs, Y, Ys, Z)


def test_mma_scaled_dtype_error_full_texts():
    X = torch.zeros((16, 64)).to(f8e4m3fn)
    S = torch.ones((16, 2)).to(f8e8m0fnu)
    with pytest.raises(ct.TileTypeError, match=r"x and y must have the same dtype, got float8_e4m3fn and float8_e5m2"):
        ct.mma_scaled(X, S, X.T.to(f8e5m2), S.T, torch.zeros(16, 16))
    with pytest.raises(ct.TileTypeError, match=r"Unsupported input dtype float16 for mma_scaled, supported input dtypes "
                                               r"are float8_e4m3fn, float8_e5m2, float4_e2m1fn"):
        ct.mma_scaled(X.to(f16), S, X.T.to(f16), S.T, torch.zeros(16, 16))
    with pytest.raises(ct.TileTypeError, match=r"Unsupported scale dtype bfloat16 for input dtype float8_e4m3fn, "
                                               r"supported scale dtypes are float8_e8m0fnu"):
        ct.mma_scaled(X, S.to(bf16), X.T, S.T.to(bf16), torch.zeros(16, 16))
    with pytest.raises(ct.TileTypeError, match=r"Unsupported acc dtype float16 for mma_scaled, expected float32"):
        ct.mma_scaled(X, S, X.T, S.T, torch.zeros(16, 16, dtype=f16))


shape_error_cases = [
    # tm, tn, tk, tms, tns, tks, message
    (16, 16, 64, 8, 16, 2, "x_scale shape .* is not compatible with x shape"),
    (16, 16, 64, 16, 8, 2, "y_scale shape .* is not compatible with y shape"),
    (16, 16, 16, 16, 16, 32,
     r"x\.shape\[1\] must be an exact multiple of x_scale\.shape\[1\] with scaling block size B = K // K_s in \{32\}, got x\.shape\[1\] = 16 and x_scale\.shape\[1\] = 32"),  # noqa
    (16, 16, 64, 16, 16, 8,
     r"x\.shape\[1\] must be an exact multiple of x_scale\.shape\[1\] with scaling block size B = K // K_s in \{32\}, got x\.shape\[1\] = 64 and x_scale\.shape\[1\] = 8"),  # noqa
]


@pytest.mark.parametrize("tm,tn,tk,tms,tns,tks,message", shape_error_cases)
def test_mma_scaled_shape_error(tm, tn, tk, tms, tns, tks, message):
    X = torch.randn((tm, tk)).to(f8e4m3fn)
    Xs = torch.randn((tms, tks)).to(f8e8m0fnu)
    Y = torch.randn((tk, tn)).to(f8e4m3fn)
    Ys = torch.randn((tks, tns)).to(f8e8m0fnu)
    Z = torch.zeros((tm, tn), dtype=f32)
    with pytest.raises(ct.TileTypeError, match=message):
        ct.mma_scaled(X, Xs, Y, Ys, Z)


def test_mma_scaled_rank_and_acc_shape_errors():
    S = torch.ones((16, 2)).to(f8e8m0fnu)
    Y = torch.ones((64, 16)).to(f8e4m3fn)
    with pytest.raises(ct.TileTypeError, match=r"Expect shape of `x` to be 2D or 3D"):
        ct.mma_scaled(torch.ones(16 * 64).to(f8e4m3fn), S, Y, S.T, torch.zeros(16, 16))
    X = torch.ones((16, 64)).to(f8e4m3fn)
    with pytest.raises(ct.TileTypeError, match=r"Expect acc shape to be \(16, 16\), got \(16, 8\)"):
        ct.mma_scaled(X, S, Y, S.T, torch.zeros(16, 8))
    with pytest.raises(ct.TileTypeError, match=r"Incompatible shapes for matrix mul on tiles"):
        ct.mma_scaled(X, S, torch.ones((32, 16)).to(f8e4m3fn), torch.ones((1, 16)).to(f8e8m0fnu), torch.zeros(16, 16))
    # FP4: block 16 is allowed with E8M0, 8 is not
    Xp = torch.zeros((16, 32), dtype=torch.uint8)
    with pytest.raises(ct.TileTypeError, match=r"scaling block size B = K // K_s in \{16, 32\}"):
        ct.mma_scaled(Xp, torch.ones((16, 8)).to(f8e8m0fnu), torch.zeros((64, 8), dtype=torch.uint8),
                      torch.ones((8, 16)).to(f8e8m0fnu), torch.zeros(16, 16), x_format="e2m1", y_format="e2m1")


def test_block_scaled_matmul_value_errors():
    A = torch.zeros((64, 128)).to(f8e4m3fn)
    As = torch.ones((64, 4)).to(f8e8m0fnu)
    B = torch.zeros((32, 96)).to(f8e4m3fn).T
    Bs = torch.ones((32, 3)).to(f8e8m0fnu).T
    with pytest.raises(ValueError, match=r"Incompatible matrices: K dimension of A \(128\) must match K dimension of B \(96\)"):
        ct.block_scaled_matmul(A, As, B, Bs)
    B = torch.zeros((32, 128)).to(f8e4m3fn).T
    Bs = torch.ones((32, 4)).to(f8e8m0fnu).T
    with pytest.raises(ValueError, match="Input tensors must be on a CUDA device."):
        ct.block_scaled_matmul(A, As, B, Bs)
    with pytest.raises(ValueError, match="Input tensors must be on the same device."):
        ct.block_scaled_matmul(A, As.to("meta"), B, Bs)
    with pytest.raises(ValueError, match="larger than the inner most dimension"):
        ct.block_quantize(torch.zeros(4, 16), 32)
