"""GPU restatement of the reference's unit tests of ct.mma_scaled (test/test_mma_scaled.py:82-183): tiny
tiles, row-major K x N operands, accumulator pre-loaded, raw-byte operands, FP4 packed along N, block 16
and E4M3 scales.  These layouts run on the general kernel.  atol = rtol = 1e-2 as in the reference."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu
f8e8m0 = torch.float8_e8m0fnu


def _ref(xc, xs, yc, ys, z, fmt, block, scale_fmt="e8m0"):
    dec_s = O.decode_e8m0 if scale_fmt == "e8m0" else O.decode_e4m3
    x = torch.from_numpy(O.decode_elem(xc, fmt)) * torch.repeat_interleave(torch.from_numpy(dec_s(xs)), block, dim=-1)
    y = torch.from_numpy(O.decode_elem(yc, fmt)) * torch.repeat_interleave(torch.from_numpy(dec_s(ys)), block, dim=-2)
    return x @ y + z


def _scales(shape, seed, dtype=f8e8m0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g).to(dtype)     # randn -> e8m0 spans 2^-12 .. 2^2


@pytest.mark.parametrize("dtype,fmt", [(torch.float8_e4m3fn, O.E4M3), (torch.float8_e5m2, O.E5M2)], ids=str)
def test_mma_scaled_fp8(ct, dev, dtype, fmt):
    m, n, k, ks = 16, 16, 64, 2
    g = torch.Generator().manual_seed(1)
    X = torch.randn((m, k), generator=g).to(dtype)
    Y = torch.randn((k, n), generator=g).to(dtype)
    Xs, Ys = _scales((m, ks), 2), _scales((ks, n), 3)
    Z = torch.randn((m, n), generator=g)
    ref = _ref(X.view(torch.uint8).numpy(), Xs.view(torch.uint8).numpy(), Y.view(torch.uint8).numpy(),
               Ys.view(torch.uint8).numpy(), Z, fmt, 32)
    out = ct.mma_scaled(X.to(dev), Xs.to(dev), Y.to(dev), Ys.to(dev), Z.to(dev))
    torch.testing.assert_close(out.cpu(), ref, atol=1e-2, rtol=1e-2)
    # K-contiguous y (transposed view) takes the MFMA path and must agree as well
    Yt = Y.T.contiguous().to(dev)
    out2 = ct.mma_scaled(X.to(dev), Xs.to(dev), Yt.T, Ys.T.contiguous().to(dev).T, Z.to(dev))
    torch.testing.assert_close(out2.cpu(), ref, atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("fmt,name", [(O.E4M3, "e4m3"), (O.E5M2, "e5m2")])
def test_mma_scaled_general_fp8_raw_bytes(ct, dev, fmt, name):
    m, n, k, ks = 16, 16, 64, 2
    rng = np.random.default_rng(4)
    X = rng.integers(0, 256, (m, k), dtype=np.uint8)
    Y = rng.integers(0, 256, (k, n), dtype=np.uint8)
    Xs, Ys = _scales((m, ks), 5), _scales((ks, n), 6)
    Z = torch.randn((m, n), generator=torch.Generator().manual_seed(7))
    ref = _ref(X, Xs.view(torch.uint8).numpy(), Y, Ys.view(torch.uint8).numpy(), Z, fmt, 32)
    out = ct.mma_scaled(torch.from_numpy(X).to(dev), Xs.to(dev), torch.from_numpy(Y).to(dev), Ys.to(dev),
                        Z.to(dev), x_format=name, y_format=name)
    torch.testing.assert_close(out.cpu(), ref, atol=1e-2, rtol=1e-2, equal_nan=True)


def test_batch_mma_scaled_fp8(ct, dev):
    b, m, n, k, ks = 2, 16, 16, 128, 4
    g = torch.Generator().manual_seed(8)
    X = torch.randn((m, k), generator=g).to(torch.float8_e4m3fn)
    Y = torch.randn((b, k, n), generator=g).to(torch.float8_e4m3fn)
    Xs, Ys = _scales((m, ks), 9), _scales((b, ks, n), 10)
    Z = torch.randn((b, m, n), generator=g)
    ref = _ref(X.view(torch.uint8).numpy(), Xs.view(torch.uint8).numpy(), Y.view(torch.uint8).numpy(),
               Ys.view(torch.uint8).numpy(), Z, O.E4M3, 32)
    out = ct.mma_scaled(X.to(dev), Xs.to(dev), Y.to(dev), Ys.to(dev), Z.to(dev))
    assert out.shape == (b, m, n)
    torch.testing.assert_close(out.cpu(), ref, atol=1e-2, rtol=1e-2)


def test_batch_mma_scaled_k_contiguous_broadcast(ct, dev):
    """Batched operands whose matrices are K-contiguous (y given as the transposed view of (b, n, k)) take
    the MFMA kernels entry by entry; x has a batch of one and is broadcast (test/test_mma_scaled.py:128-145,
    batch rules src/cuda/tile/_stub.py:2232-2235)."""
    b, m, n, k, ks = 3, 96, 160, 256, 8
    g = torch.Generator().manual_seed(21)
    X = torch.randn((1, m, k), generator=g).to(torch.float8_e4m3fn)
    Yt = torch.randn((b, n, k), generator=g).to(torch.float8_e4m3fn)
    Xs, Yst = _scales((1, m, ks), 22), _scales((b, n, ks), 23)
    Z = torch.randn((b, m, n), generator=g)
    ref = _ref(X.view(torch.uint8).numpy(), Xs.view(torch.uint8).numpy(),
               Yt.view(torch.uint8).numpy().transpose(0, 2, 1), Yst.view(torch.uint8).numpy().transpose(0, 2, 1),
               Z, O.E4M3, 32)
    out = ct.mma_scaled(X.to(dev), Xs.to(dev), Yt.to(dev).transpose(1, 2), Yst.to(dev).transpose(1, 2), Z.to(dev))
    assert out.shape == (b, m, n)
    assert O.rel_fro(out.cpu(), ref) < 1e-3


@pytest.mark.parametrize("scale_dtype,block", [(f8e8m0, 32), (f8e8m0, 16), (torch.float8_e4m3fn, 16)], ids=str)
def test_mma_scaled_general_f4(ct, dev, scale_dtype, block):
    m, n, k = 16, 16, 64
    ks = k // block
    rng = np.random.default_rng(11)
    Xp = rng.integers(0, 256, (m, k // 2), dtype=np.uint8)      # packed along K
    Yp = rng.integers(0, 256, (k, n // 2), dtype=np.uint8)      # row-major K x N, packed along N
    Xs, Ys = _scales((m, ks), 12, scale_dtype), _scales((ks, n), 13, scale_dtype)
    Z = torch.randn((m, n), generator=torch.Generator().manual_seed(14))
    ref = _ref(O.unpack_fp4(Xp), Xs.view(torch.uint8).numpy(), O.unpack_fp4(Yp), Ys.view(torch.uint8).numpy(), Z,
               O.E2M1, block, "e8m0" if scale_dtype == f8e8m0 else "e4m3")
    out = ct.mma_scaled(torch.from_numpy(Xp).to(dev), Xs.to(dev), torch.from_numpy(Yp).to(dev), Ys.to(dev),
                        Z.to(dev), x_format="e2m1", y_format="e2m1")
    torch.testing.assert_close(out.cpu(), ref, atol=1e-2, rtol=1e-2)


def test_mma_scaled_mixed_formats_extension(ct, dev):
    """E4M3 x E2M1: rejected by the reference (src/cuda/tile/_datatype.py:497-499), native on CDNA4."""
    m, n, k = 32, 64, 256
    rng = np.random.default_rng(15)
    X = rng.integers(0, 256, (m, k), dtype=np.uint8)
    X[(X & 0x7F) == 0x7F] = 0x30
    Wp = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)      # N x K storage, packed along K
    Xs, Ws = _scales((m, k // 32), 16), _scales((n, k // 32), 17)
    Z = torch.zeros((m, n))
    x = torch.from_numpy(O.decode_e4m3(X)) * torch.repeat_interleave(torch.from_numpy(O.decode_e8m0(Xs.view(torch.uint8).numpy())), 32, 1)
    w = torch.from_numpy(O.decode_e2m1(O.unpack_fp4(Wp))) * torch.repeat_interleave(torch.from_numpy(O.decode_e8m0(Ws.view(torch.uint8).numpy())), 32, 1)
    ref = x @ w.T
    args = (torch.from_numpy(X).to(dev).view(torch.float8_e4m3fn), Xs.to(dev), torch.from_numpy(Wp).to(dev).T,
            Ws.to(dev).T, Z.to(dev))
    with pytest.raises(ct.TileTypeError, match="x and y must have the same dtype"):
        ct.mma_scaled(*args, y_format="e2m1")
    for kernel in ("generic", "mfma128", "auto"):
        out = ct.mma_scaled(*args, y_format="e2m1", allow_mixed_dtypes=True, kernel=kernel)
        assert O.rel_fro(out.cpu(), ref) < 1e-3, kernel
