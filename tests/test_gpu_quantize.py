"""GPU parity of the on-device MX quantiser and the scale re-layout: bit-exact against the oracle."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu
DT = {O.E4M3: torch.float8_e4m3fn, O.E5M2: torch.float8_e5m2, O.E2M1: "e2m1"}


def _special_rows(K):
    """Rows that exercise the corners: zeros, one-hot, subnormals, huge, exact powers of two, the fp32
    log2 edge 2^k(1+2^-23), values on rounding ties."""
    rows = []
    z = np.zeros(K, np.float32); rows.append(z.copy())
    r = z.copy(); r[3] = 1.0; rows.append(r)
    r = z.copy(); r[::2] = np.float32(1e-41); r[1] = np.float32(3e-39); rows.append(r)      # subnormal inputs
    r = z.copy(); r[:] = np.float32(3e38); r[5] = -np.float32(3.4e38); rows.append(r)       # near fp32 max
    r = z.copy(); r[:32] = np.float32(448.0) * np.float32(2.0 ** -8) * (np.float32(1) + np.float32(2.0 ** -23)); rows.append(r)
    r = z.copy(); r[:32] = 448.0; r[32:64] = 464.0 / 2; r[64:96] = 6.0; rows.append(r)
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0, 7.0, 0.0625, 17.0, 18.0, 19.0, 20.0, 21.0, 22.0],
                    np.float32)
    r = z.copy(); r[:16] = ties; r[16:32] = -ties; r[32:48] = ties * 8; r[48:64] = ties * 2.0 ** -12; rows.append(r)
    r = z.copy(); r[:] = np.float32(2.0 ** -126); r[7] = np.float32(2.0 ** -120); rows.append(r)
    return np.stack(rows)


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2, O.E2M1])
@pytest.mark.parametrize("mode", ["ceil", "floor"])
def test_quantize_bit_exact(ct, dev, fmt, mode):
    K = 256
    g = torch.Generator().manual_seed(5)
    x = torch.cat([torch.randn((61, K), generator=g), torch.randn((30, K), generator=g) * 1e-3,
                   torch.rand((20, K), generator=g) * 12 - 6, torch.from_numpy(_special_rows(K))])
    xq, sc = ct.block_quantize(x.to(dev), 32, DT[fmt], scale_mode=mode)
    codes, sb = O.block_quantize(x.numpy(), 32, fmt, mode)
    got_s = sc.view(torch.uint8).cpu().numpy()
    assert np.array_equal(got_s, sb), np.argwhere(got_s != sb)[:10]
    got = xq.view(torch.uint8).cpu().numpy()
    want = O.pack_fp4(codes) if fmt == O.E2M1 else codes
    assert got.shape == want.shape
    bad = np.argwhere(got != want)
    assert bad.size == 0, (bad[:10], got[tuple(bad[0])], want[tuple(bad[0])], x.numpy()[bad[0][0]].max())
    assert sc.dtype == torch.float8_e8m0fnu and sc.shape == (x.shape[0], K // 32)


def test_quantize_padding_3d_and_bf16(ct, dev):
    g = torch.Generator().manual_seed(6)
    x = torch.randn((3, 5, 72), generator=g)          # K = 72 -> padded to 96 (kernel_utils.py:62-67)
    xq, sc = ct.block_quantize(x.to(dev), 32)
    codes, sb = O.block_quantize(x.numpy(), 32, O.E4M3, "ceil")
    assert xq.shape == (3, 5, 96) and xq.dtype == torch.float8_e4m3fn and sc.shape == (3, 5, 3)
    assert np.array_equal(xq.view(torch.uint8).cpu().numpy(), codes)
    assert np.array_equal(sc.view(torch.uint8).cpu().numpy(), sb)
    xb = torch.randn((33, 160), generator=g).to(torch.bfloat16)
    xq, sc = ct.block_quantize(xb.to(dev), 32, scale_mode="floor")
    codes, sb = O.block_quantize(xb.float().numpy(), 32, O.E4M3, "floor")
    assert np.array_equal(xq.view(torch.uint8).cpu().numpy(), codes)
    assert np.array_equal(sc.view(torch.uint8).cpu().numpy(), sb)
    with pytest.raises(ValueError, match="larger than the inner most dimension"):
        ct.block_quantize(torch.zeros((4, 16), device=dev), 32)


def test_quantize_dequantize_roundtrip_large(ct, dev):
    """Full benchmark-size operand (8192 x 8192): quantise on the GPU, check invariants that do not need the
    CPU oracle at this size, and compare a 64-row sample bit-for-bit."""
    g = torch.Generator().manual_seed(1234)
    x = torch.randn((8192, 8192), generator=g)
    xq, sc = ct.block_quantize(x.to(dev), 32, scale_mode="floor")
    rows = torch.arange(0, 8192, 128)
    codes, sb = O.block_quantize(x[rows].numpy(), 32, O.E4M3, "floor")
    assert np.array_equal(xq[rows.to(dev)].view(torch.uint8).cpu().numpy(), codes)
    assert np.array_equal(sc[rows.to(dev)].view(torch.uint8).cpu().numpy(), sb)
    q = xq.view(torch.uint8)
    assert int(((q & 0x7F) == 0x7F).sum()) == 0                       # saturating: no NaN codes
    # idempotence: quantising the dequantised tensor with the same rule reproduces codes and scales
    deq = xq.float() * torch.repeat_interleave(sc.float(), 32, dim=1)
    xq2, sc2 = ct.block_quantize(deq, 32, scale_mode="floor")
    assert torch.equal(sc2.view(torch.uint8), sc.view(torch.uint8))
    assert torch.equal(xq2.view(torch.uint8), q)


def _bperm_row(j: int, c: int) -> int:
    """Row of a 64-row group that the 16x16x128 kernels feed to the instruction as operand row c of tile j."""
    return 32 * (j // 2) + 8 * (c // 4) + 4 * (j % 2) + c % 4


def _native_layout_loops(scales: np.ndarray, target: str = "a") -> np.ndarray:
    """Plain-numpy statement of the native scale layouts, element by element.  16 bytes per (64-row group G,
    K-quad Q, lane = c + 16 g), holding the scales of K block (4 Q + t) * 4 + g for t = 0..3 and four rows:
      "a":      byte [t][b] = row 64 G + 16 b + c        (MX_SCALE_NATIVE, A operand)
      "b":      byte [t][b] = row 64 G + bperm_row(b, c) (MX_SCALE_NATIVE, B operand)
      "tile32": byte [b][t] = row 64 G + 16 b + c        (MX_SCALE_NATIVE32)
    padding byte 127."""
    R, KB = scales.shape
    R64, KQ = -(-R // 64), -(-KB // 16)
    out = np.full((R64, KQ, 64, 4, 4), 127, dtype=np.uint8)
    for G in range(R64):
        for b in range(4):
            for c in range(16):
                row = 64 * G + (_bperm_row(b, c) if target == "b" else 16 * b + c)
                if row >= R:
                    continue
                for kb in range(KB):
                    ks, g = divmod(kb, 4)
                    Q, t = divmod(ks, 4)
                    if target == "tile32":
                        out[G, Q, g * 16 + c, b, t] = scales[row, kb]
                    else:
                        out[G, Q, g * 16 + c, t, b] = scales[row, kb]
    return out.reshape(-1)


_PACK_KW = {"a": dict(operand="a"), "b": dict(operand="b"), "tile32": dict(operand="a", kernel="pingpong32")}


@pytest.mark.parametrize("target", ["a", "b", "tile32"])
@pytest.mark.parametrize("R,K", [(64, 512), (100, 160), (256, 1024), (16, 32), (128, 128), (384, 2048)])
def test_pack_scales_layout_all_sources_agree(ct, dev, R, K, target):
    """Element-by-element statement of each layout, and the same bytes from every source form: row-major,
    transposed (how B_scale is passed) and the 4-D swizzle_32_4_4 tensor."""
    rng = np.random.default_rng(R + K)
    s = rng.integers(0, 255, (R, K // 32), dtype=np.uint8)
    t = torch.from_numpy(s).to(dev)
    kw = _PACK_KW[target]
    p = ct.pack_scales(t.view(torch.float8_e8m0fnu), **kw)
    want = _native_layout_loops(s, target)
    got = p.data.cpu().numpy()[:want.size]
    assert np.array_equal(got, want)
    # transposed source (how B_scale is passed) gives the same bytes
    p2 = ct.pack_scales(t.T.contiguous().view(torch.float8_e8m0fnu), transposed=True, **kw)
    assert torch.equal(p.data, p2.data)
    if R % 128 == 0 and (K // 32) % 4 == 0:
        p3 = ct.pack_scales(ct.swizzle_32_4_4(t), **kw)
        assert torch.equal(p.data, p3.data)


def test_pack_scales_operand_defaults_and_mismatch(ct, dev):
    s = torch.randint(100, 140, (128, 16), dtype=torch.uint8, device=dev)
    assert ct.pack_scales(s).operand == "a" and ct.pack_scales(s.T.contiguous(), transposed=True).operand == "b"
    assert ct.pack_scales(s.reshape(2, 64, 16)).operand == "b"          # a batch of expert weights
    a = torch.zeros((128, 512), dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    with pytest.raises(ValueError, match="packed for operand"):
        ct.block_scaled_matmul(a, ct.pack_scales(s, operand="b"), a.T, ct.pack_scales(s, operand="b"))
    with pytest.raises(ct.TileTypeError, match="native-layout scales of kind"):
        ct.block_scaled_matmul(a, ct.pack_scales(s, operand="a", kernel="pingpong32"), a.T,
                               ct.pack_scales(s, operand="b", kernel="pingpong32"), kernel="mfma128")


def test_swizzle_roundtrip_device(ct, dev):
    # experimental/cuda-lang/test/examples/tk/test_mxfp8_b200_gemm.py:835-837 checks the same round trip
    s = torch.arange(256 * 8, device=dev, dtype=torch.int32).reshape(256, 8)
    sw = ct.swizzle_32_4_4(s)
    assert np.array_equal(sw.cpu().numpy(), O.swizzle_32_4_4(s.cpu().numpy()))
    assert torch.equal(ct.unswizzle_32_4_4(sw), s)


def _native_layout(sc: np.ndarray, target: str = "a") -> np.ndarray:
    """The packed layouts restated with array slicing (see _native_layout_loops for the element-wise form); rows
    padded to 64 and K blocks to 16 with 127."""
    rows, KB = sc.shape
    R, KQ = -(-rows // 64) * 64, -(-KB // 16)
    full = np.full((R, KQ * 16), 127, dtype=np.uint8)
    full[:rows, :KB] = sc
    out = np.zeros((R // 64, KQ, 64, 4, 4), dtype=np.uint8)   # [G][Q][lane][first index][second index]
    for lane in range(64):
        c, g = lane % 16, lane // 16
        for b in range(4):
            row = _bperm_row(b, c) if target == "b" else 16 * b + c
            for t in range(4):
                v = full[row::64, :].reshape(R // 64, KQ, 16)[:, :, 4 * t + g]
                if target == "tile32":
                    out[:, :, lane, b, t] = v
                else:
                    out[:, :, lane, t, b] = v
    return out.reshape(-1)


@pytest.mark.gpu
@pytest.mark.parametrize("rows,KB", [(64, 16), (100, 37), (256, 256), (1, 1), (130, 5)])
@pytest.mark.parametrize("form", ["row_major", "transposed", "sliced", "batched"])
@pytest.mark.parametrize("target", ["a", "b", "tile32"])
def test_pack_scales_layout(ct, dev, rows, KB, form, target):
    """mx_pack_scales against a restatement of the layout, for every source form the staging code
    distinguishes (16-byte loads along K or along rows, misaligned sources, batches)."""
    rng = np.random.default_rng(rows * 1000 + KB)
    kw = _PACK_KW[target]
    if form == "batched":
        sc = rng.integers(0, 255, size=(3, rows, KB), dtype=np.uint8)
        got = ct.pack_scales(torch.from_numpy(sc).to(dev), **kw).data.cpu().numpy()
        want = np.concatenate([_native_layout(sc[b], target) for b in range(3)])
    else:
        sc = rng.integers(0, 255, size=(rows, KB), dtype=np.uint8)
        if form == "row_major":
            t = torch.from_numpy(sc).to(dev)
            got = ct.pack_scales(t, **kw).data.cpu().numpy()
        elif form == "transposed":
            t = torch.from_numpy(np.ascontiguousarray(sc.T)).to(dev)   # [K/32, rows], as B_scale arrives
            got = ct.pack_scales(t, transposed=True, **kw).data.cpu().numpy()
        else:
            big = torch.zeros((rows + 3, KB + 7), dtype=torch.uint8, device=dev)
            big[1:rows + 1, 3:KB + 3] = torch.from_numpy(sc).to(dev)
            got = ct.pack_scales(big[1:rows + 1, 3:KB + 3], **kw).data.cpu().numpy()
        want = _native_layout(sc, target)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("fmt,mode", [(O.E4M3, "floor"), (O.E4M3, "ceil"), (O.E2M1, "floor"), (O.E5M2, "floor")])
@pytest.mark.parametrize("rows,F", [(5, 32), (33, 96), (16, 48), (7, 1000)])
def test_silu_mul_quantize_bit_exact(ct, dev, in_dtype, fmt, mode, rows, F):
    """The fused SiLU(gate) * up + MX quantise pass (silu_and_mul_kernel, test/kernels/fused_moe.py:85-108,
    then block_quantize) is bit-identical to the oracle's restatement, ragged F and extreme gates included."""
    g = torch.Generator().manual_seed(rows * 31 + F)
    x = torch.randn((rows, 2 * F), generator=g) * 4
    x[0, :8] = torch.tensor([0.0, -0.0, 90.0, -90.0, 1e-30, -200.0, 30.0, -30.0])
    x = x.to(in_dtype)
    want_q, want_s = O.silu_mul_quantize(x.float().numpy(), fmt, mode)
    got_q, got_s = ct.silu_and_mul_quantize(x.to(dev), DT[fmt], scale_mode=mode)
    got_codes = got_q.view(torch.uint8).cpu().numpy()
    if fmt == O.E2M1:
        got_codes = O.unpack_fp4(got_codes)
    assert np.array_equal(got_s.view(torch.uint8).cpu().numpy(), want_s)
    assert np.array_equal(got_codes, want_q)


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2, O.E2M1])
@pytest.mark.parametrize("mode", ["floor", "ceil"])
def test_quantize_dense_rounding_grid(ct, dev, fmt, mode):
    """Every block holds one anchor (which fixes the shared exponent) and 31 values from a dense grid of
    fractions of it: all rounding ties, the subnormal range of the element format, values just below and
    above the largest finite code.  Bit-exact against the oracle (encoders pinned by tests/test_oracle.py)."""
    rng = np.random.default_rng(17)
    anchors = np.array([1.0, 1.75, 447.9, 448.0, 3.0e-5, 7.3e11, 0.013, 5.99, 6.0, 57344.0], np.float32)
    fr = np.concatenate([np.arange(0, 4097, dtype=np.float64) / 4096.0,             # 12-bit fractions: all ties
                         2.0 ** -np.arange(1, 24, dtype=np.float64) * 1.5,           # deep into the subnormals
                         1.0 + np.arange(-8, 9, dtype=np.float64) * 2.0 ** -10])     # around the anchor itself
    fr = fr[: (len(fr) // 31) * 31].reshape(-1, 31)
    blocks = []
    for a in anchors:
        for row in fr:
            sign = rng.choice([-1.0, 1.0], 31)
            blocks.append(np.concatenate([[a], np.minimum(row, 1.0) * a * sign]))
    x = np.asarray(blocks, np.float32).reshape(-1, 32 * 7)                            # 7 blocks per row
    want_q, want_s = O.block_quantize(x, 32, fmt, mode)
    got_q, got_s = ct.block_quantize(torch.from_numpy(x).to(dev), 32, DT[fmt], scale_mode=mode)
    got_codes = got_q.view(torch.uint8).cpu().numpy()
    if fmt == O.E2M1:
        got_codes = O.unpack_fp4(got_codes)
    assert np.array_equal(got_s.view(torch.uint8).cpu().numpy(), want_s)
    assert np.array_equal(got_codes, want_q)


@pytest.mark.parametrize("dt", [torch.float8_e4m3fn, torch.float8_e5m2], ids=str)
def test_quantize_nonfinite_blocks_follow_the_reference_rule(ct, dev, dt):
    """Blocks holding NaN or inf under the reference's rule (test/kernels/kernel_utils.py:69-78 as torch
    evaluates it): scale byte 0xFF, NaN codes where x / scale is NaN, signed zeros elsewhere.  Compared with
    the literal torch restatement on the CPU, and with the oracle's integer formulation."""
    x = np.random.default_rng(0).standard_normal((8, 96)).astype(np.float32)
    x[0, 3] = np.nan
    x[1, 5] = np.inf
    x[2, 40] = -np.inf
    x[3, 1] = -np.float32(np.nan)
    x[3, 2] = np.inf
    x[4, 33] = np.inf
    x[4, 34] = -np.inf
    x[5, 64:96] = np.nan
    lit_q, lit_s = O.block_quantize_ceil_literal(torch.from_numpy(x), 32, dt)
    got_q, got_s = ct.block_quantize(torch.from_numpy(x).to(dev), 32, dt, scale_mode="ceil")
    assert np.array_equal(got_s.view(torch.uint8).cpu().numpy(), lit_s.view(torch.uint8).numpy())
    assert np.array_equal(got_q.view(torch.uint8).cpu().numpy(), lit_q.view(torch.uint8).numpy())
    fmt = O.E4M3 if dt == torch.float8_e4m3fn else O.E5M2
    codes, sb = O.block_quantize(x, 32, fmt, "ceil")
    assert np.array_equal(got_s.view(torch.uint8).cpu().numpy(), sb)
    assert np.array_equal(got_q.view(torch.uint8).cpu().numpy(), codes)
