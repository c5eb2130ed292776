"""Pins the CPU oracle (oracle/mx_oracle.py) against the reference's own golden data and against
what the mathematics fixes.  No GPU, no reference import."""
import json
import math
import pathlib

import numpy as np
import pytest
import torch

from oracle import mx_oracle as O

GOLDEN = pathlib.Path(__file__).parent / "golden"


def _table(name):
    t = json.loads((GOLDEN / "float_tables.json").read_text())[name]
    out = []
    for v in t:
        out.append(math.nan if v == "nan" else (-0.0 if v == "-0.0" else float(v)))
    return np.array(out, dtype=np.float64)


def _same(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    nan = np.isnan(a)
    return np.array_equal(nan, np.isnan(b)) and np.array_equal(a[~nan], b[~nan]) and \
        np.array_equal(np.signbit(a[~nan]), np.signbit(b[~nan]))


# ---- decode tables: the reference's value tables (test/test_float_encoding.py:49-186) -------------
def test_decode_e2m1_table():
    assert _same(O.decode_e2m1(np.arange(16, dtype=np.uint8)), _table("f4e2m1fn_values"))


def test_decode_e4m3_table_and_torch_view():
    codes = np.arange(256, dtype=np.uint8)
    assert _same(O.decode_e4m3(codes), _table("f8e4m3fn_values"))
    tv = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    assert _same(O.decode_e4m3(codes), tv)


def test_decode_e8m0_table_and_torch_view():
    codes = np.arange(256, dtype=np.uint8)
    assert _same(O.decode_e8m0(codes), _table("f8e8m0fnu_values"))
    tv = torch.from_numpy(codes).view(torch.float8_e8m0fnu).float().numpy()
    assert _same(O.decode_e8m0(codes), tv)


def test_decode_e5m2_torch_view():
    codes = np.arange(256, dtype=np.uint8)
    tv = torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()
    assert _same(O.decode_e5m2(codes), tv)


# ---- encoders ------------------------------------------------------------------------------------
def test_e4m3_roundtrip_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    vals = O.decode_e4m3(codes)
    back = O.encode_e4m3(vals, saturate=False)
    ok = ~np.isnan(vals)
    assert np.array_equal(back[ok], codes[ok])
    assert np.all((back[~ok] & 0x7F) == 0x7F)


def _nearest_even_bruteforce(x, table_vals, table_codes, even_of):
    """Independent formulation: nearest representable value, ties to the candidate whose code is even."""
    out = np.empty(x.shape, dtype=np.uint8)
    for i, v in enumerate(x.ravel()):
        d = np.abs(table_vals - abs(float(v)))
        best = np.flatnonzero(d == d.min())
        if len(best) > 1:
            best = [b for b in best if even_of(table_codes[b])]
        out.ravel()[i] = table_codes[best[0]]
    return out


def test_e4m3_encode_bruteforce_nearest_even():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.uniform(-460, 460, 4000), rng.normal(0, 1, 4000), rng.normal(0, 0.01, 2000),
        # exact midpoints between neighbours, and the 464 boundary
        (O.decode_e4m3(np.arange(0, 126, dtype=np.uint8)).astype(np.float64) +
         O.decode_e4m3(np.arange(1, 127, dtype=np.uint8)).astype(np.float64)) / 2,
        [463.9, 464.0, 448.0, 2.0 ** -10, 2.0 ** -9, 1.5 * 2.0 ** -10, 0.0],
    ]).astype(np.float32)
    x = x[np.abs(x) <= 464.0]
    pos = O.decode_e4m3(np.arange(0, 127, dtype=np.uint8)).astype(np.float64)
    mag = _nearest_even_bruteforce(x, pos, np.arange(0, 127), lambda c: c % 2 == 0)
    want = mag | (np.signbit(x).astype(np.uint8) << 7)
    assert np.array_equal(O.encode_e4m3(x, saturate=False), want)
    # above the 464 midpoint the non-saturating cast gives NaN, the saturating one 448
    big = np.array([464.5, 470.0, 1e6, -1e6], dtype=np.float32)
    assert np.all((O.encode_e4m3(big, False) & 0x7F) == 0x7F)
    assert np.array_equal(O.encode_e4m3(big, True) & 0x7F, np.full(4, 0x7E, np.uint8))


def test_e2m1_roundtrip_and_bruteforce():
    codes = np.arange(16, dtype=np.uint8)
    assert np.array_equal(O.encode_e2m1(O.decode_e2m1(codes)), codes)
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.uniform(-7, 7, 5000), [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -5.0, 6.0, 100.0,
                                                  -100.0, 0.0, -0.0]]).astype(np.float32)
    pos = O.E2M1_VALUES[:8].astype(np.float64)
    mag = _nearest_even_bruteforce(np.clip(x, -6, 6), pos, np.arange(8), lambda c: c % 2 == 0)
    want = mag | (np.signbit(x).astype(np.uint8) << 3)
    assert np.array_equal(O.encode_e2m1(x), want)


def test_e8m0_pow2_closed_form_and_torch():
    e = np.arange(-127, 128)
    s = np.ldexp(1.0, e).astype(np.float32)
    b = O.encode_e8m0_pow2(s[1:])          # 2^-127 is subnormal: frexp still exact
    assert np.array_equal(b, (e[1:] + 127).astype(np.uint8))
    tv = torch.from_numpy(s[1:]).to(torch.float8_e8m0fnu).view(torch.uint8).numpy()
    assert np.array_equal(b, tv)
    assert O.encode_e8m0_pow2(np.float32(2.0 ** -39)) == 88 and O.encode_e8m0_pow2(np.float32(1.0)) == 127


def test_fp4_pack_unpack_roundtrip():
    # test/test_pack_unpack.py:123-138 round trip; nibble order test/test_mma_scaled.py:155-160
    rng = np.random.default_rng(2)
    raw = rng.integers(0, 256, (7, 16), dtype=np.uint8)
    un = O.unpack_fp4(raw)
    assert np.array_equal(un[:, 0::2], raw & 0xF) and np.array_equal(un[:, 1::2], raw >> 4)
    assert np.array_equal(O.pack_fp4(un), raw)


# ---- quantisers ------------------------------------------------------------------------------------
def _inputs(seed, shape, kind="randn"):
    g = torch.Generator().manual_seed(seed)
    if kind == "randn":
        return torch.randn(shape, generator=g)
    if kind == "rand":
        return torch.rand(shape, generator=g)
    return (torch.rand(shape, generator=g) * 12 - 6)


@pytest.mark.parametrize("kind", ["randn", "rand", "uniform6"])
def test_block_quantize_ceil_vs_literal_torch(kind):
    x = _inputs(3, (64, 256), kind)
    x[0, :32] = 0                      # all-zero block
    x[1, :32] = 448.0 * 2.0 ** -5      # amax/448 exactly a power of two
    xq_lit, s_lit = O.block_quantize_ceil_literal(x, 32)
    codes, sb = O.block_quantize(x.numpy(), 32, O.E4M3, "ceil")
    lit_s = s_lit.view(torch.uint8).numpy()
    lit_q = xq_lit.view(torch.uint8).numpy()
    same = lit_s == sb
    # the literal form differs only where fp32 log2 rounds 2^k(1+eps) down (rare); elsewhere bit-equal
    assert same.mean() > 0.999
    assert np.array_equal(np.repeat(same, 32, axis=1) * lit_q, np.repeat(same, 32, axis=1) * codes)
    assert sb[0, 0] == 88              # clamp(min=1e-12) -> 2^-39
    assert sb[1, 0] == 127 - 5
    # invariants: |x/scale| <= 448, so no NaN codes; dequant error <= 2^-4 relative for normals
    assert not np.any((codes & 0x7F) == 0x7F)
    deq = O.dequantize(codes, sb, O.E4M3).numpy()
    xn = x.numpy()
    big = np.abs(xn) > np.repeat(O.decode_e8m0(sb), 32, axis=1) * 2.0 ** -6
    assert np.all(np.abs(deq - xn)[big] <= np.abs(xn)[big] * 2.0 ** -4)


def test_block_quantize_ceil_log2_edge_case_is_exact():
    # v = 2^k (1 + 2^-23): exact ceil gives k+1 (the literal fp32 log2 form may give k)
    amax = np.float32(448.0) * np.float32(2.0 ** -8) * (np.float32(1.0) + np.float32(2.0 ** -23))
    v = np.float32(amax) / np.float32(448.0)
    m, e = np.frexp(v)
    x = np.zeros((1, 32), np.float32)
    x[0, 0] = amax
    _, sb = O.block_quantize(x, 32, O.E4M3, "ceil")
    want = (e - 1 if m == 0.5 else e) + 127
    assert sb[0, 0] == want


@pytest.mark.parametrize("fmt,emax,vmax", [(O.E4M3, 8, 448.0), (O.E2M1, 2, 6.0), (O.E5M2, 15, 57344.0)])
def test_block_quantize_floor_closed_form(fmt, emax, vmax):
    x = _inputs(4, (32, 128), "randn").numpy() * 3
    x[0, :32] = 0
    x[1, :32] = 0
    x[1, 5] = 1.0                      # amax = 1 -> scale 2^-emax
    x[2, :32] = np.linspace(-1.99, 1.99, 32)   # amax < 2 -> floor(log2) = 0 -> saturation must clamp
    codes, sb = O.block_quantize(x, 32, fmt, "floor")
    assert sb[0, 0] == 0
    assert sb[1, 0] == 127 - emax
    assert sb[2, 0] == 127 - emax
    # scale is 2^(floor(log2 amax) - emax): amax / scale in [2^emax, 2^(emax+1))
    amax = np.abs(x.reshape(32, 4, 32)).max(-1)
    sc = O.decode_e8m0(sb).astype(np.float64)
    nz = amax > 0
    ratio = amax[nz] / sc[nz]
    assert np.all((ratio >= 2.0 ** emax) & (ratio < 2.0 ** (emax + 1)))
    # saturating: every decoded magnitude <= max normal, no NaN codes
    dec = O.decode_elem(codes, fmt)
    assert not np.any(np.isnan(dec)) and np.all(np.abs(dec) <= vmax)
    # nearest: each element is within half a quantum (or clamped)
    deq = dec.reshape(32, 4, 32).astype(np.float64) * sc[..., None]
    xb = x.reshape(32, 4, 32)
    clamped = np.abs(xb) > vmax * sc[..., None]
    assert np.all(np.abs(deq)[clamped] == (vmax * np.broadcast_to(sc[..., None], xb.shape))[clamped])
    mbits, emin = {O.E4M3: (3, -6), O.E2M1: (1, 0), O.E5M2: (2, -14)}[fmt]
    half_min_quantum = sc[..., None].repeat(32, -1) * 2.0 ** (emin - mbits - 1)
    assert np.all(np.abs(deq - xb)[~clamped] <= np.maximum(np.abs(xb)[~clamped] * 2.0 ** -(mbits + 1),
                                                          half_min_quantum[~clamped]))


def test_block_quantize_padding_and_error():
    x = _inputs(5, (4, 40), "randn").numpy()
    codes, sb = O.block_quantize(x, 32, O.E4M3, "ceil")
    assert codes.shape == (4, 64) and sb.shape == (4, 2)
    assert np.all(codes[:, 40:] == 0)
    with pytest.raises(ValueError, match="larger than the inner most dimension"):
        O.block_quantize(np.zeros((2, 16), np.float32), 32)


# ---- scale layouts / tile order ------------------------------------------------------------------------
@pytest.mark.parametrize("M,Ks", [(128, 4), (256, 8), (384, 12)])
def test_swizzle_32_4_4_closed_form_and_roundtrip(M, Ks):
    s = np.arange(M * Ks, dtype=np.int64).reshape(M, Ks)
    sw = O.swizzle_32_4_4(s)
    assert sw.shape == (M // 128, Ks // 4, 32, 16)
    flat = sw.reshape(-1)
    for r in range(0, M, 7):
        for c in range(Ks):
            assert flat[O.swizzle_32_4_4_offset(r, c, Ks)] == s[r, c]
    assert sorted(flat.tolist()) == list(range(M * Ks))        # bijection
    assert np.array_equal(O.unswizzle_32_4_4(sw), s)            # round trip


@pytest.mark.parametrize("M,N,tm,tn", [(512, 512, 128, 128), (1000, 300, 128, 64), (256, 8192, 256, 256),
                                       (2304, 512, 256, 256)])
def test_swizzle_2d_is_a_bijection(M, N, tm, tn):
    nm, nn = -(-M // tm), -(-N // tn)
    seen = {O.swizzle_2d_from_bid(M, N, tm, tn, 8, b) for b in range(nm * nn)}
    assert seen == {(i, j) for i in range(nm) for j in range(nn)}


# ---- GEMM semantics --------------------------------------------------------------------------------------
def test_reference_matmul_known_answers():
    # src/cuda/tile/_stub.py:2248-2259: ones(2x64) . ones(64x2), all scales 2.0 -> 256.0
    one = O.encode_e4m3(np.ones((2, 64), np.float32), False)
    two = O.encode_e8m0_pow2(np.full((2, 2), 2.0, np.float32))
    r = O.reference_matmul(one, two, one.T.copy(), two.T.copy())
    assert torch.equal(r, torch.full((2, 2), 256.0))
    # src/cuda/tile/_stub.py:2309-2328: 128^3 ones, scales 2.0 -> 512.0
    one = O.encode_e4m3(np.ones((128, 128), np.float32), False)
    two = O.encode_e8m0_pow2(np.full((128, 4), 2.0, np.float32))
    r = O.reference_matmul(one, two, one.T.copy(), two.T.copy())
    assert r.unique().tolist() == [512.0]


def test_reference_matmul_bruteforce_float64_and_unit_scales():
    rng = np.random.default_rng(7)
    M, N, K = 5, 6, 64
    a = rng.integers(0, 256, (M, K), dtype=np.uint8)
    b = rng.integers(0, 256, (K, N), dtype=np.uint8)
    a[(a & 0x7F) == 0x7F] = 0
    b[(b & 0x7F) == 0x7F] = 0
    sa = rng.integers(120, 134, (M, K // 32), dtype=np.uint8)
    sb = rng.integers(120, 134, (K // 32, N), dtype=np.uint8)
    acc = torch.from_numpy(rng.normal(size=(M, N)).astype(np.float32))
    got = O.reference_matmul(a, sa, b, sb, acc=acc).double().numpy()
    av, bv = O.decode_e4m3(a).astype(np.float64), O.decode_e4m3(b).astype(np.float64)
    want = np.zeros((M, N))
    for i in range(M):
        for j in range(N):
            for k in range(K):
                want[i, j] += av[i, k] * 2.0 ** (int(sa[i, k // 32]) - 127) * bv[k, j] * 2.0 ** (int(sb[k // 32, j]) - 127)
    want += acc.numpy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # all scales 1.0 -> plain matmul of the decoded values
    ones_a, ones_b = np.full_like(sa, 127), np.full_like(sb, 127)
    got1 = O.reference_matmul(a, ones_a, b, ones_b)
    assert torch.equal(got1, torch.from_numpy(O.decode_e4m3(a)) @ torch.from_numpy(O.decode_e4m3(b)))


def test_reference_matmul_fp4_lut():
    # FP4 through the 16-entry LUT of test/test_mma_scaled.py:149-160
    rng = np.random.default_rng(8)
    ap = rng.integers(0, 256, (16, 32), dtype=np.uint8)
    a = O.unpack_fp4(ap)
    lut = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])
    low, high = torch.from_numpy(ap & 0xF).long(), torch.from_numpy(ap >> 4).long()
    want = torch.stack([lut[low], lut[high]], dim=-1).reshape(16, 64)
    assert torch.equal(torch.from_numpy(O.decode_e2m1(a)), want)


# ---- MoE grouping ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,topk,E,tile", [(7, 2, 4, 4), (48, 8, 64, 16), (5, 1, 8, 128), (64, 2, 3, 8)])
def test_moe_align_invariants(T, topk, E, tile):
    rng = np.random.default_rng(T * 31 + E)
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)])
    sorted_ids, eids = O.moe_align_tile_size(ids, tile, E)
    total = T * topk
    counts = np.bincount(ids.reshape(-1), minlength=E)
    assert len(sorted_ids) == int(((counts + tile - 1) // tile).sum()) * tile
    assert len(eids) == len(sorted_ids) // tile
    flat = ids.reshape(-1)
    real = sorted_ids[sorted_ids < total]
    assert sorted(real.tolist()) == list(range(total))                 # every slot exactly once
    for blk, e in enumerate(eids):
        chunk = sorted_ids[blk * tile:(blk + 1) * tile]
        live = chunk[chunk < total]
        assert np.all(flat[live] == e)                                 # one expert per block
        assert np.all(np.diff(live) > 0)                               # stable order inside a block
        assert np.all(chunk[len(live):] == total)                      # sentinel padding at the end
    for e in range(E):                                                 # stable across an expert's blocks
        mine = real[flat[real] == e]
        assert np.all(np.diff(mine) > 0)


def test_grouped_reference_matches_dense_per_token():
    rng = np.random.default_rng(11)
    T, K, N, E, topk = 6, 64, 8, 3, 2
    a, sa = O.block_quantize(rng.normal(size=(T, K)).astype(np.float32), 32, O.E4M3, "floor")
    w, sw = O.block_quantize(rng.normal(size=(E, N, K)).astype(np.float32), 32, O.E4M3, "floor")
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)])
    out = O.grouped_reference(a, sa, w, sw, ids)
    for t in range(T):
        for j in range(topk):
            e = ids[t, j]
            want = O.reference_matmul(a[t:t + 1], sa[t:t + 1], w[e].T.copy(), sw[e].T.copy())
            assert torch.allclose(out[t * topk + j], want[0], rtol=1e-6, atol=1e-6)


def test_silu_mul_matches_library_and_closed_forms():
    """silu_mul (test/kernels/fused_moe.py:85-108) against torch's silu in float64 and its limits."""
    rng = np.random.default_rng(5)
    a = (rng.standard_normal(100000) * 8).astype(np.float32)
    b = rng.standard_normal(100000).astype(np.float32)
    got = O.silu_mul(a, b).astype(np.float64)
    ref = (torch.nn.functional.silu(torch.from_numpy(a).double()) * torch.from_numpy(b).double()).numpy()
    assert np.all(np.abs(got - ref) <= 2e-6 * np.abs(ref) + 1e-37)
    one = np.ones(5, np.float32)
    out = O.silu_mul(np.array([0.0, 100.0, -100.0, 1e30, -1e30], np.float32), one)
    assert out[0] == 0.0 and out[1] == 100.0 and out[2] == 0.0 and out[3] == np.float32(1e30) and out[4] == 0.0
    assert O.silu_mul(np.array([1.0], np.float32), np.array([2.0], np.float32))[0] == pytest.approx(2 / (1 + np.exp(-1.0)), rel=1e-6)
    # a dropped minus sign or a swapped operand would show here: silu is not odd and gate comes first
    assert O.silu_mul(np.array([2.0], np.float32), np.array([0.0], np.float32))[0] == 0.0
    assert O.silu_mul(np.array([-2.0], np.float32), one[:1])[0] == pytest.approx(-2 / (1 + np.exp(2.0)), rel=1e-6)


def test_moe_forward_against_float64_dense_loop():
    """moe_forward against an independent float64 loop over (token, k) pairs (structure of torch_moe,
    samples/MoE.py:292-334), with the same intermediate rounding steps applied."""
    rng = np.random.default_rng(11)
    T, H, F, E, topk = 6, 64, 32, 3, 2
    hq, hs = O.block_quantize(rng.standard_normal((T, H)).astype(np.float32), 32, O.E4M3, "floor")
    w1q, w1s = O.block_quantize((rng.standard_normal((E, 2 * F, H)) * 0.3).astype(np.float32), 32, O.E4M3, "floor")
    w2q, w2s = O.block_quantize((rng.standard_normal((E, H, F)) * 0.3).astype(np.float32), 32, O.E4M3, "floor")
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)])
    wts = rng.random((T, topk)).astype(np.float32)
    got = O.moe_forward(hq, hs, w1q, w1s, w2q, w2s, wts, ids).numpy()
    h = O.dequantize(hq, hs, O.E4M3).double().numpy()
    want = np.zeros((T, H))
    for t in range(T):
        for j in range(topk):
            e = ids[t, j]
            w1 = O.dequantize(w1q[e], w1s[e], O.E4M3).double().numpy()
            w2 = O.dequantize(w2q[e], w2s[e], O.E4M3).double().numpy()
            gu = torch.tensor(w1 @ h[t]).float().bfloat16().float().numpy()
            act = O.silu_mul(gu[:F], gu[F:])
            aq, asc = O.block_quantize(act[None, :], 32, O.E4M3, "floor")
            want[t] += wts[t, j] * (w2 @ O.dequantize(aq, asc, O.E4M3).double().numpy()[0])
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4)
