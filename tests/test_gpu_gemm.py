"""GPU parity: the HIP block-scaled GEMM (through the C ABI) against the CPU oracle on the same
seeded inputs.  Tolerances: relative Frobenius error <= 1e-3 (fp32 output) / 8e-3 (bf16 output)."""
import numpy as np
import pytest
import torch

from mxutil import Operand, oracle_matmul, randn_operand, raw_operand
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-3, torch.bfloat16: 8e-3}
MFMA = ["mfma128", "mfma256", "mfma256w4", "pingpong", "pingpong32"]


def _run(ct, a: Operand, b: Operand, **kw):
    if kw.get("kernel") == "pingpong32" and (a.fmt, b.fmt) not in ((O.E4M3, O.E4M3), (O.E5M2, O.E5M2)):
        pytest.skip("the 32x32x64 ping-pong kernel takes 8-bit element formats only")
    return ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, a_format=a.fmt_kw,
                                  b_format=b.fmt_kw, **kw)


def _check(c, ref, out_dtype, what=""):
    assert c.dtype == out_dtype
    err = O.rel_fro(c.float().cpu(), ref)
    print(f"{what} rel_fro={err:.3e}", flush=True)
    assert err <= TOL[out_dtype], f"{what}: relative Frobenius error {err:.3e}"


@pytest.mark.parametrize("kernel", ["generic"] + MFMA)
def test_known_answers(ct, dev, kernel):
    # src/cuda/tile/_stub.py:2309-2328: 128^3 ones with all scales 2.0 -> 512.0 everywhere
    one = torch.ones((128, 128), device=dev).to(torch.float8_e4m3fn)
    two = torch.full((128, 4), 2.0, device=dev).to(torch.float8_e8m0fnu)
    c = ct.block_scaled_matmul(one, two, one.T, two.T, kernel=kernel)
    assert c.unique().tolist() == [512.0]


def test_known_answer_small_generic(ct, dev):
    # src/cuda/tile/_stub.py:2248-2259: ones(2x64) . ones(64x2), scales 2.0 -> 256.0
    x = torch.ones((2, 64), device=dev).to(torch.float8_e4m3fn)
    s = torch.full((2, 2), 2.0, device=dev).to(torch.float8_e8m0fnu)
    z = ct.mma_scaled(x, s, x.T.contiguous(), s.T.contiguous(), torch.zeros((2, 2), device=dev))
    assert z.tolist() == [[256.0, 256.0], [256.0, 256.0]]


FORMATS = [(O.E4M3, O.E4M3), (O.E5M2, O.E5M2), (O.E2M1, O.E2M1), (O.E4M3, O.E2M1)]


@pytest.mark.parametrize("kernel", MFMA)
@pytest.mark.parametrize("fa,fb", FORMATS, ids=lambda f: str(f))
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16], ids=str)
def test_gemm_aligned(ct, dev, kernel, fa, fb, out_dtype):
    M, N, K = 256, 512, 1024
    a = randn_operand(M, K, fa, 11, dev, "uniform6" if fa == O.E2M1 else "randn")
    b = randn_operand(N, K, fb, 12, dev, "uniform6" if fb == O.E2M1 else "randn")
    c = _run(ct, a, b, out_dtype=out_dtype, kernel=kernel)
    _check(c, oracle_matmul(a, b), out_dtype, f"{kernel} {fa}x{fb} {out_dtype}")


@pytest.mark.parametrize("kernel", MFMA)
@pytest.mark.parametrize("fa,fb", FORMATS, ids=lambda f: str(f))
@pytest.mark.parametrize("M,N,K", [(300, 200, 160), (1, 1, 32), (129, 257, 96), (64, 700, 544), (512, 772, 256),
                                   (520, 1032, 512)])
def test_gemm_ragged(ct, dev, kernel, fa, fb, M, N, K):
    """Edge tiles in M and N and a K that is a multiple of 32 but not of the K tile: zero padding of
    test/kernels/scaled_matmul.py:66-104.  The last two shapes mix interior and edge tiles of the 256x256
    kernels, once with an output pitch that allows their 16-byte bf16 stores (1032) and once without (772)."""
    a = randn_operand(M, K, fa, 21, dev)
    b = randn_operand(N, K, fb, 22, dev)
    for out_dtype in (torch.float32, torch.bfloat16):
        c = _run(ct, a, b, out_dtype=out_dtype, kernel=kernel)
        _check(c, oracle_matmul(a, b), out_dtype, f"{kernel} {fa}x{fb} {M}x{N}x{K} {out_dtype}")


@pytest.mark.parametrize("kernel", ["generic"] + MFMA)
def test_sample_shape_rand_inputs_both_scale_layouts(ct, dev, kernel):
    """samples/BlockScaledMatMul.py:323-364: 512x512x768, torch.rand inputs, ceil-rule quantiser, plain and
    swizzle_32_4_4 scales, assert_close(atol=1e-4, rtol=1e-3)."""
    a = randn_operand(512, 768, O.E4M3, 31, dev, "rand", "ceil")
    b = randn_operand(512, 768, O.E4M3, 32, dev, "rand", "ceil")
    ref = oracle_matmul(a, b)
    c = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, kernel=kernel)
    torch.testing.assert_close(c.cpu(), ref, atol=1e-4, rtol=1e-3)
    a_sw = ct.swizzle_32_4_4(a.scale_t)
    b_sw = ct.swizzle_32_4_4(b.scale_t.T.T.contiguous())  # (N, K/32), as the sample passes it
    c2 = ct.block_scaled_matmul(a.storage, a_sw, b.storage.T, b_sw, kernel=kernel)
    torch.testing.assert_close(c2.cpu(), ref, atol=1e-4, rtol=1e-3)
    assert torch.equal(c, c2)


@pytest.mark.parametrize("kernel", MFMA)
def test_prepacked_scales_and_accumulate(ct, dev, kernel):
    a = randn_operand(256, 512, O.E4M3, 41, dev)
    b = randn_operand(384, 512, O.E4M3, 42, dev)
    ref = oracle_matmul(a, b)
    pa = ct.pack_scales(a.scale_t, operand="a", kernel=kernel)
    pb = ct.pack_scales(b.scale_t.T, transposed=True, operand="b", kernel=kernel)
    c = ct.block_scaled_matmul(a.storage, pa, b.storage.T, pb, kernel=kernel)
    c_plain = _run(ct, a, b, kernel=kernel)
    assert torch.equal(c, c_plain)
    _check(c, ref, torch.float32, "prepacked")
    g = torch.Generator().manual_seed(43)
    z = torch.randn((256, 384), generator=g)
    acc = z.to(dev)
    out = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, C=acc, accumulate=True,
                                 kernel=kernel)
    assert out.data_ptr() == acc.data_ptr()
    _check(out, ref + z, torch.float32, "accumulate")


@pytest.mark.parametrize("kernel", MFMA + ["generic"])
def test_raw_bytes_with_nan_codes(ct, dev, kernel):
    """test/test_mma_scaled.py:103-125 feeds raw random bytes, NaN encodings included; NaNs must propagate
    to exactly the rows/columns the oracle says (assert_close with equal_nan)."""
    a = raw_operand(64, 256, O.E4M3, 51, dev, allow_nan=True)
    b = raw_operand(48, 256, O.E4M3, 52, dev, allow_nan=True)
    ref = oracle_matmul(a, b)
    c = _run(ct, a, b, kernel=kernel).cpu()
    assert torch.equal(torch.isnan(c), torch.isnan(ref))
    torch.testing.assert_close(c, ref, atol=1e-2, rtol=1e-2, equal_nan=True)


def test_auto_dispatch_matches_explicit(ct, dev):
    a = randn_operand(384, 1024, O.E4M3, 61, dev)
    b = randn_operand(1536, 1024, O.E4M3, 62, dev)
    ref = oracle_matmul(a, b)
    _check(_run(ct, a, b), ref, torch.float32, "auto")
    # a layout the MFMA kernels cannot take (row-major K x N operand) goes to the general kernel
    b_rowmajor = b.storage.T.contiguous()
    bs_rowmajor = b.scale_t.T.contiguous()
    c = ct.block_scaled_matmul(a.storage, a.scale_t, b_rowmajor, bs_rowmajor)
    _check(c, ref, torch.float32, "auto->generic")
    with pytest.raises(ct.TileTypeError, match="cannot run this problem"):
        ct.block_scaled_matmul(a.storage, a.scale_t, b_rowmajor, bs_rowmajor, kernel="mfma128")


def test_concurrent_launch_threads(ct, dev):
    """test/test_concurrent_launch.py:49-72: several Python threads launching at once.  Every thread has its
    own operands and scales (different shapes too), so a scale re-layout of one thread landing between
    another thread's re-layout and GEMM launches would show as a wrong result."""
    import threading
    cases = []
    for t in range(8):
        a = randn_operand(128 + 64 * (t % 3), 256 + 128 * (t % 2), O.E4M3, 710 + t, dev, std=1.0 + t)
        b = randn_operand(128 + 32 * (t % 4), 256 + 128 * (t % 2), O.E4M3, 720 + t, dev)
        cases.append((a, b, _run(ct, a, b)))
    torch.cuda.synchronize()
    errs = []

    def work(t):
        a, b, want = cases[t]
        try:
            outs = [_run(ct, a, b) for _ in range(50)]
            torch.cuda.synchronize()
            if not all(torch.equal(c, want) for c in outs):
                errs.append(f"thread {t}: mismatch")
        except Exception as e:  # noqa: BLE001
            errs.append(repr(e))

    ts = [threading.Thread(target=work, args=(t,)) for t in range(8)]
    [t.start() for t in ts]
    [t.join() for t in ts]
    assert not errs, errs
    for a, b, want in cases:
        _check(want, oracle_matmul(a, b), torch.float32, "threads")


@pytest.mark.parametrize("kernel", ["generic"] + MFMA + ["auto"])
def test_config_c1_mxfp8_512_floor_fp32(ct, dev, kernel):
    """The CPU-reference configuration of the metric: M = N = K = 512, A and B^T drawn N(0, 1) from seed 1234,
    quantised by the oracle with the floor rule, fp32 output, every kernel; the input recipe and the check
    mirror samples/BlockScaledMatMul.py:323-364."""
    g = torch.Generator().manual_seed(1234)
    a = torch.randn((512, 512), generator=g)
    bt = torch.randn((512, 512), generator=g)
    ac, asc = O.block_quantize(a.numpy(), 32, O.E4M3, "floor")
    bc, bsc = O.block_quantize(bt.numpy(), 32, O.E4M3, "floor")
    A, B = Operand(ac, asc, O.E4M3, dev), Operand(bc, bsc, O.E4M3, dev)
    ref = oracle_matmul(A, B)
    c = _run(ct, A, B, out_dtype=torch.float32, kernel=kernel)
    _check(c, ref, torch.float32, f"C1 {kernel}")
    # the device quantiser produces the same operands from the same fp32 inputs
    aq, asq = ct.block_quantize(a.to(dev), 32, scale_mode="floor")
    assert np.array_equal(aq.view(torch.uint8).cpu().numpy(), ac) and np.array_equal(asq.view(torch.uint8).cpu().numpy(), asc)


@pytest.mark.parametrize("kernel", ["auto", "generic", "mfma128"])
def test_list_of_problems(ct, dev, kernel):
    """The list API (block-scaled counterpart of grouped_matmul_kernel, test/kernels/group_gemm.py:10-38;
    the reference's test, test/test_group_gemm.py, also mixes problem sizes): every problem of a list with
    different sizes and element formats matches its own oracle product; an empty problem is skipped."""
    shapes = [(128, 256, 512, O.E4M3, O.E4M3), (33, 80, 96, O.E4M3, O.E2M1), (300, 130, 2048, O.E2M1, O.E2M1),
              (0, 64, 64, O.E4M3, O.E4M3), (512, 512, 1024, O.E5M2, O.E5M2)]
    ops = [(randn_operand(m, k, fa, 900 + i, dev), randn_operand(n, k, fb, 950 + i, dev))
           for i, (m, n, k, fa, fb) in enumerate(shapes)]
    got = ct.grouped_block_scaled_matmul([a.storage if a.fmt != O.E2M1 else a.storage.view(torch.float4_e2m1fn_x2)
                                          for a, _ in ops],
                                         [a.scale_t for a, _ in ops],
                                         [(b.storage if b.fmt != O.E2M1 else b.storage.view(torch.float4_e2m1fn_x2)).T
                                          for _, b in ops],
                                         [b.scale_t.T for _, b in ops], kernel=kernel)
    assert len(got) == len(shapes)
    for (a, b), c, (m, n, k, _, _) in zip(ops, got, shapes):
        assert tuple(c.shape) == (m, n)
        if m:
            _check(c, oracle_matmul(a, b), torch.float32, f"list {m}x{n}x{k}")


def test_list_of_many_small_problems_matches_single_calls(ct, dev):
    """test/test_group_gemm.py:14-34 drives grouped_matmul_kernel with lists of small problems, tiles larger than
    a problem included.  70 problems (more than one persistent launch takes), ragged sizes from one tile row to a
    few tiles, two element formats interleaved, one problem large enough to leave the batched path: every
    result is bit-identical to the same problem run alone, and within tolerance of the oracle."""
    rng = np.random.default_rng(5)
    As, Ass, Bs, Bss, single = [], [], [], [], []
    ops = []
    for i in range(70):
        m, n, k = int(rng.integers(1, 300)), int(rng.integers(1, 300)), 32 * int(rng.integers(1, 20))
        if i == 40:
            m, n, k = 3072, 3072, 512      # 144 tiles of 256 x 256: goes to the persistent 256 x 256 kernel
        fmt = O.E4M3 if i % 3 else O.E5M2
        a, b = randn_operand(m, k, fmt, 2000 + i, dev), randn_operand(n, k, fmt, 3000 + i, dev)
        ops.append((a, b))
        As.append(a.storage); Ass.append(a.scale_t); Bs.append(b.storage.T); Bss.append(b.scale_t.T)
        single.append(_run(ct, a, b))
    got = ct.grouped_block_scaled_matmul(As, Ass, Bs, Bss)
    for i, ((a, b), c, c1) in enumerate(zip(ops, got, single)):
        assert torch.equal(c, c1), i
        if i % 10 == 0:
            _check(c, oracle_matmul(a, b), torch.float32, f"list problem {i}")


def test_list_of_problems_reports_the_failing_index(ct, dev):
    a = randn_operand(64, 64, O.E4M3, 1, dev)
    b = randn_operand(64, 64, O.E4M3, 2, dev)
    bad_scale = torch.zeros((64, 3), dtype=torch.uint8, device=dev).view(torch.float8_e8m0fnu)
    with pytest.raises(Exception, match="problem 1 of the list"):
        ct.grouped_block_scaled_matmul([a.storage, a.storage], [a.scale_t, bad_scale],
                                       [b.storage.T, b.storage.T], [b.scale_t.T, b.scale_t.T])


@pytest.mark.parametrize("M,N,K,split_k", [(64, 256, 8192, 0), (200, 130, 4096, 4), (128, 128, 16384, 0),
                                           (96, 512, 2048, 2), (33, 64, 1024, 2)])
@pytest.mark.parametrize("fa,fb,out_dtype", [(O.E4M3, O.E4M3, torch.float32), (O.E4M3, O.E2M1, torch.bfloat16)])
def test_split_k(ct, dev, M, N, K, split_k, fa, fb, out_dtype):
    """Small M x N with a long K: slices of K run side by side and a second kernel adds the fp32 partials
    (the scheme of matmul_split_k_kernel, test/kernels/matmul.py:103-140).  Automatic (0) and forced splits,
    ragged M / N, with and without accumulation into C; M > 32 keeps the mixed-format case off the decode kernel."""
    a, b = randn_operand(M, K, fa, 700 + M, dev), randn_operand(N, K, fb, 800 + N, dev)
    ref = oracle_matmul(a, b)
    c = _run(ct, a, b, out_dtype=out_dtype, split_k=split_k)
    _check(c, ref, out_dtype, f"split_k={split_k} {M}x{N}x{K}")
    c1 = _run(ct, a, b, out_dtype=out_dtype, split_k=1)
    _check(c1, ref, out_dtype, "unsplit")
    z = torch.randn((M, N), generator=torch.Generator().manual_seed(5)).to(out_dtype)
    acc = z.to(dev).clone()
    _run(ct, a, b, C=acc, accumulate=True, split_k=split_k)
    _check(acc, ref + z.float(), out_dtype, "split-K accumulate")


def test_split_k_rejects_impossible_requests(ct, dev):
    a, b = randn_operand(64, 1536, O.E4M3, 1, dev), randn_operand(64, 1536, O.E4M3, 2, dev)
    with pytest.raises(Exception, match="multiple of"):
        _run(ct, a, b, split_k=2)          # 1536 is not a multiple of 1024
    with pytest.raises(Exception, match="one-tile MFMA kernels"):
        _run(ct, a, b, split_k=3, kernel="generic")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("M,N,K", [(256, 256, 512), (512, 768, 1024), (300, 520, 384), (256, 256, 416), (3072, 3072, 1024),
                                   (1, 1, 384), (777, 1030, 4096)])
def test_four_wave_persistent_kernel(ct, dev, fmt, M, N, K):
    """The four-wave kernel (128 x 128 per wave, 32x32x64 instruction, five-buffer half-stage ring): aligned and
    ragged shapes, a K that ends inside a half-stage and inside a K-quad, more tiles than workgroups' first
    round, fp32 and bf16 output with and without accumulation."""
    a, b = randn_operand(M, K, fmt, 31, dev), randn_operand(N, K, fmt, 32, dev)
    ref = oracle_matmul(a, b)
    for out_dtype in (torch.float32, torch.bfloat16):
        c = _run(ct, a, b, out_dtype=out_dtype, kernel="w4p")
        _check(c, ref, out_dtype, f"w4p {fmt} {M}x{N}x{K} {out_dtype}")
    z = torch.randn((M, N), generator=torch.Generator().manual_seed(33))
    acc = z.to(dev)
    _run(ct, a, b, C=acc, accumulate=True, kernel="w4p")
    _check(acc, ref + z, torch.float32, "w4p accumulate")


def test_four_wave_kernel_rejects_what_it_cannot_run(ct, dev):
    a, b = randn_operand(256, 256, O.E4M3, 1, dev), randn_operand(256, 256, O.E4M3, 2, dev)
    with pytest.raises(ct.TileTypeError, match="K >= 384"):
        _run(ct, a, b, kernel="w4p")
    a4, b4 = randn_operand(256, 512, O.E2M1, 1, dev), randn_operand(256, 512, O.E2M1, 2, dev)
    with pytest.raises(ct.TileTypeError, match="8-bit"):
        _run(ct, a4, b4, kernel="w4p")


def test_cached_scale_relayout(ct, dev):
    """cache_scales=True: same bits as without, one re-layout per live scale tensor, recomputed after torch writes
    to the tensor, and no effect on problems the general kernel runs."""
    from cutile_amd import ops
    ct.clear_scale_cache()
    a = randn_operand(256, 512, O.E4M3, 71, dev)
    b = randn_operand(384, 512, O.E4M3, 72, dev)
    bs_t = b.scale_t.T                      # the view the sample passes; a new view object per call below
    plain = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, bs_t)
    c1 = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, cache_scales=True)
    assert len(ops._SCALE_CACHE._entries) == 2
    c2 = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, cache_scales=True)
    assert len(ops._SCALE_CACHE._entries) == 2, "second call must hit both entries"
    assert torch.equal(plain, c1) and torch.equal(plain, c2)
    # swizzle_32_4_4 input
    a_sw = ct.swizzle_32_4_4(a.scale_t)
    c3 = ct.block_scaled_matmul(a.storage, a_sw, b.storage.T, b.scale_t.T, cache_scales=True)
    assert torch.equal(plain, c3)
    # torch writes to the scales: the stale copy must not be used
    a.scale_t.view(torch.uint8).add_(1)     # every A scale doubled
    c4 = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, cache_scales=True)
    assert torch.equal(c4, plain * 2)
    # another stream uses the cached copy behind the event of the re-layout
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        c5 = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, cache_scales=True)
    s.synchronize()
    assert torch.equal(c5, c4)
    # the entry is dropped while a GEMM on the other stream still reads the cached copy: the copy's block must not
    # be handed out again before that GEMM is done (new allocations of the same size right behind the clear)
    big_a = randn_operand(2048, 4096, O.E4M3, 73, dev)
    big_b = randn_operand(2048, 4096, O.E4M3, 74, dev)
    want = ct.block_scaled_matmul(big_a.storage, big_a.scale_t, big_b.storage.T, big_b.scale_t.T)
    ct.block_scaled_matmul(big_a.storage, big_a.scale_t, big_b.storage.T, big_b.scale_t.T, cache_scales=True)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        for _ in range(4):                   # a few launches deep, so the last one is still queued at the clear
            c7 = ct.block_scaled_matmul(big_a.storage, big_a.scale_t, big_b.storage.T, big_b.scale_t.T,
                                        cache_scales=True)
    ct.clear_scale_cache()
    junk = [torch.full((ct.lib().mx_packed_scale_bytes(2048, 4096),), 0xFF, dtype=torch.uint8, device=dev)
            for _ in range(4)]
    s.synchronize()
    torch.cuda.synchronize()
    assert torch.equal(c7, want)
    del junk
    # a problem of the general kernel (row-major B) ignores the cache
    b_rm = b.storage.T.contiguous()
    ref = ct.block_scaled_matmul(a.storage, a.scale_t, b_rm, b.scale_t.T)
    c6 = ct.block_scaled_matmul(a.storage, a.scale_t, b_rm, b.scale_t.T, cache_scales=True)
    assert torch.equal(ref, c6)
    # a dead tensor's entry never matches a new tensor at the same address
    n_before = len(ops._SCALE_CACHE._entries)
    del a_sw
    ct.clear_scale_cache()
    assert len(ops._SCALE_CACHE._entries) == 0 and n_before >= 2


def test_drop_in_signature_caches_scale_relayout(ct, dev):
    """cutile_block_scaled_matmul(A, A_scale, B, B_scale) -> fp32 C (samples/BlockScaledMatMul.py:229-297): same bits
    as the general entry, the scale re-layout kept between calls, redone after torch writes to a scale tensor."""
    from cutile_amd import ops
    ct.clear_scale_cache()
    a = randn_operand(512, 768, O.E4M3, 75, dev)
    b = randn_operand(512, 768, O.E4M3, 76, dev)
    a_sw, b_sw = ct.swizzle_32_4_4(a.scale_t), ct.swizzle_32_4_4(b.scale_t)     # as the sample passes them
    want = ct.block_scaled_matmul(a.storage, a_sw, b.storage.T, b_sw)
    c1 = ct.cutile_block_scaled_matmul(a.storage, a_sw, b.storage.T, b_sw)
    c2 = ct.cutile_block_scaled_matmul(a.storage, a_sw, b.storage.T, b_sw)
    assert c1.dtype == torch.float32 and torch.equal(c1, want) and torch.equal(c2, want)
    assert len(ops._SCALE_CACHE._entries) == 2
    assert O.rel_fro(c1.cpu(), oracle_matmul(a, b)) <= 1e-3
    a_sw.view(torch.uint8).add_(1)                                              # every A scale doubled, through torch
    c3 = ct.cutile_block_scaled_matmul(a.storage, a_sw, b.storage.T, b_sw)
    assert torch.equal(c3, want * 2)
    ct.clear_scale_cache()
