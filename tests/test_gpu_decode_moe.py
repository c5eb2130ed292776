"""GPU parity of the skinny-M weight-streaming kernel and of the grouped (MoE) GEMM."""
import numpy as np
import pytest
import torch

from mxutil import oracle_matmul, randn_operand
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("M,N,K", [(32, 256, 1024), (7, 1792, 2048), (16, 48, 512), (32, 4096, 8192), (1, 16, 4096),
                                   (17, 4176, 4096), (29, 12320, 8192), (32, 16, 8192), (24, 36864, 4096),
                                   (8, 20480, 4096), (16, 16400, 8192),
                                   # K that ends inside the kernel's K-slices: lanes beyond K fetch nothing
                                   (32, 1792, 7168), (9, 528, 5120), (32, 272, 3072), (16, 64, 1536), (32, 4112, 6144),
                                   # K beyond one launch's 8192: chunks summed in fp32 (down-projection shapes)
                                   (32, 512, 14336), (5, 1040, 28672), (17, 64, 8704)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=str)
def test_decode_kernel(ct, dev, M, N, K, out_dtype):
    x = randn_operand(M, K, O.E4M3, 81, dev)
    w = randn_operand(N, K, O.E2M1, 82, dev, std=0.02)
    ref = oracle_matmul(x, w)
    c = ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1",
                               out_dtype=out_dtype, kernel="decode")
    err = O.rel_fro(c.float().cpu(), ref)
    print(f"decode {M}x{N}x{K} {out_dtype} rel_fro={err:.3e}", flush=True)
    assert err <= (1e-3 if out_dtype == torch.float32 else 8e-3)
    # the automatic choice for this shape family is the same kernel
    c2 = ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1",
                                out_dtype=out_dtype)
    assert torch.equal(c, c2)
    # and the tiled MFMA kernel agrees within tolerance
    c3 = ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1",
                                out_dtype=out_dtype, kernel="mfma128")
    assert O.rel_fro(c3.float().cpu(), ref) <= (1e-3 if out_dtype == torch.float32 else 8e-3)


def test_decode_long_k_accumulate_and_static_scratch(ct, dev):
    """K = 14336 through the chunked path: C += into bf16 (the conversion pass adds the old C once, in fp32) and the
    library's static scratch as the chunk buffer."""
    M, N, K = 24, 336, 14336
    x = randn_operand(M, K, O.E4M3, 181, dev)
    w = randn_operand(N, K, O.E2M1, 182, dev, std=0.02)
    ref = oracle_matmul(x, w)
    z = torch.randn((M, N), generator=torch.Generator().manual_seed(183)).to(torch.bfloat16)
    acc = z.to(dev)
    ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1", C=acc, accumulate=True)
    assert O.rel_fro(acc.float().cpu(), ref + z.float()) <= 8e-3
    c = ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1", static_scratch=True)
    c2 = ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1", kernel="decode")
    assert torch.equal(c, c2) and O.rel_fro(c.cpu(), ref) <= 1e-3


@pytest.mark.parametrize("M,N,K,kernel", [(48, 528, 4096, "auto"), (64, 1040, 8192, "auto"), (33, 64, 14336, "auto"),
                                          (100, 272, 2048, "decode"), (128, 64, 9216, "decode")])
def test_decode_more_than_32_rows(ct, dev, M, N, K, kernel):
    """More than 32 rows of X run slab by slab on the same kernel (the automatic choice up to 64 rows)."""
    x = randn_operand(M, K, O.E4M3, 281, dev)
    w = randn_operand(N, K, O.E2M1, 282, dev, std=0.02)
    ref = oracle_matmul(x, w)
    for out_dtype, tol in ((torch.float32, 1e-3), (torch.bfloat16, 8e-3)):
        c = ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1",
                                   out_dtype=out_dtype, kernel=kernel)
        assert O.rel_fro(c.float().cpu(), ref) <= tol
        # the slabs are what single calls on 32 rows give
        c0 = ct.block_scaled_matmul(x.storage[:32], x.scale_t[:32], w.storage.T, w.scale_t.T, b_format="e2m1",
                                    out_dtype=out_dtype, kernel="decode")
        assert torch.equal(c[:32], c0)


def test_decode_accumulate(ct, dev):
    x = randn_operand(32, 1024, O.E4M3, 83, dev)
    w = randn_operand(64, 1024, O.E2M1, 84, dev)
    z = torch.randn((32, 64), generator=torch.Generator().manual_seed(85))
    acc = z.to(dev)
    ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1", C=acc,
                           accumulate=True, kernel="decode")
    assert O.rel_fro(acc.cpu(), oracle_matmul(x, w) + z) < 1e-3


@pytest.mark.parametrize("T,topk,E,tile", [(7, 2, 4, 4), (48, 8, 64, 16), (5, 1, 8, 128), (4096, 2, 8, 256),
                                           (110, 4, 16, 128), (256, 6, 1408, 128), (1024, 8, 128, 256), (333, 3, 256, 64),
                                           (3, 1, 200, 32)])
def test_moe_align_matches_oracle(ct, dev, T, topk, E, tile):
    """test/kernels/fused_moe.py:113-173; shapes from samples/MoE.py:420-462 and test/bench_moe.py:16-24."""
    g = torch.Generator().manual_seed(T + E)
    ids = torch.topk(torch.rand((T, E), generator=g), topk, dim=1).indices
    want_ids, want_e = O.moe_align_tile_size(ids.numpy(), tile, E)
    got_ids, got_e = ct.moe_align_tile_size(ids.to(dev), tile, E)
    assert got_ids.dtype == torch.int32 and got_e.dtype == torch.int32
    assert np.array_equal(got_ids.cpu().numpy(), want_ids)
    assert np.array_equal(got_e.cpu().numpy(), want_e)
    # without the trim nothing synchronises; the tail is sentinel / expert 0
    all_ids, all_e = ct.moe_align_tile_size(ids.to(dev), tile, E, exact=False)
    assert np.array_equal(all_ids[:len(want_ids)].cpu().numpy(), want_ids)
    assert bool((all_ids[len(want_ids):] == T * topk).all()) and bool((all_e[len(want_e):] == 0).all())


@pytest.mark.parametrize("n,E,tile,skew", [(200_000, 3, 256, True), (70_000, 1, 128, False), (300_000, 300, 64, True),
                                          (5000, 8, 256, False), (1025, 5, 16, False), (1024, 5, 16, False)])
def test_moe_align_many_ids_per_expert(ct, dev, n, E, tile, skew):
    """Routings that span many workgroups: one expert holding more than 65535 ids (a 16-bit running count
    would wrap), more than 256 experts (the ballot placement) over several chunks, and sizes either side of
    the one-workgroup limit."""
    rng = np.random.default_rng(n + E)
    if skew:
        p = np.full(E, 0.1 / max(E - 1, 1))
        p[E // 2] = 0.9
        ids = rng.choice(E, size=n, p=p / p.sum()).astype(np.int32)
    else:
        ids = rng.integers(0, E, size=n, dtype=np.int32)
    want_ids, want_e = O.moe_align_tile_size(ids.reshape(-1, 1), tile, E)
    got_ids, got_e = ct.moe_align_tile_size(torch.from_numpy(ids).to(dev).reshape(-1, 1), tile, E)
    assert np.array_equal(got_ids.cpu().numpy(), want_ids)
    assert np.array_equal(got_e.cpu().numpy(), want_e)
    all_ids, all_e = ct.moe_align_tile_size(torch.from_numpy(ids).to(dev).reshape(-1, 1), tile, E, exact=False)
    assert bool((all_ids[len(want_ids):] == n).all()) and bool((all_e[len(want_e):] == 0).all())


def _moe_case(T, K, N, E, topk, seed, dev, w_std=0.1):
    a = randn_operand(T, K, O.E4M3, seed, dev, std=0.5)
    w = randn_operand(E * N, K, O.E4M3, seed + 1, dev, std=w_std)
    g = torch.Generator().manual_seed(seed + 2)
    ids = torch.topk(torch.rand((T, E), generator=g), topk, dim=1).indices
    ref = O.grouped_reference(a.codes, a.scales, w.codes.reshape(E, N, K), w.scales.reshape(E, N, K // 32),
                              ids.numpy())
    W = w.storage.view(E, N, K)
    Ws = w.scale_t.view(E, N, K // 32)
    return a, W, Ws, ids, ref


@pytest.mark.parametrize("kernel,tile", [("generic", 16), ("generic", 128), ("mfma128", 128), ("mfma128", 256),
                                         ("mfma256", 256), ("mfma256w4", 256), ("pingpong", 256), ("pingpong32", 256), ("auto", 128), ("auto", 256)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=str)
def test_grouped_gemm_sample_shape(ct, dev, kernel, tile, out_dtype):
    """samples/MoE.py:420-462 shape: 48 tokens, hidden 512, 64 experts, top-8; N = 1024."""
    T, K, N, E, topk = 48, 512, 1024, 64, 8
    a, W, Ws, ids, ref = _moe_case(T, K, N, E, topk, 91, dev)
    sid, eid = ct.moe_align_tile_size(ids.to(dev), tile, E)
    C = torch.full((T, topk, N), float("nan"), device=dev, dtype=out_dtype)
    ct.invoke_fused_moe_scaled(a.storage, a.scale_t, W, Ws, C, None, sid, eid, False, topk, tile, kernel=kernel)
    err = O.rel_fro(C.view(-1, N).float().cpu(), ref)
    print(f"grouped {kernel} tile={tile} {out_dtype} rel_fro={err:.3e}", flush=True)
    assert err <= (1e-3 if out_dtype == torch.float32 else 8e-3)


@pytest.mark.parametrize("K,x_fmt", [(4096, O.E4M3), (8192, O.E4M3)])
def test_decode_two_halves_accumulate(ct, dev, K, x_fmt):
    """16 < M <= 32 at K = 4096 / 8192 runs the variant whose waves split M as well as K: E5M2 activations,
    C += into fp32 and bf16 (test_decode_kernel covers the ragged and the more-than-one-batch tile splits)."""
    M, N = 27, 16 * 300
    x = randn_operand(M, K, x_fmt, 86, dev)
    w = randn_operand(N, K, O.E2M1, 87, dev, std=0.02)
    ref = oracle_matmul(x, w)
    for out_dtype, tol in ((torch.float32, 1e-3), (torch.bfloat16, 8e-3)):
        z = torch.randn((M, N), generator=torch.Generator().manual_seed(88)).to(out_dtype)
        acc = z.to(dev)
        ct.block_scaled_matmul(x.storage, x.scale_t, w.storage.T, w.scale_t.T, b_format="e2m1", C=acc,
                               accumulate=True, kernel="decode")
        assert O.rel_fro(acc.float().cpu(), ref + z.float()) <= tol


@pytest.mark.parametrize("kernel", ["generic", "mfma128", "mfma256", "pingpong", "pingpong32"])
def test_grouped_gemm_routed_weight_replicas1_and_padded_ids(ct, dev, kernel):
    """Second GEMM of the sample: replicas = 1, rows multiplied by the routed weight
    (test/kernels/fused_moe.py:75-77); index arrays left at their worst-case length."""
    T, K, N, E, topk = 300, 256, 384, 8, 1
    a, W, Ws, ids, ref = _moe_case(T, K, N, E, topk, 95, dev)
    wts = torch.rand((T, topk), generator=torch.Generator().manual_seed(96))
    sid, eid = ct.moe_align_tile_size(ids.to(dev), 256, E, exact=False)
    C = torch.zeros((T * topk, N), device=dev, dtype=torch.float32)
    ct.invoke_fused_moe_scaled(a.storage, a.scale_t, W, Ws, C, wts.to(dev), sid, eid, True, 1, 256, kernel=kernel)
    assert O.rel_fro(C.cpu(), ref * wts.reshape(-1, 1)) < 1e-3
    # pre-packed expert scales give the same bits
    if kernel != "generic":
        C2 = torch.zeros_like(C)
        ct.invoke_fused_moe_scaled(a.storage, a.scale_t, W, ct.pack_scales(Ws, operand="b", kernel=kernel), C2, wts.to(dev), sid, eid, True, 1,
                                   256, kernel=kernel)
        assert torch.equal(C, C2)
        # bf16 output (the full-vector store path of the scatter epilogue where the tile's columns are inside N)
        C3 = torch.zeros((T * topk, N), device=dev, dtype=torch.bfloat16)
        ct.invoke_fused_moe_scaled(a.storage, a.scale_t, W, Ws, C3, wts.to(dev), sid, eid, True, 1, 256, kernel=kernel)
        assert O.rel_fro(C3.float().cpu(), ref * wts.reshape(-1, 1)) < 8e-3


@pytest.mark.parametrize("kernel", ["generic", "mfma128", "mfma256", "pingpong", "pingpong32"])
def test_grouped_gemm_sentinels_anywhere_and_expert_ids_out_of_range(ct, dev, kernel):
    """Caller-built index arrays: the sentinel may sit in any slot of a tile (here in the first slot of each
    128-row half, with routed rows behind it), as fused_moe_kernel masks slot by slot
    (test/kernels/fused_moe.py:40-47); blocks whose expert id lies outside [0, E) hold only sentinels and must not
    make the kernel read outside W."""
    T, K, N, E, topk = 200, 256, 512, 4, 1
    a, W, Ws, ids, ref = _moe_case(T, K, N, E, topk, 97, dev)
    flat = ids.reshape(-1).numpy()
    sent = T * topk
    slots, experts = [], []
    for e in range(E):
        mine = np.nonzero(flat == e)[0].astype(np.int32)
        assert 2 <= len(mine) <= 254
        half = len(mine) // 2
        block = np.full(256, sent, dtype=np.int32)
        block[1:1 + half] = mine[:half]                      # slot 0 stays a sentinel
        block[129:129 + len(mine) - half] = mine[half:]      # and so does slot 128
        slots.append(block)
        experts.append(e)
    for bad in (E + 5, -3, 2 ** 30):
        slots.append(np.full(256, sent, dtype=np.int32))
        experts.append(bad)
    sid = torch.from_numpy(np.concatenate(slots)).to(dev)
    eid = torch.tensor(experts, dtype=torch.int32, device=dev)
    for out_dtype, tol in ((torch.float32, 1e-3), (torch.bfloat16, 8e-3)):
        C = torch.full((T * topk, N), float("nan"), device=dev, dtype=out_dtype)
        ct.invoke_fused_moe_scaled(a.storage, a.scale_t, W, Ws, C, None, sid, eid, False, topk, 256, kernel=kernel)
        torch.cuda.synchronize()
        assert O.rel_fro(C.float().cpu(), ref) <= tol


@pytest.mark.parametrize("kernel,tile_m", [("auto", 128), ("auto", 256), ("generic", 16)])
@pytest.mark.parametrize("w_fmt", [O.E4M3, O.E2M1])
def test_moe_pipeline_matches_oracle(ct, dev, kernel, tile_m, w_fmt):
    """cutile_moe_scaled (structure of cutile_moe, samples/MoE.py:197-288) against the oracle's
    moe_forward.  The intermediate is rounded to bf16 and re-quantised on both sides, so a last-bit
    difference of the first GEMM can move single elements by one E4M3 step: tolerance 2e-2 relative
    Frobenius (the reference's own MoE check uses atol 1e-1, samples/MoE.py:462).
    PARITY UNPINNED: the reference has no block-scaled MoE and no test of one; this composition (re-quantising the
    SiLU-gated intermediate) is checked against the oracle's own per-expert formula only.  The grouped GEMM it is
    built from has its own gate against the dense per-expert reference (test_grouped_gemm_*, 1e-3 / 8e-3)."""
    T, H, F, E, topk = 96, 256, 128, 4, 2
    rng = np.random.default_rng(3)
    hq, hs = O.block_quantize(rng.standard_normal((T, H)).astype(np.float32), 32, O.E4M3, "floor")
    w1q, w1s = O.block_quantize((rng.standard_normal((E, 2 * F, H)) * 0.2).astype(np.float32), 32, w_fmt, "floor")
    w2q, w2s = O.block_quantize((rng.standard_normal((E, H, F)) * 0.2).astype(np.float32), 32, w_fmt, "floor")
    ids = np.stack([rng.permutation(E)[:topk] for _ in range(T)])
    wts = rng.random((T, topk)).astype(np.float32)
    want = O.moe_forward(hq, hs, w1q, w1s, w2q, w2s, wts, ids, w_fmt=w_fmt)

    def dev_elems(codes, fmt):
        if fmt == O.E2M1:
            return torch.from_numpy(O.pack_fp4(codes)).to(dev)
        return torch.from_numpy(codes).to(dev).view(torch.float8_e4m3fn)

    def dev_scale(sc):
        return torch.from_numpy(sc).to(dev).view(torch.float8_e8m0fnu)

    got = ct.cutile_moe_scaled(dev_elems(hq, O.E4M3), dev_scale(hs), dev_elems(w1q, w_fmt), dev_scale(w1s),
                               dev_elems(w2q, w_fmt), dev_scale(w2s), torch.from_numpy(wts).to(dev),
                               torch.from_numpy(ids).to(dev), tile_m, out_dtype=torch.float32,
                               w_format="e2m1" if w_fmt == O.E2M1 else None, kernel=kernel)
    assert got.shape == (T, H)
    assert O.rel_fro(got.cpu(), want) < 2e-2
