"""GPU parity on seeded random problems: shape, element formats, kernel, output dtype, accumulate and split-K are
drawn together, so that combinations no hand-written parametrisation lists are met.  Every accepted problem is
checked against the CPU oracle (relative Frobenius error <= 1e-3 for fp32 output, 8e-3 for bf16 output); a
combination a kernel does not take must be refused (ValueError / TileTypeError, as the wrapper maps the library's
error codes) before anything is launched."""
import random

import numpy as np
import pytest
import torch

from mxutil import oracle_matmul, randn_operand, raw_operand
from oracle import mx_oracle as O

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-3, torch.bfloat16: 8e-3}
PAIRS = [(O.E4M3, O.E4M3), (O.E5M2, O.E5M2), (O.E2M1, O.E2M1), (O.E4M3, O.E2M1)]
KERNELS = ["auto", "auto", "mfma128", "mfma256", "mfma256w4", "pingpong", "pingpong32", "w4p", "decode", "generic"]
ROWS = [1, 7, 16, 31, 32, 33, 64, 100, 128, 200, 256, 257, 300, 513]
COLS = [16, 48, 64, 100, 128, 130, 256, 272, 384, 520]
KBLOCKS = [1, 2, 3, 4, 5, 8, 12, 16, 17, 24, 32, 33, 48, 64]


def _draw(rnd):
    af, bf = rnd.choice(PAIRS)
    K = 32 * rnd.choice(KBLOCKS)
    if O.E2M1 in (af, bf):
        K = max(64, K // 64 * 64)      # packed rows must stay 16-byte aligned for the fast kernels to be eligible
    return dict(af=af, bf=bf, kernel=rnd.choice(KERNELS), M=rnd.choice(ROWS), N=rnd.choice(COLS), K=K,
                out=rnd.choice([torch.float32, torch.bfloat16]), acc=rnd.random() < 0.3,
                split=rnd.choice([0, 0, 0, 1, 2, 3]), raw=rnd.random() < 0.3)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_problems_match_oracle(ct, dev, seed):
    rnd = random.Random(seed)
    ran = refused = 0
    for case in range(30):
        p = _draw(rnd)
        make = raw_operand if p["raw"] else randn_operand
        a = make(p["M"], p["K"], p["af"], 1000 * seed + 2 * case, dev)
        b = make(p["N"], p["K"], p["bf"], 1000 * seed + 2 * case + 1, dev)
        what = (f"seed {seed} case {case}: {p['af']} x {p['bf']} {p['kernel']} {p['M']} x {p['N']} x {p['K']} "
                f"{p['out']} acc={p['acc']} split_k={p['split']} raw={p['raw']}")
        print(what, flush=True)
        c0 = None
        if p["acc"]:
            g = torch.Generator().manual_seed(seed * 77 + case)
            c0 = torch.randn((p["M"], p["N"]), generator=g).to(p["out"])
        try:
            got = ct.block_scaled_matmul(a.storage, a.scale_t, b.storage.T, b.scale_t.T, a_format=a.fmt_kw,
                                         b_format=b.fmt_kw, out_dtype=p["out"], kernel=p["kernel"], split_k=p["split"],
                                         C=None if c0 is None else c0.to(dev), accumulate=p["acc"])
        except (ValueError, ct.TileTypeError) as e:     # the kernel asked for does not take this problem
            assert p["kernel"] != "auto" and p["kernel"] != "generic" or p["split"] > 1, f"{what}: {e}"
            refused += 1
            continue
        ref = oracle_matmul(a, b, None if c0 is None else c0.float())
        assert got.dtype == p["out"] and tuple(got.shape) == (p["M"], p["N"])
        err = O.rel_fro(got.float().cpu(), ref)
        assert err <= TOL[p["out"]], f"{what}: relative Frobenius error {err:.3e}"
        ran += 1
    print(f"seed {seed}: {ran} problems checked, {refused} refused", flush=True)
    assert ran >= 10


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_moe_routings_match_oracle(ct, dev, seed):
    """Grouped GEMM on random routings: token count, expert count, top-k, tile_m, kernel, weight format, skew of the
    router (experts that get nothing, one expert that gets most), trimmed or worst-case-length slot arrays, routed
    weights.  Every routed row must be written (C starts as NaN) and is compared with the oracle."""
    rnd = random.Random(seed)
    for case in range(10):
        E = rnd.choice([1, 2, 5, 8, 16, 64])
        topk = rnd.choice([k for k in (1, 2, 4, 8) if k <= E])
        T = rnd.choice([1, 3, 17, 48, 130, 300])
        K = rnd.choice([128, 512, 1024])
        N = rnd.choice([64, 256, 320, 1024])
        wf = rnd.choice([O.E4M3, O.E4M3, O.E2M1])
        kernel, tile = rnd.choice([("generic", 16), ("mfma128", 128), ("mfma128", 256), ("mfma256", 256),
                                   ("mfma256w4", 256), ("pingpong", 256), ("auto", 128), ("auto", 256)])
        out = rnd.choice([torch.float32, torch.bfloat16])
        exact, routed = rnd.random() < 0.5, rnd.random() < 0.5
        skew = rnd.choice([0.0, 0.0, 2.0, 8.0])
        what = (f"seed {seed} case {case}: T={T} E={E} top{topk} K={K} N={N} w={wf} {kernel} tile_m={tile} {out} "
                f"exact={exact} routed_weights={routed} skew={skew}")
        print(what, flush=True)
        a = randn_operand(T, K, O.E4M3, 1000 * seed + 3 * case, dev, std=0.5)
        w = randn_operand(E * N, K, wf, 1000 * seed + 3 * case + 1, dev, std=0.1)
        g = torch.Generator().manual_seed(1000 * seed + 3 * case + 2)
        logits = torch.rand((T, E), generator=g)
        logits[:, 0] += skew                      # expert 0 takes (nearly) every token ...
        if E > 2:
            logits[:, E - 1] -= 10.0              # ... and the last expert none
        ids = torch.topk(logits, topk, dim=1).indices
        tw = torch.rand((T, topk), generator=g) if routed else None
        ref = O.grouped_reference(a.codes, a.scales, w.codes.reshape(E, N, K), w.scales.reshape(E, N, K // 32),
                                  ids.numpy(), w_fmt=wf)
        if routed:
            ref = ref * tw.reshape(-1, 1)
        W = w.storage.view(E, N, -1)
        Ws = w.scale_t.view(E, N, K // 32)
        sid, eid = ct.moe_align_tile_size(ids.to(dev), tile, E, exact=exact)
        C = torch.full((T, topk, N), float("nan"), device=dev, dtype=out)
        ct.invoke_fused_moe_scaled(a.storage, a.scale_t, W, Ws, C, None if tw is None else tw.to(dev), sid, eid, routed,
                                   topk, tile, kernel=kernel, b_format="e2m1" if wf == O.E2M1 else None)
        got = C.view(-1, N).float().cpu()
        assert not torch.isnan(got).any(), f"{what}: a routed row was not written"
        err = O.rel_fro(got, ref)
        assert err <= TOL[out], f"{what}: relative Frobenius error {err:.3e}"
