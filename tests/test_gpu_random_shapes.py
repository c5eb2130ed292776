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
