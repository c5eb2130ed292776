"""Helpers shared by the GPU parity tests: seeded operands in every storage layout the library takes,
with the matching one-element-per-entry codes for the CPU oracle."""
from __future__ import annotations

import numpy as np
import torch

from oracle import mx_oracle as O

TORCH_ELEM = {O.E4M3: torch.float8_e4m3fn, O.E5M2: torch.float8_e5m2}


class Operand:
    """rows x K MX operand.  ``codes`` [rows, K] uint8 one element per entry and ``scales`` [rows, K/32]
    uint8 live on the CPU for the oracle; ``storage`` (K-contiguous, FP4 packed two per byte along K) and
    ``scale_t`` (float8_e8m0fnu [rows, K/32]) are the device tensors."""

    def __init__(self, codes: np.ndarray, scales: np.ndarray, fmt: str, device):
        self.codes, self.scales, self.fmt = codes, scales, fmt
        self.rows, self.K = codes.shape
        st = O.pack_fp4(codes) if fmt == O.E2M1 else codes
        self.storage_np = np.ascontiguousarray(st)
        t = torch.from_numpy(self.storage_np).to(device)
        self.storage = t if fmt == O.E2M1 else t.view(TORCH_ELEM[fmt])
        self.scale_t = torch.from_numpy(np.ascontiguousarray(scales)).to(device).view(torch.float8_e8m0fnu)

    @property
    def fmt_kw(self):
        return "e2m1" if self.fmt == O.E2M1 else None


def randn_operand(rows, K, fmt, seed, device, dist="randn", scale_mode="floor", std=1.0) -> Operand:
    g = torch.Generator().manual_seed(seed)
    if dist == "randn":
        x = torch.randn((rows, K), generator=g) * std
    elif dist == "rand":
        x = torch.rand((rows, K), generator=g)
    elif dist == "uniform6":
        x = torch.rand((rows, K), generator=g) * 12 - 6
    else:
        raise ValueError(dist)
    codes, sb = O.block_quantize(x.numpy(), 32, fmt, scale_mode)
    return Operand(codes, sb, fmt, device)


def raw_operand(rows, K, fmt, seed, device, scale_lo=115, scale_hi=130, allow_nan=False) -> Operand:
    """Raw random bytes as elements (test/test_mma_scaled.py:103-125) with scales spanning 2^-12..2^2."""
    rng = np.random.default_rng(seed)
    if fmt == O.E2M1:
        codes = rng.integers(0, 16, (rows, K), dtype=np.uint8)
    else:
        codes = rng.integers(0, 256, (rows, K), dtype=np.uint8)
        if not allow_nan:
            if fmt == O.E4M3:
                codes[(codes & 0x7F) == 0x7F] = 0x3C
            else:
                codes[(codes & 0x7C) == 0x7C] = 0x3C
    sb = rng.integers(scale_lo, scale_hi, (rows, K // 32), dtype=np.uint8)
    return Operand(codes, sb, fmt, device)


def oracle_matmul(a: Operand, b: Operand, acc=None) -> torch.Tensor:
    """fp32 CPU result of A[M,K] x B[N,K]^T through the oracle's dequantize + matmul."""
    return O.reference_matmul(a.codes, a.scales, np.ascontiguousarray(b.codes.T),
                              np.ascontiguousarray(b.scales.T), a.fmt, b.fmt, 32, acc)
