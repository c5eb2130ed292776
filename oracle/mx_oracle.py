"""CPU oracle for the block-scaled (MX) matmul path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU with numpy + torch-CPU, the algorithms the reference
(NVIDIA cuTile Python) uses around ``ct.mma_scaled``.  It is the checker the HIP kernels are
compared with; it is never the product path.  Only the tests, the smoke check and the
``cpu_baseline`` leg of the benchmark may import it.

Every function cites the reference file:line it follows (paths relative to the reference root).

Pinning status (what each function is checked against in ``tests/test_oracle*.py``):
  * decode tables e2m1/e4m3/e8m0   -> value tables held by test/test_float_encoding.py:49-186
                                      (committed as tests/golden/float_tables.json) and torch views
  * e4m3 encode                    -> torch CPU ``.to(float8_e4m3fn)`` (library routine), all 256
                                      code round trips, independent integer formulation
  * e2m1 encode                    -> round trip of all 16 codes, brute force nearest-value search
                                      with ties-to-even, saturation to +-6 (_bytecode/float.py:192-197)
  * e8m0 encode of powers of two   -> closed form byte = exponent + 127, torch view
  * block_quantize (ceil rule)     -> literal torch restatement of test/kernels/kernel_utils.py:38-80
                                      vs the exact-integer formulation; invariants (power-of-two
                                      scale, |x/scale| <= 448, all-zero block -> byte 88)
  * block_quantize (floor rule)    -> OCP MX v1.0 closed form via frexp; invariants
  * swizzle_32_4_4 / inverse       -> closed-form index map, bijection, round trip
  * swizzle_2d_from_bid            -> bijection by brute force
  * reference_matmul               -> known answers 256.0 and 512.0 of src/cuda/tile/_stub.py:2248-2259,
                                      2309-2328; all-ones-scale reduction to a plain fp32 matmul;
                                      float64 brute force on tiny shapes
  * moe_align_tile_size            -> brute-force invariants on tiny routings (one expert per block,
                                      stable order, sentinel padding, block count formula)
  * grouped_reference              -> per-expert dense loop (structure of samples/MoE.py:292-334);
                                      the reference holds no test of an MX MoE GEMM:
                                      PARITY UNPINNED beyond the dense per-expert formula.
  * silu_mul                       -> torch.nn.functional.silu(a) * b (library routine) to a few 1e-7
                                      relative; closed forms silu(0) = 0, silu(x) -> x for large x,
                                      silu(-x) -> 0; the reference's own kernel
                                      (test/kernels/fused_moe.py:85-108) uses approximate division and
                                      flush-to-zero, so only the formula, not its bits, is the contract
  * moe_forward                    -> structure of torch_moe (samples/MoE.py:292-334) with the dequantised
                                      operands; the intermediate re-quantisation is this build's own step:
                                      PARITY UNPINNED beyond the dense formula (no reference MX MoE exists)
  * bit-level accumulation order of the reference GPU result: PARITY UNPINNED (the arithmetic of
    mma_scaled lives in the closed tileiras compiler and Blackwell hardware).
"""
from __future__ import annotations

import numpy as np
import torch

# ----------------------------------------------------------------------------------------------
# Formats (src/cuda/tile/_bytecode/float.py:30-43)
# ----------------------------------------------------------------------------------------------
E4M3, E5M2, E2M1 = "e4m3", "e5m2", "e2m1"
ELEM_MAX = {E4M3: 448.0, E5M2: 57344.0, E2M1: 6.0}
# exponent of the largest power of two representable in the element format (OCP MX "emax_elem")
ELEM_EMAX = {E4M3: 8, E5M2: 15, E2M1: 2}

# test/test_mma_scaled.py:149-152 and test/test_float_encoding.py:49-52
E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
                        -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], dtype=np.float32)


def decode_e4m3(code: np.ndarray) -> np.ndarray:
    """uint8 -> float32.  E4M3FN: bias 7, subnormal step 2^-9, 0x7F/0xFF NaN, no infinity
    (src/cuda/tile/_bytecode/float.py:35, 63-93)."""
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    sign = np.where(c & 0x80, -1.0, 1.0)
    e = (c >> 3) & 0xF
    m = c & 7
    mag = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2((e - 7).astype(np.float64)))
    out = (sign * mag).astype(np.float32)
    out = np.where((c & 0x7F) == 0x7F, np.float32(np.nan), out)
    return out.astype(np.float32)


def decode_e5m2(code: np.ndarray) -> np.ndarray:
    """uint8 -> float32.  E5M2 is IEEE-like: bias 15, inf and NaN (float.py:36)."""
    c = np.asarray(code, dtype=np.uint8)
    return (c.astype(np.uint16) << 8).view(np.float16).astype(np.float32)


def decode_e2m1(code: np.ndarray) -> np.ndarray:
    """4-bit code (0..15) -> float32 (float.py:40; table test/test_float_encoding.py:49-52)."""
    return E2M1_VALUES[np.asarray(code, dtype=np.uint8) & 0xF]


def decode_e8m0(code: np.ndarray) -> np.ndarray:
    """uint8 -> float32 value 2^(b-127); 0xFF is NaN; there is no zero and no sign
    (float.py:37-39, 96-130).  2^-127 is an fp32 subnormal and is represented exactly."""
    c = np.asarray(code, dtype=np.uint8).astype(np.int32)
    out = np.ldexp(np.float64(1.0), c - 127).astype(np.float32)
    return np.where(c == 0xFF, np.float32(np.nan), out).astype(np.float32)


def decode_elem(code: np.ndarray, fmt: str) -> np.ndarray:
    return {E4M3: decode_e4m3, E5M2: decode_e5m2, E2M1: decode_e2m1}[fmt](code)


def encode_e4m3(x: np.ndarray, saturate: bool) -> np.ndarray:
    """float32 -> E4M3FN byte.  Round to nearest even; without ``saturate`` everything that rounds
    above 448 becomes NaN (0x7F), which is what torch's cast does and what the reference's
    quantizer relies on (test/kernels/kernel_utils.py:77); with ``saturate`` the value is clamped
    to +-448 first (OCP MX conversion).  Uses torch's CPU cast, a library routine."""
    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32))
    if saturate:
        t = torch.clamp(t, -448.0, 448.0)
    return t.to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def encode_e5m2(x: np.ndarray, saturate: bool) -> np.ndarray:
    t = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32))
    if saturate:
        t = torch.clamp(t, -57344.0, 57344.0)
    return t.to(torch.float8_e5m2).view(torch.uint8).numpy()


def encode_e2m1(x: np.ndarray) -> np.ndarray:
    """float32 -> 4-bit E2M1 code.  Round to nearest, ties to the even mantissa, overflow clamps to
    +-6 (float.py:184-197: finite-only format clamps).  NaN has no encoding; it maps to +6 with the
    sign bit taken from the input so that the function is total (the reference raises instead)."""
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    # midpoints between consecutive magnitudes 0,.5,1,1.5,2,3,4,6; a tie goes to the neighbour whose
    # code is even (mantissa bit 0): 0.25->0, 0.75->1.0, 1.25->1.0, 1.75->2.0, 2.5->2.0, 3.5->4.0, 5->4.0
    mids = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    tie_up = np.array([False, True, False, True, False, True, False])
    code = np.zeros(a.shape, dtype=np.uint8)
    for i in range(7):
        code += ((a > mids[i]) | ((a == mids[i]) & tie_up[i])).astype(np.uint8)
    code = np.where(np.isnan(a), np.uint8(7), code)
    sign = (np.signbit(x)).astype(np.uint8) << 3
    return (code | sign).astype(np.uint8)


def encode_e8m0_pow2(scale: np.ndarray) -> np.ndarray:
    """float32 power of two -> E8M0 byte = exponent + 127 (float.py:96-130; the general encoder
    rounds ties up, but the quantizers only ever hand it exact powers of two)."""
    m, e = np.frexp(np.asarray(scale, dtype=np.float32))
    assert np.all(m == 0.5), "encode_e8m0_pow2 expects exact powers of two"
    return np.clip(e.astype(np.int32) - 1 + 127, 0, 254).astype(np.uint8)


# ----------------------------------------------------------------------------------------------
# FP4 transport (src/cuda/tile/_stub.py:2625-2679; test/test_mma_scaled.py:155-160)
# ----------------------------------------------------------------------------------------------
def pack_fp4(codes: np.ndarray) -> np.ndarray:
    """[..., 2n] 4-bit codes -> [..., n] bytes, low nibble = element 2i, high nibble = 2i+1."""
    c = np.asarray(codes, dtype=np.uint8)
    return (c[..., 0::2] & 0xF) | ((c[..., 1::2] & 0xF) << 4)


def unpack_fp4(packed: np.ndarray) -> np.ndarray:
    p = np.asarray(packed, dtype=np.uint8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = p & 0xF
    out[..., 1::2] = p >> 4
    return out


# ----------------------------------------------------------------------------------------------
# Quantizers
# ----------------------------------------------------------------------------------------------
def _blocks(x: np.ndarray, block_size: int) -> np.ndarray:
    x = np.asarray(x, dtype=np.float32)
    if x.shape[-1] < block_size:
        # test/kernels/kernel_utils.py:58-60
        raise ValueError(f'The requested block size {block_size} is larger than the inner most '
                         f'dimension of the input tensor {x.shape[-1]}')
    pad = (-x.shape[-1]) % block_size
    if pad:
        # kernel_utils.py:62-67 zero-pads the last dimension
        x = np.concatenate([x, np.zeros(x.shape[:-1] + (pad,), np.float32)], axis=-1)
    return x.reshape(*x.shape[:-1], x.shape[-1] // block_size, block_size)


def block_quantize_ceil_literal(x: torch.Tensor, block_size: int = 32,
                                dtype: torch.dtype = torch.float8_e4m3fn):
    """Literal torch restatement of ``block_quantize`` (test/kernels/kernel_utils.py:38-80):
    scale = 2^ceil(log2(clamp(amax/448, 1e-12))), x_q = (x/scale).to(dtype), scale.to(e8m0).
    Uses torch's fp32 ``log2``; see :func:`block_quantize` for the exact-integer variant."""
    dtype_max = torch.finfo(torch.float8_e4m3fn).max
    if x.shape[-1] < block_size:
        raise ValueError(f'The requested block size {block_size} is larger than the inner most '
                         f'dimension of the input tensor {x.shape[-1]}')
    if x.shape[-1] % block_size != 0:
        pad_len = (block_size - (x.shape[-1] % block_size)) % block_size
        x = torch.nn.functional.pad(x, (0, pad_len), value=0)
    xb = x.reshape(*x.shape[:-1], x.shape[-1] // block_size, block_size)
    scale = torch.max(xb.abs(), dim=-1, keepdim=True)[0]
    scale = torch.clamp(scale / dtype_max, min=1e-12)
    scale = torch.pow(2.0, torch.ceil(torch.log2(scale)))
    x_q = (xb / scale).to(dtype).reshape(x.shape)
    return x_q, scale.to(torch.float8_e8m0fnu).squeeze(-1)


def block_quantize(x: np.ndarray, block_size: int = 32, fmt: str = E4M3, scale_mode: str = "ceil"):
    """MX quantization of the last axis in blocks of ``block_size``.

    Returns ``(codes uint8 [..., Kpad], scale_bytes uint8 [..., Kpad/block])``; E2M1 codes are
    returned one per byte (use :func:`pack_fp4`).

    scale_mode "ceil"  -- the reference's rule (test/kernels/kernel_utils.py:69-78):
        v = fl32(amax/448) clamped below at fl32(1e-12); scale = 2^ceil(log2 v) with the ceiling
        taken exactly on the fp32 value v (integer exponent arithmetic; torch's fp32 log2 returns k
        instead of k+1 for v = 2^k(1+eps), eps <~ 3*2^-23, which is the only place the literal
        restatement differs); elements = rne(x/scale) cast without saturation (above 464 -> NaN).
        448 is used for every element format, as the reference hard-codes it (kernel_utils.py:56).
    scale_mode "floor" -- OCP Microscaling v1.0 float->MX rule (the benchmark configurations):
        scale = 2^(floor(log2 amax) - emax_elem), clamped to the E8M0 range, amax == 0 -> byte 0;
        elements = rne(clamp(x/scale, +-max_normal)).
    """
    xb = _blocks(x, block_size)
    amax = np.max(np.abs(xb), axis=-1, keepdims=True).astype(np.float32)
    if scale_mode == "ceil":
        with np.errstate(invalid="ignore"):
            v = np.maximum((amax / np.float32(448.0)).astype(np.float32), np.float32(1e-12))
        v = np.where(np.isfinite(v), v, np.float32(1.0))   # non-finite blocks are overwritten below
        m, e = np.frexp(v)                       # v = m * 2^e, m in [0.5, 1)
        se = np.where(m == 0.5, e - 1, e).astype(np.int32)   # exact ceil(log2 v)
        saturate = False
    elif scale_mode == "floor":
        m, e = np.frexp(amax)
        se = (e.astype(np.int32) - 1) - ELEM_EMAX[fmt]
        se = np.where(amax == 0, -127, se)
        saturate = True
    else:
        raise ValueError(f"unknown scale_mode {scale_mode!r}")
    se = np.clip(se, -127, 127)
    # x / 2^se is exact in fp32 unless it leaves the normal range; do it in float64 and round once
    q = (xb.astype(np.float64) * np.ldexp(1.0, -se)).astype(np.float32)
    if fmt == E4M3:
        codes = encode_e4m3(q, saturate)
    elif fmt == E5M2:
        codes = encode_e5m2(q, saturate)
    elif fmt == E2M1:
        codes = encode_e2m1(q)
    else:
        raise ValueError(fmt)
    scale_bytes = (se[..., 0] + 127).astype(np.uint8)
    if scale_mode == "ceil" and not np.all(np.isfinite(amax)):
        # Non-finite blocks under the reference's rule (kernel_utils.py:69-78 evaluated by torch): clamp(min=)
        # keeps NaN and inf / 448 is inf, so the scale is NaN or inf and its float8_e8m0fnu byte is 0xFF;
        # x / scale is NaN for every element of a NaN block (an element that is NaN itself keeps its sign),
        # and in an inf block NaN with the sign bit set where |x| is inf (inf / inf) and a signed zero
        # elsewhere.  E2M1 has no NaN: non-finite elements saturate to +-6.
        nf = ~np.isfinite(amax)
        blk_nan = np.isnan(amax)
        a_nan, a_inf = np.isnan(xb), np.isinf(xb)
        sgn = np.signbit(xb).astype(np.uint8)
        if fmt == E2M1:
            special = (sgn << 3) | np.where(blk_nan | a_inf, np.uint8(7), np.uint8(0))
        else:
            special = np.where(a_nan, (sgn << 7) | np.uint8(0x7F),
                               np.where(blk_nan, np.uint8(0x7F), np.where(a_inf, np.uint8(0xFF), sgn << 7)))
        codes = np.where(nf, special.astype(np.uint8), codes.reshape(xb.shape))
        scale_bytes = np.where(nf[..., 0], np.uint8(0xFF), scale_bytes)
    codes = codes.reshape(*xb.shape[:-2], xb.shape[-2] * block_size)
    return codes, scale_bytes.astype(np.uint8)


# ----------------------------------------------------------------------------------------------
# Dequantize + reference math (samples/BlockScaledMatMul.py:358-364, test/test_mma_scaled.py:94-96)
# ----------------------------------------------------------------------------------------------
def dequantize(codes: np.ndarray, scale_bytes: np.ndarray, fmt: str, block_size: int = 32,
               k_axis: int = -1) -> torch.Tensor:
    """codes [..., K] (one element per entry) and E8M0 bytes [..., K/block] along ``k_axis`` ->
    fp32 torch tensor elem * repeat_interleave(scale, block)."""
    el = torch.from_numpy(decode_elem(codes, fmt))
    sc = torch.from_numpy(decode_e8m0(scale_bytes))
    return el * torch.repeat_interleave(sc, block_size, dim=k_axis)


def reference_matmul(a_codes, a_scale, b_codes, b_scale, a_fmt=E4M3, b_fmt=E4M3, block_size=32,
                     acc: torch.Tensor | None = None) -> torch.Tensor:
    """ref = (A.f32 * repeat(As)) @ (B.f32 * repeat(Bs)) [+ acc], fp32 torch matmul.
    a_codes [..., M, K], a_scale [..., M, K/B]; b_codes [..., K, N], b_scale [..., K/B, N]
    (one element per entry: unpack FP4 first).  src/cuda/tile/_stub.py:2204-2205."""
    a = dequantize(a_codes, a_scale, a_fmt, block_size, k_axis=-1)
    b = dequantize(b_codes, b_scale, b_fmt, block_size, k_axis=-2)
    out = a @ b
    return out if acc is None else out + acc


# ----------------------------------------------------------------------------------------------
# Scale layouts and tile order (test/kernels/kernel_utils.py:19-29, 83-112)
# ----------------------------------------------------------------------------------------------
def swizzle_32_4_4(scale: np.ndarray) -> np.ndarray:
    """(M, K_s) -> (M/128, K_s/4, 32, 16): reshape (m0, 4, 32, k0, 4), permute (0, 3, 2, 1, 4)."""
    m1, m2, k1 = 32, 4, 4
    M, K_s = scale.shape
    m0, k0 = M // (m1 * m2), K_s // k1
    s = scale.reshape(m0, m2, m1, k0, k1).transpose(0, 3, 2, 1, 4)
    return np.ascontiguousarray(s).reshape(m0, k0, 32, 16)


def unswizzle_32_4_4(sw: np.ndarray) -> np.ndarray:
    m1, m2, k1 = 32, 4, 4
    m0, k0 = sw.shape[0], sw.shape[1]
    s = sw.reshape(m0, k0, m1, m2, k1).transpose(0, 3, 2, 1, 4)
    return np.ascontiguousarray(s).reshape(m0 * m2 * m1, k0 * k1)


def swizzle_32_4_4_offset(r: int, c: int, K_s: int) -> int:
    """Flat offset of logical element (r, c) inside the swizzled tensor (closed form)."""
    m0, rem = divmod(r, 128)
    m2, m1 = divmod(rem, 32)
    k0, k1 = divmod(c, 4)
    return ((m0 * (K_s // 4) + k0) * 32 + m1) * 16 + m2 * 4 + k1


def swizzle_2d_from_bid(M, N, tm, tn, group_size_m, bid):
    """1-D block id -> (bid_m, bid_n), groups of ``group_size_m`` row tiles sweeping N
    (test/kernels/kernel_utils.py:19-29)."""
    num_bid_m = -(-M // tm)
    num_bid_n = -(-N // tn)
    num_bid_in_group = group_size_m * num_bid_n
    group_id = bid // num_bid_in_group
    first_bid_m = group_id * group_size_m
    gsm = min(num_bid_m - first_bid_m, group_size_m)
    return first_bid_m + (bid % gsm), (bid % num_bid_in_group) // gsm


# ----------------------------------------------------------------------------------------------
# MoE grouping (test/kernels/fused_moe.py:113-173, 14-82; samples/MoE.py:292-334)
# ----------------------------------------------------------------------------------------------
def moe_align_tile_size(topk_ids: np.ndarray, tile_m: int, num_experts: int):
    """Stable sort of the flattened (token, k) slots by expert, each expert padded to a multiple of
    ``tile_m`` with the sentinel ``num_tokens*topk``.  Returns (sorted_token_ids int32
    [blocks*tile_m], sorted_expert_ids int32 [blocks])."""
    flat = np.asarray(topk_ids).reshape(-1).astype(np.int64)
    total = flat.size
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=num_experts)
    blocks = (counts + tile_m - 1) // tile_m
    ids = np.full((int(blocks.sum()) * tile_m,), total, dtype=np.int32)
    eids = np.zeros((int(blocks.sum()),), dtype=np.int32)
    cb = ct = 0
    for e in range(num_experts):
        eids[cb:cb + blocks[e]] = e
        ids[cb * tile_m: cb * tile_m + counts[e]] = order[ct:ct + counts[e]]
        ct += counts[e]
        cb += blocks[e]
    return ids, eids


def grouped_reference(a_codes, a_scale, w_codes, w_scale, topk_ids, a_fmt=E4M3, w_fmt=E4M3,
                      block_size=32) -> torch.Tensor:
    """Per-expert dense oracle of the MoE up-projection:
    C[t*topk + j, :] = dequant(A[t]) @ dequant(W[topk_ids[t, j]]).T
    a_codes (T, K), a_scale (T, K/B); w_codes (E, N, K), w_scale (E, N, K/B); fp32 (T*topk, N)."""
    topk_ids = np.asarray(topk_ids)
    T, topk = topk_ids.shape
    a = dequantize(a_codes, a_scale, a_fmt, block_size)
    out = torch.zeros((T * topk, w_codes.shape[1]), dtype=torch.float32)
    flat = topk_ids.reshape(-1)
    for e in np.unique(flat):
        rows = np.nonzero(flat == e)[0]
        w = dequantize(w_codes[e], w_scale[e], w_fmt, block_size)
        out[torch.from_numpy(rows)] = a[torch.from_numpy(rows // topk)] @ w.T
    return out


def silu_mul(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """silu(a) * b = a / (1 + exp(-a)) * b (silu_and_mul_kernel, test/kernels/fused_moe.py:85-108) as the
    fixed sequence of correctly rounded fp32 operations the device executes: exp(-a) = 2^z with
    z = -a * log2(e) clamped to +-125, z = n + f, n = rint(z), 2^f by the degree-7 Taylor polynomial in
    f ln 2 evaluated by Horner's rule with separate multiplies and adds, scaled by 2^n exactly."""
    f32 = np.float32
    a = np.asarray(a, dtype=f32)
    b = np.asarray(b, dtype=f32)
    with np.errstate(invalid="ignore", over="ignore", under="ignore"):
        z = (-a) * f32(1.44269504)
        z = np.fmin(np.fmax(z, f32(-125.0)), f32(125.0))
        n = np.rint(z)
        f = z - n
        p = np.full_like(f, f32(1.52527338e-5))
        for c in (1.54035304e-4, 1.33335581e-3, 9.61812911e-3, 5.55041087e-2, 2.40226507e-1, 6.93147181e-1, 1.0):
            p = p * f + f32(c)          # numpy rounds the product to fp32 before the add: no fused operation
        two_n = ((np.nan_to_num(n).astype(np.int32) + 127).astype(np.uint32) << np.uint32(23)).view(f32)
        e = p * two_n
        s = f32(1.0) / (f32(1.0) + e)
        t = np.where(a < f32(-87.5), f32(0.0), a * s)   # exp(-a) is past the clamp: the true value is below 2^-120
        return t * b


def silu_mul_quantize(gate_up: np.ndarray, fmt: str = E4M3, scale_mode: str = "floor"):
    """silu(gate) * up of a (rows, 2F) array (gate first), MX-quantised along F: the fused producer between
    the two grouped GEMMs of the MoE pipeline (samples/MoE.py:262-266 followed by block_quantize)."""
    gate_up = np.asarray(gate_up, dtype=np.float32)
    F = gate_up.shape[-1] // 2
    return block_quantize(silu_mul(gate_up[..., :F], gate_up[..., F:]), 32, fmt, scale_mode)


def moe_forward(h_codes, h_scale, w1_codes, w1_scale, w2_codes, w2_scale, topk_weights, topk_ids,
                h_fmt=E4M3, w_fmt=E4M3, scale_mode="floor") -> torch.Tensor:
    """Block-scaled MoE forward with the structure of cutile_moe / torch_moe (samples/MoE.py:197-334):
    gate+up projection per routed (token, k) pair, rounded to bf16 as the intermediate buffer is,
    silu(gate) * up re-quantised to E4M3, down projection, routed-weight multiply, sum over k.
    Returns fp32 (tokens, H)."""
    topk_ids = np.asarray(topk_ids)
    T, topk = topk_ids.shape
    c1 = grouped_reference(h_codes, h_scale, w1_codes, w1_scale, topk_ids, h_fmt, w_fmt)
    c1 = c1.to(torch.bfloat16).to(torch.float32).numpy()
    a2_codes, a2_scale = silu_mul_quantize(c1, E4M3, scale_mode)
    a2 = dequantize(a2_codes, a2_scale, E4M3)
    out = torch.zeros((T * topk, w2_codes.shape[1]), dtype=torch.float32)
    flat = topk_ids.reshape(-1)
    for e in np.unique(flat):
        rows = torch.from_numpy(np.nonzero(flat == e)[0])
        w = dequantize(w2_codes[e], w2_scale[e], w_fmt)
        out[rows] = a2[rows] @ w.T
    out = out * torch.as_tensor(np.asarray(topk_weights, dtype=np.float32)).reshape(-1, 1)
    return out.reshape(T, topk, -1).sum(dim=1)


def rel_fro(x: torch.Tensor, ref: torch.Tensor) -> float:
    """Relative Frobenius error ||x - ref|| / ||ref|| in float64."""
    x = x.double()
    ref = ref.double()
    return float(torch.linalg.norm(x - ref) / torch.linalg.norm(ref))
