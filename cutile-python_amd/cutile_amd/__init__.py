"""cutile_amd -- MI355X-native block-scaled (MX) matmul behind cuTile Python's ``mma_scaled`` surface.

    import cutile_amd as ct
    A_q, A_s = ct.block_quantize(A, 32)
    B_q, B_s = ct.block_quantize(Bt, 32)          # Bt is (N, K)
    C = ct.block_scaled_matmul(A_q, A_s, B_q.T, B_s.T)

All compute runs in libmxgemm.so (hand-written HIP for gfx950) through the C ABI of
include/mxgemm.h; see ops.py for the reference counterparts of each function.
"""
from ._lib import LIB_PATH, MXLibraryError, lib
from .errors import TileTypeError, TileValueError
from .ops import (PackedScales, bench_block_scaled_matmul, block_quantize, clear_scale_cache, block_scaled_matmul, cutile_block_scaled_matmul,
                  cutile_moe_scaled, grouped_block_scaled_matmul, invoke_fused_moe_scaled, mma_scaled, moe_align_tile_size, pack_scales,
                  silu_and_mul_quantize, swizzle_32_4_4, unswizzle_32_4_4)

__all__ = [
    "LIB_PATH", "MXLibraryError", "lib", "TileTypeError", "TileValueError", "PackedScales",
    "block_quantize", "block_scaled_matmul", "cutile_block_scaled_matmul", "invoke_fused_moe_scaled",
    "mma_scaled", "moe_align_tile_size", "pack_scales", "swizzle_32_4_4", "unswizzle_32_4_4",
    "silu_and_mul_quantize", "cutile_moe_scaled", "grouped_block_scaled_matmul", "bench_block_scaled_matmul",
    "clear_scale_cache",
]
