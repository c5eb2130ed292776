"""ctypes binding of libmxgemm.so (the C ABI declared in include/mxgemm.h)."""
from __future__ import annotations

import ctypes
import os
import pathlib
import threading

import torch

_HERE = pathlib.Path(__file__).resolve().parent
# the library built in-tree; MXGEMM_LIB names another build of it (for example one with other compiler flags)
LIB_PATH = pathlib.Path(os.environ["MXGEMM_LIB"]) if os.environ.get("MXGEMM_LIB") else _HERE / "libmxgemm.so"

# ---- constants mirrored from include/mxgemm.h -------------------------------------------------
MX_OK = 0
MX_ERR_INVALID, MX_ERR_SHAPE, MX_ERR_DTYPE, MX_ERR_LAYOUT = -1, -2, -3, -4
MX_ERR_WORKSPACE, MX_ERR_DEVICE, MX_ERR_LAUNCH = -5, -6, -7

MX_E4M3, MX_E5M2, MX_E2M1, MX_E8M0 = 0, 1, 4, 8
MX_F32, MX_BF16, MX_F16, MX_I32 = 16, 17, 18, 24

MX_SCALE_2D, MX_SCALE_SWIZZLE_32_4_4, MX_SCALE_NATIVE, MX_SCALE_NATIVE32 = 0, 1, 2, 3
MX_OPERAND_A, MX_OPERAND_B = 0, 1
# kernels that read MX_SCALE_NATIVE32 (the 32x32x64 instruction); every other MFMA kernel reads MX_SCALE_NATIVE
NATIVE32_KERNELS = ("pingpong32", "w4p")

MX_KERNEL_AUTO, MX_KERNEL_GENERIC = 0, 1
MX_KERNEL_MFMA_128x128, MX_KERNEL_MFMA_256x256, MX_KERNEL_MFMA_256x256_W4, MX_KERNEL_DECODE = 2, 3, 4, 5
MX_KERNEL_MFMA_PINGPONG = 6
MX_KERNEL_MFMA_PINGPONG32 = 7
MX_KERNEL_MFMA_W4_PERSISTENT = 8

KERNELS = {
    "auto": MX_KERNEL_AUTO, "generic": MX_KERNEL_GENERIC, "mfma128": MX_KERNEL_MFMA_128x128,
    "mfma256": MX_KERNEL_MFMA_256x256, "mfma256w4": MX_KERNEL_MFMA_256x256_W4, "decode": MX_KERNEL_DECODE,
    "pingpong": MX_KERNEL_MFMA_PINGPONG, "pingpong32": MX_KERNEL_MFMA_PINGPONG32,
    "w4p": MX_KERNEL_MFMA_W4_PERSISTENT,
}


class MxTensor(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.c_int64 * 4), ("stride", ctypes.c_int64 * 4),
                ("packed_dim", ctypes.c_int32), ("reserved", ctypes.c_int32)]


class MxGemmOpts(ctypes.Structure):
    _fields_ = [("struct_size", ctypes.c_int32), ("accumulate", ctypes.c_int32),
                ("a_scale_layout", ctypes.c_int32), ("b_scale_layout", ctypes.c_int32),
                ("kernel", ctypes.c_int32), ("block_size", ctypes.c_int32),
                ("split_k", ctypes.c_int32), ("reserved", ctypes.c_int32)]


# every symbol include/mxgemm.h declares: name -> (restype, argtypes)
_P = ctypes.POINTER
SYMBOLS = {
    "mx_version": (ctypes.c_int, []),
    "mx_last_error": (ctypes.c_char_p, []),
    "mx_device_check": (ctypes.c_int, []),
    "mx_gemm_workspace_bytes": (ctypes.c_int64, [ctypes.c_int64] * 3 + [_P(MxGemmOpts)]),
    "mx_gemm": (ctypes.c_int, [_P(MxTensor)] * 5 + [_P(MxGemmOpts), ctypes.c_void_p, ctypes.c_int64,
                                                   ctypes.c_void_p]),
    "mx_static_scratch_bytes": (ctypes.c_int64, []),
    "mx_gemm_static": (ctypes.c_int, [_P(MxTensor)] * 5 + [_P(MxGemmOpts), ctypes.c_void_p]),
    "mx_gemm_grouped_workspace_bytes": (ctypes.c_int64, [ctypes.c_int64] * 4 + [_P(MxGemmOpts)]),
    "mx_gemm_grouped": (ctypes.c_int, [_P(MxTensor)] * 5 + [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
        ctypes.c_int64, _P(MxGemmOpts), ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]),
    "mx_moe_align_max_slots": (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int32, ctypes.c_int32]),
    "mx_moe_align_workspace_bytes": (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int32]),
    "mx_moe_align": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32,
                                    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                    ctypes.c_int64, ctypes.c_void_p]),
    "mx_bench_gemm": (ctypes.c_int, [ctypes.c_int32] + [_P(MxTensor)] * 5 + [
        _P(MxGemmOpts), ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32,
        _P(ctypes.c_float), ctypes.c_void_p]),
    "mx_gemm_list_workspace_bytes": (ctypes.c_int64, [ctypes.c_int32, _P(MxTensor), _P(MxTensor), _P(MxGemmOpts)]),
    "mx_gemm_list": (ctypes.c_int, [ctypes.c_int32] + [_P(MxTensor)] * 5 + [_P(MxGemmOpts), ctypes.c_void_p,
                                    ctypes.c_int64, ctypes.c_void_p]),
    "mx_quantize": (ctypes.c_int, [_P(MxTensor)] * 3 + [ctypes.c_int32, ctypes.c_void_p]),
    "mx_silu_mul_quantize": (ctypes.c_int, [_P(MxTensor)] * 3 + [ctypes.c_int32, ctypes.c_void_p]),
    "mx_probe_mfma_rate": (ctypes.c_int, [ctypes.c_int32, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32,
                                          ctypes.c_void_p, ctypes.c_void_p]),
    "mx_packed_scale_bytes": (ctypes.c_int64, [ctypes.c_int64, ctypes.c_int64]),
    "mx_pack_scales": (ctypes.c_int, [_P(MxTensor), ctypes.c_int32, ctypes.c_int64, ctypes.c_int64,
                                      ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p]),
}

_lib = None
_lock = threading.Lock()


class MXLibraryError(RuntimeError):
    """libmxgemm.so is missing or a call into it failed for a non-argument reason."""


def lib() -> ctypes.CDLL:
    """Loads libmxgemm.so once.  There is no fallback: without the HIP library nothing runs."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not LIB_PATH.exists():
                    raise MXLibraryError(
                        f"{LIB_PATH} not found: build it with `python cutile-python_amd/build.py` "
                        "(hipcc, gfx950).  There is no CPU or PyTorch fallback for this path.")
                h = ctypes.CDLL(str(LIB_PATH))
                for name, (res, args) in SYMBOLS.items():
                    fn = getattr(h, name)
                    fn.restype = res
                    fn.argtypes = args
                _lib = h
    return _lib


def last_error() -> str:
    return lib().mx_last_error().decode("utf-8", "replace")


_TORCH_TO_MX = {
    torch.float8_e4m3fn: MX_E4M3, torch.float8_e5m2: MX_E5M2, torch.float8_e8m0fnu: MX_E8M0,
    torch.float32: MX_F32, torch.bfloat16: MX_BF16, torch.float16: MX_F16, torch.int32: MX_I32,
}
if hasattr(torch, "float4_e2m1fn_x2"):
    _TORCH_TO_MX[torch.float4_e2m1fn_x2] = MX_E2M1


def desc(t: torch.Tensor, mx_dtype: int, packed_dim: int = -1) -> MxTensor:
    """Descriptor of a torch tensor.  ``packed_dim`` >= 0 marks an FP4 tensor whose storage holds two
    logical elements per byte along that dimension (the logical extent is doubled)."""
    nd = t.dim()
    shape = tuple(t.shape)
    if packed_dim >= 0:
        shape = tuple(n * 2 if i == packed_dim else n for i, n in enumerate(shape))
    d = MxTensor()
    d.ptr = t.data_ptr()
    d.dtype = mx_dtype
    d.ndim = nd
    d.shape[0:nd] = shape
    # strides are in units of the storage type; all sub-byte / byte formats are 1 byte wide
    d.stride[0:nd] = t.stride()
    d.packed_dim = packed_dim
    return d


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream
