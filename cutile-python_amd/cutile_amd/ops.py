"""Host-side mirror of the reference's block-scaled matmul interface, on PyTorch-ROCm tensors.

Every function validates like its reference counterpart (same argument order, same error
classes and messages) and then calls libmxgemm.so through ctypes on the current HIP stream.
PyTorch is used for device memory and streams only; there is no PyTorch or CPU compute
fallback: if the library is missing, calls raise.

Reference counterparts
  block_scaled_matmul / cutile_block_scaled_matmul -> samples/BlockScaledMatMul.py:229-297
  mma_scaled                                        -> src/cuda/tile/_stub.py:2198-2329,
                                                       src/cuda/tile/_ir/ops.py:2089-2149,
                                                       src/cuda/tile/_datatype.py:482-527
  block_quantize                                    -> test/kernels/kernel_utils.py:38-80
  swizzle_32_4_4 / unswizzle_32_4_4                 -> test/kernels/kernel_utils.py:83-112
  moe_align_tile_size                               -> test/kernels/fused_moe.py:113-173
  invoke_fused_moe_scaled                           -> samples/MoE.py:338-375
"""
from __future__ import annotations

import collections
import ctypes
import threading
import weakref
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib as L
from .errors import TileTypeError, TileValueError

_FMT_CODE = {"e4m3": L.MX_E4M3, "e5m2": L.MX_E5M2, "e2m1": L.MX_E2M1}
_FMT_NAME = {"e4m3": "float8_e4m3fn", "e5m2": "float8_e5m2", "e2m1": "float4_e2m1fn"}
_F4X2 = getattr(torch, "float4_e2m1fn_x2", None)
_DTYPE_FMT = {torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}
if _F4X2 is not None:
    _DTYPE_FMT[_F4X2] = "e2m1"
_SCALE_NAME = {L.MX_E8M0: "float8_e8m0fnu", L.MX_E4M3: "float8_e4m3fn"}

# operand format -> {scale code: allowed block sizes}   (src/cuda/tile/_datatype.py:482-489;
# float8_e5m3fnu scales need hardware this build does not target)
_SUPPORTED = {
    "e4m3": {L.MX_E8M0: (32,)},
    "e5m2": {L.MX_E8M0: (32,)},
    "e2m1": {L.MX_E8M0: (16, 32), L.MX_E4M3: (16,)},
}


def _check(rc: int):
    if rc == L.MX_OK:
        return
    msg = L.last_error()
    if rc in (L.MX_ERR_SHAPE, L.MX_ERR_INVALID):
        raise ValueError(msg)
    if rc in (L.MX_ERR_DTYPE, L.MX_ERR_LAYOUT):
        raise TileTypeError(msg)
    if rc == L.MX_ERR_LAUNCH:
        # cext/tile_kernel.cpp:3910-3916
        raise RuntimeError(f"Failed to launch mxgemm kernel: {msg}")
    raise RuntimeError(msg)


def _dtype_name(dt) -> str:
    return str(dt).removeprefix("torch.")


def _elem_format(t: torch.Tensor, fmt: Optional[str]) -> Optional[str]:
    """'e4m3' | 'e5m2' | 'e2m1' for an operand tensor, or None if its dtype is not an MX element type.
    Raw ``uint8`` storage needs an explicit ``fmt`` (FP4 has no byte-sized torch dtype)."""
    if fmt is not None:
        if fmt not in _FMT_CODE:
            raise TileValueError(f"unknown element format {fmt!r}; expected one of {sorted(_FMT_CODE)}")
        if t.dtype != torch.uint8 and _DTYPE_FMT.get(t.dtype) != fmt:
            raise TileTypeError(f"format {fmt!r} does not match tensor dtype {_dtype_name(t.dtype)}")
        return fmt
    return _DTYPE_FMT.get(t.dtype)


def _scale_code(t: torch.Tensor) -> Optional[int]:
    if t.dtype in (torch.float8_e8m0fnu, torch.uint8):
        return L.MX_E8M0
    if t.dtype == torch.float8_e4m3fn:
        return L.MX_E4M3
    return None


def _packed_dim(t: torch.Tensor, k_dim: int, override: Optional[int]) -> int:
    """FP4 storage is packed along the contiguous axis (src/cuda/tile/_stub.py:2625-2679 is a raw byte
    reinterpretation).  Ties (several unit strides) go to the K axis."""
    if override is not None:
        return override % t.dim()
    nd = t.dim()
    cands = [d for d in (nd - 2, nd - 1) if t.stride(d) == 1]
    if not cands:
        raise TileTypeError("FP4 operand has no unit-stride axis to be packed along")
    return k_dim if k_dim in cands else cands[0]


def _logical_shape(t: torch.Tensor, packed_dim: int) -> Tuple[int, ...]:
    return tuple(s * 2 if i == packed_dim else s for i, s in enumerate(t.shape))


@dataclass
class PackedScales:
    """Scales in one of the library's MFMA-ready layouts (see :func:`pack_scales`): ``operand`` "a" or "b" says
    which side of the product they were packed for, ``layout`` which kernels read them (``MX_SCALE_NATIVE``:
    all MFMA kernels but "pingpong32" and "w4p", which read ``MX_SCALE_NATIVE32``)."""
    data: torch.Tensor   # uint8 [batch * bytes]
    rows: int
    K: int
    batch: int = 1
    operand: str = "a"
    layout: int = L.MX_SCALE_NATIVE


def _as_u8(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.uint8 else t.view(torch.uint8)


def _opts(accumulate=False, a_layout=L.MX_SCALE_2D, b_layout=L.MX_SCALE_2D, kernel="auto", block=32, split_k=0):
    o = L.MxGemmOpts()
    o.struct_size = ctypes.sizeof(L.MxGemmOpts)
    o.accumulate = int(bool(accumulate))
    o.a_scale_layout = a_layout
    o.b_scale_layout = b_layout
    if kernel not in L.KERNELS:
        raise TileValueError(f"unknown kernel {kernel!r}; expected one of {sorted(L.KERNELS)}")
    o.kernel = L.KERNELS[kernel]
    o.block_size = block
    o.split_k = int(split_k)
    return o


def _scale_desc(s, rows: int, K: int, block: int, is_b: bool):
    """(descriptor, layout code, tensors to keep alive).  Accepts the plain 2-D/3-D layout, the 4-D
    swizzle_32_4_4 layout, or PackedScales."""
    if isinstance(s, PackedScales):
        if s.rows != rows or s.K != K:
            raise ValueError(f"packed scales were built for rows={s.rows}, K={s.K}; need rows={rows}, K={K}")
        if s.operand != ("b" if is_b else "a"):
            raise ValueError(f"scales packed for operand {s.operand!r} passed as operand {'b' if is_b else 'a'!r}: "
                             "pack_scales(..., operand=...) orders the rows differently for the two sides")
        d = L.MxTensor()
        d.ptr = s.data.data_ptr()
        d.dtype = L.MX_E8M0
        d.ndim = 2
        d.shape[0], d.shape[1] = rows, K // 32
        d.stride[0], d.stride[1] = K // 32, 1
        d.packed_dim = -1
        return d, s.layout
    code = _scale_code(s)
    if s.dim() == 4:
        return L.desc(_as_u8(s), code), L.MX_SCALE_SWIZZLE_32_4_4
    return L.desc(_as_u8(s), code), L.MX_SCALE_2D


class _ScaleCache:
    """PackedScales of scale tensors that were passed before (``cache_scales=True``): what the reference gets by
    reading swizzle_32_4_4 scales in place (test/kernels/scaled_matmul.py:77-104), a weight's scales cost one
    re-layout here instead of one per call.  An entry belongs to a tensor OBJECT (the base tensor of a view, held
    by weak reference) at one ``_version``: a new tensor at the same address, a tensor that died, or one that torch
    has written to since never match.  Writes that bypass torch's version counter (another library writing through
    the raw pointer) are not seen; callers that do that must not ask for caching."""

    def __init__(self, max_entries: int = 64):
        self.max_entries = max_entries
        self._lock = threading.Lock()
        self._entries = collections.OrderedDict()   # key -> (weakref to base, version, PackedScales, event, stream)

    def clear(self):
        with self._lock:
            self._entries.clear()

    def lookup(self, s: torch.Tensor, transposed: bool) -> PackedScales:
        base = s._base if s._base is not None else s
        key = (id(base), s.data_ptr(), tuple(s.shape), tuple(s.stride()), s.dtype, transposed)
        stream = torch.cuda.current_stream(s.device)
        with self._lock:
            e = self._entries.get(key)
            if e is not None and e[0]() is base and e[1] == base._version:
                self._entries.move_to_end(key)
                if e[4] != stream.cuda_stream:
                    stream.wait_event(e[3])          # the re-layout ran on another stream
                    # the copy belongs to the allocator pool of that stream: tell it that this one reads it too,
                    # so that dropping the entry while this stream's GEMM is in flight does not recycle the block
                    e[2].data.record_stream(stream)
                return e[2]
        packed = pack_scales(s, transposed=transposed, operand="b" if transposed else "a")
        if torch.cuda.is_current_stream_capturing():
            return packed                             # memory of the capture's private pool: not for later eager calls
        ev = torch.cuda.Event()
        ev.record(stream)
        with self._lock:
            self._entries[key] = (weakref.ref(base), base._version, packed, ev, stream.cuda_stream)
            # entries of dead tensors first, then the least recently used
            for k in [k for k, v in self._entries.items() if v[0]() is None]:
                del self._entries[k]
            while len(self._entries) > self.max_entries:
                self._entries.popitem(last=False)
        return packed


_SCALE_CACHE = _ScaleCache()


def clear_scale_cache() -> None:
    """Drops every cached scale re-layout (see ``cache_scales`` of :func:`block_scaled_matmul`)."""
    _SCALE_CACHE.clear()


_WS_LOCAL = threading.local()


def _workspace(dev: torch.device, nbytes: int, stream: Optional[int] = None) -> Optional[torch.Tensor]:
    """Scratch for the per-call scale re-layout: one buffer per (host thread, device, stream), grown on
    demand, so the hot path does not go through the allocator.  The kernels that use a buffer are ordered
    on its stream, and no other host thread is ever handed the same buffer, so concurrent callers cannot
    overwrite each other's scales between the re-layout launch and the GEMM launch.  While the stream is
    being captured into a graph the buffer comes fresh from the allocator (the capture's private pool) and
    is not cached: a cached one would later be reused by eager calls while replays of the graph still
    write to it."""
    if nbytes <= 0:
        return None
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=dev)
    cache = _WS_LOCAL.__dict__.setdefault("buffers", {})
    key = (dev.index, L.stream_ptr(dev) if stream is None else stream)
    buf = cache.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=dev)
        cache[key] = buf
    return buf


def _gemm_descs(A, a_fmt, a_pd, As, B, b_fmt, b_pd, Bs, C, block):
    a_log = _logical_shape(A, a_pd if a_fmt == "e2m1" else -1)
    b_log = _logical_shape(B, b_pd if b_fmt == "e2m1" else -1)
    M, K, N = a_log[-2], a_log[-1], b_log[-1]
    dA = L.desc(_as_u8(A), _FMT_CODE[a_fmt], a_pd if a_fmt == "e2m1" else -1)
    dB = L.desc(_as_u8(B), _FMT_CODE[b_fmt], b_pd if b_fmt == "e2m1" else -1)
    dAs, la = _scale_desc(As, M, K, block, False)
    dBs, lb = _scale_desc(Bs, N, K, block, True)
    dC = L.desc(C, L._TORCH_TO_MX[C.dtype])
    return (dA, dAs, dB, dBs, dC), (la, lb), (M, N, K)


def _cacheable_scale(s, block: int) -> bool:
    return (isinstance(s, torch.Tensor) and block == 32 and s.dim() in (2, 4) and _scale_code(s) == L.MX_E8M0)


def _launch_gemm(A, a_fmt, a_pd, As, B, b_fmt, b_pd, Bs, C, *, accumulate, kernel, block, split_k=0,
                 static_scratch=False, cache_scales=False):
    if cache_scales and kernel != "generic" and A.dim() == 2 and B.dim() == 2 and \
            (_cacheable_scale(As, block) or _cacheable_scale(Bs, block)):
        # Native-layout scales are only read by the MFMA kernels: a problem that needs the general kernel reports
        # that before anything is enqueued, and runs with the scales as given.
        As_c = _SCALE_CACHE.lookup(As, False) if _cacheable_scale(As, block) else As
        Bs_c = _SCALE_CACHE.lookup(Bs, True) if _cacheable_scale(Bs, block) else Bs
        try:
            return _launch_gemm(A, a_fmt, a_pd, As_c, B, b_fmt, b_pd, Bs_c, C, accumulate=accumulate, kernel=kernel,
                                block=block, split_k=split_k, static_scratch=static_scratch)
        except (RuntimeError, ValueError, TypeError) as e:
            if "native-layout" not in str(e):
                raise
    dev = A.device
    (dA, dAs, dB, dBs, dC), (la, lb), (M, N, K) = _gemm_descs(A, a_fmt, a_pd, As, B, b_fmt, b_pd, Bs, C, block)
    o = _opts(accumulate, la, lb, kernel, block, split_k)
    lib = L.lib()
    stream = L.stream_ptr(dev)
    if static_scratch:
        fn = lib.mx_gemm_static
        args = (ctypes.byref(dA), ctypes.byref(dAs), ctypes.byref(dB), ctypes.byref(dBs), ctypes.byref(dC),
                ctypes.byref(o), stream)
    else:
        fn = lib.mx_gemm
        need = lib.mx_gemm_workspace_bytes(M, N, K, ctypes.byref(o))
        ws = _workspace(dev, need, stream)
        args = (ctypes.byref(dA), ctypes.byref(dAs), ctypes.byref(dB), ctypes.byref(dBs), ctypes.byref(dC),
                ctypes.byref(o), ws.data_ptr() if ws is not None else None, need, stream)
    if torch.cuda.current_device() == dev.index:
        rc = fn(*args)
    else:
        with torch.cuda.device(dev):
            rc = fn(*args)
    if rc == L.MX_ERR_WORKSPACE:
        raise ValueError(L.last_error())
    _check(rc)
    return C


def bench_block_scaled_matmul(operand_sets, *, warmup: int = 5, iters: int = 20, kernel: str = "auto",
                              a_format: Optional[str] = None, b_format: Optional[str] = None):
    """Times ``block_scaled_matmul(A, A_scale, B, B_scale, C=C)`` the way the reference's tuner times a kernel
    (``_benchmark``, cext/tile_kernel.cpp:3921-4042; protocol of src/cuda/tile/tune/_tune.py:339-395): every
    call between its own pair of HIP events on the current stream.  ``operand_sets`` is a list of
    ``(A, A_scale, B, B_scale, C)`` tuples of one problem shape; call i uses set i % len(operand_sets), which
    takes the place of the reference's cache-flushing memset.  Returns the ``iters`` durations in
    milliseconds (a list of floats); synchronises the stream."""
    n = len(operand_sets)
    if n == 0:
        raise TileValueError("bench_block_scaled_matmul needs at least one operand set")
    arr = [(L.MxTensor * n)() for _ in range(5)]
    layouts, dims, keep = set(), set(), []
    dev = operand_sets[0][0].device
    for i, (A, As, B, Bs, C) in enumerate(operand_sets):
        a_fmt, b_fmt = _elem_format(A, a_format), _elem_format(B, b_format)
        if a_fmt is None or b_fmt is None:
            raise TileTypeError("Unsupported input dtype for mma_scaled, supported input dtypes are "
                                "float8_e4m3fn, float8_e5m2, float4_e2m1fn")
        a_pd = _packed_dim(A, 1, None) if a_fmt == "e2m1" else -1
        b_pd = _packed_dim(B, 0, None) if b_fmt == "e2m1" else -1
        descs, lay, mnk = _gemm_descs(A, a_fmt, a_pd, As, B, b_fmt, b_pd, Bs, C, 32)
        for j in range(5):
            arr[j][i] = descs[j]
        layouts.add(lay)
        dims.add(mnk)
        keep.append((A, As, B, Bs, C))
    if len(layouts) != 1 or len(dims) != 1:
        raise TileValueError("all operand sets must share one problem shape and one scale layout")
    (la, lb), (M, N, K) = layouts.pop(), dims.pop()
    o = _opts(False, la, lb, kernel, 32)
    lib = L.lib()
    need = lib.mx_gemm_workspace_bytes(M, N, K, ctypes.byref(o))
    stream = L.stream_ptr(dev)
    ws = _workspace(dev, need, stream)
    times = (ctypes.c_float * iters)()
    with torch.cuda.device(dev):
        rc = lib.mx_bench_gemm(n, arr[0], arr[1], arr[2], arr[3], arr[4], ctypes.byref(o),
                               ws.data_ptr() if ws is not None else None, need, warmup, iters, times, stream)
    _check(rc)
    return list(times)


# ==================================================================================================
# block_scaled_matmul  (samples/BlockScaledMatMul.py:229-297)
# ==================================================================================================
def block_scaled_matmul(A: torch.Tensor, A_scale, B: torch.Tensor, B_scale, *,
                        out_dtype: torch.dtype = torch.float32, C: Optional[torch.Tensor] = None,
                        accumulate: bool = False, a_format: Optional[str] = None,
                        b_format: Optional[str] = None, kernel: str = "auto", split_k: int = 0,
                        static_scratch: bool = False, cache_scales: bool = False) -> torch.Tensor:
    """C = (A * A_scale) @ (B * B_scale) with fp32 accumulation, returned as ``out_dtype``.

    A (M, K) and B (K, N) hold MX elements: ``float8_e4m3fn`` / ``float8_e5m2``, or FP4 E2M1 packed two
    per byte along the contiguous axis as ``uint8`` / ``float4_e2m1fn_x2`` (pass ``a_format`` /
    ``b_format`` = "e2m1" for uint8 storage).  Scales are E8M0 per 32 elements along K:
    A_scale (M, K/32) and B_scale (K/32, N), or the 4-D ``swizzle_32_4_4`` form, or
    :class:`PackedScales`.  The two operands may use different element formats (for example E4M3
    activations with E2M1 weights): the hardware takes them independently.  The fast kernels need
    K-contiguous operands, i.e. B given as the transposed view of an (N, K) tensor as the reference
    sample does; other layouts run on a slower general kernel.  ``split_k``: 0 lets the library split a
    long K over several workgroups when M x N alone cannot fill the GPU, 1 forbids it, n > 1 forces n slices.
    ``static_scratch``: take the scratch for the scale re-layout from the library's fixed per-GPU buffer
    (``mx_gemm_static``) instead of a torch allocation; with a preallocated ``C`` the call then allocates
    nothing.  Problems that need more than ``lib().mx_static_scratch_bytes()`` raise ``ValueError``; calls that
    overlap on one GPU (several streams or threads) must not share it.
    ``cache_scales``: keep the MFMA-ready re-layout of every 2-D / swizzle_32_4_4 scale tensor passed here and reuse
    it while that tensor object lives and torch has not written to it (``_version``), so that repeated calls with
    the same weights launch the GEMM kernel only; :func:`clear_scale_cache` drops the copies.
    """
    a_fmt, b_fmt = _elem_format(A, a_format), _elem_format(B, b_format)
    if a_fmt is None or b_fmt is None:
        bad = A if a_fmt is None else B
        raise TileTypeError(f"Unsupported input dtype {_dtype_name(bad.dtype)} for mma_scaled, supported input "
                            "dtypes are float8_e4m3fn, float8_e5m2, float4_e2m1fn")
    if A.dim() != 2 or B.dim() != 2:
        raise TileTypeError(f"Expect A and B to be 2D, got {tuple(A.shape)} and {tuple(B.shape)}")
    a_pd = _packed_dim(A, 1, None) if a_fmt == "e2m1" else -1
    b_pd = _packed_dim(B, 0, None) if b_fmt == "e2m1" else -1
    a_log, b_log = _logical_shape(A, a_pd), _logical_shape(B, b_pd)
    # --- the reference wrapper's three checks, same order and wording ---
    if a_log[1] != b_log[0]:
        raise ValueError(f"Incompatible matrices: K dimension of A ({a_log[1]}) "
                         f"must match K dimension of B ({b_log[0]})")
    as_t = A_scale.data if isinstance(A_scale, PackedScales) else A_scale
    bs_t = B_scale.data if isinstance(B_scale, PackedScales) else B_scale
    if A.device != B.device or A.device != as_t.device or A.device != bs_t.device:
        raise ValueError("Input tensors must be on the same device.")
    if not A.is_cuda or not as_t.is_cuda or not B.is_cuda or not bs_t.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")
    for name, s in (("A_scale", A_scale), ("B_scale", B_scale)):
        if not isinstance(s, PackedScales) and _scale_code(s) != L.MX_E8M0:
            raise TileTypeError(f"Unsupported scale dtype {_dtype_name(s.dtype)} for {name}, "
                                "supported scale dtypes are float8_e8m0fnu")
    m, n = a_log[0], b_log[1]
    if C is None:
        if accumulate:
            raise TileValueError("accumulate=True needs an output tensor C to accumulate into")
        if out_dtype not in (torch.float32, torch.bfloat16):
            raise TileTypeError(f"Unsupported output dtype {_dtype_name(out_dtype)}, expected float32 or bfloat16")
        C = torch.empty((m, n), device=A.device, dtype=out_dtype)
    else:
        if tuple(C.shape) != (m, n) or C.dtype not in (torch.float32, torch.bfloat16) or C.device != A.device:
            raise ValueError(f"C must be a ({m}, {n}) float32 or bfloat16 tensor on {A.device}")
    return _launch_gemm(A, a_fmt, a_pd, A_scale, B, b_fmt, b_pd, B_scale, C, accumulate=accumulate,
                        kernel=kernel, block=32, split_k=split_k, static_scratch=static_scratch,
                        cache_scales=cache_scales)


def grouped_block_scaled_matmul(As, A_scales, Bs, B_scales, *, out_dtype: torch.dtype = torch.float32,
                                Cs=None, kernel: str = "auto"):
    """A list of independent block-scaled products ``Cs[i] = (As[i] * A_scales[i]) @ (Bs[i] * B_scales[i])``
    whose sizes may all differ: the block-scaled counterpart of the reference's list-of-problems
    ``grouped_matmul_kernel(As, Bs, Cs, ...)`` (test/kernels/group_gemm.py:10-38, driven as in
    test/test_group_gemm.py).  Every problem follows the rules of :func:`block_scaled_matmul`; all are
    enqueued by one library call on the current stream.  Returns the list of outputs."""
    n = len(As)
    if not (len(A_scales) == len(Bs) == len(B_scales) == n) or (Cs is not None and len(Cs) != n):
        raise ValueError("As, A_scales, Bs, B_scales (and Cs) must be lists of the same length")
    if n == 0:
        return []
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise TileTypeError(f"Unsupported output dtype {_dtype_name(out_dtype)}, expected float32 or bfloat16")
    dA, dAs, dB, dBs, dC = ((L.MxTensor * n)() for _ in range(5))
    outs, keep, layouts = [], [], set()
    dev = As[0].device
    for i in range(n):
        A, B = As[i], Bs[i]
        a_fmt, b_fmt = _elem_format(A, None), _elem_format(B, None)
        if a_fmt is None or b_fmt is None:
            bad = A if a_fmt is None else B
            raise TileTypeError(f"Unsupported input dtype {_dtype_name(bad.dtype)} for mma_scaled, supported "
                                "input dtypes are float8_e4m3fn, float8_e5m2, float4_e2m1fn")
        if A.dim() != 2 or B.dim() != 2:
            raise TileTypeError(f"Expect A and B to be 2D, got {tuple(A.shape)} and {tuple(B.shape)}")
        a_pd = _packed_dim(A, 1, None) if a_fmt == "e2m1" else -1
        b_pd = _packed_dim(B, 0, None) if b_fmt == "e2m1" else -1
        a_log, b_log = _logical_shape(A, a_pd), _logical_shape(B, b_pd)
        if a_log[1] != b_log[0]:
            raise ValueError(f"Incompatible matrices: K dimension of A ({a_log[1]}) "
                             f"must match K dimension of B ({b_log[0]})")
        if not A.is_cuda or A.device != dev or B.device != dev:
            raise ValueError("Input tensors must be on the same CUDA device.")
        M, K, N = a_log[0], a_log[1], b_log[1]
        C = torch.empty((M, N), device=dev, dtype=out_dtype) if Cs is None else Cs[i]
        if tuple(C.shape) != (M, N) or C.dtype not in (torch.float32, torch.bfloat16) or C.device != dev:
            raise ValueError(f"C must be a ({M}, {N}) float32 or bfloat16 tensor on {dev}")
        au, bu = _as_u8(A), _as_u8(B)
        keep += [au, bu]
        dA[i] = L.desc(au, _FMT_CODE[a_fmt], a_pd)
        dB[i] = L.desc(bu, _FMT_CODE[b_fmt], b_pd)
        dAs[i], la = _scale_desc(A_scales[i], M, K, 32, False)
        dBs[i], lb = _scale_desc(B_scales[i], N, K, 32, True)
        layouts.add((la, lb))
        dC[i] = L.desc(C, L._TORCH_TO_MX[C.dtype])
        outs.append(C)
    if len(layouts) != 1:
        raise TileValueError("all problems of a list must pass their scales in the same layout")
    la, lb = layouts.pop()
    o = _opts(False, la, lb, kernel, 32)
    lib = L.lib()
    need = lib.mx_gemm_list_workspace_bytes(n, dA, dB, ctypes.byref(o))
    ws = _workspace(dev, need)
    with torch.cuda.device(dev):
        rc = lib.mx_gemm_list(n, dA, dAs, dB, dBs, dC, ctypes.byref(o), ws.data_ptr() if ws is not None else None,
                              need, L.stream_ptr(dev))
    _check(rc)
    return outs


def cutile_block_scaled_matmul(A, A_scale, B, B_scale) -> torch.Tensor:
    """Exact signature of the reference sample wrapper (fp32 result, samples/BlockScaledMatMul.py:229-230).  The
    reference's kernel reads the scales in place; here the MFMA-ready re-layout of each scale tensor is kept with
    ``cache_scales=True`` (see :func:`block_scaled_matmul`), so repeated calls with the same scale tensors launch the
    GEMM kernel only.  A cached copy is dropped when torch writes to the tensor (its ``_version`` changes); scale
    bytes changed behind torch's back (a foreign library writing through the raw pointer) need
    :func:`clear_scale_cache`, or the general entry :func:`block_scaled_matmul`, which never caches unless asked."""
    return block_scaled_matmul(A, A_scale, B, B_scale, cache_scales=True)


# ==================================================================================================
# mma_scaled  (src/cuda/tile/_stub.py:2198-2329)
# ==================================================================================================
def mma_scaled(x: torch.Tensor, x_scale: torch.Tensor, y: torch.Tensor, y_scale: torch.Tensor, /,
               acc: torch.Tensor, *, x_format: Optional[str] = None, y_format: Optional[str] = None,
               allow_mixed_dtypes: bool = False, kernel: str = "auto") -> torch.Tensor:
    """result[i, j] = sum_k x[i, k] * x_scale[i, k // B] * y[k, j] * y_scale[k // B, j] + acc[i, j]

    Whole-tensor form of the reference's tile op: x [..., M, K], x_scale [..., M, K_s], y [..., K, N],
    y_scale [..., K_s, N], acc [..., M, N] float32; B = K // K_s.  Batch dimensions of x and y broadcast
    against each other.  Returns a new float32 tensor; ``acc`` is not modified.  Type and shape rules
    and their messages follow src/cuda/tile/_datatype.py:492-519 and src/cuda/tile/_ir/ops.py:2089-2137.
    ``allow_mixed_dtypes`` lifts the reference's "x and y must have the same dtype" rule, which the
    CDNA4 instruction does not need.
    """
    for name, t in (("x", x), ("y", y), ("acc", acc), ("x_scale", x_scale), ("y_scale", y_scale)):
        if t.dim() not in (2, 3):
            raise TileTypeError(f"Expect shape of `{name}` to be 2D or 3D, got {tuple(t.shape)}")
    xf, yf = _elem_format(x, x_format), _elem_format(y, y_format)
    x_name = _FMT_NAME.get(xf, _dtype_name(x.dtype))
    y_name = _FMT_NAME.get(yf, _dtype_name(y.dtype))
    if x_name != y_name and not (allow_mixed_dtypes and xf and yf):
        raise TileTypeError(f"x and y must have the same dtype, got {x_name} and {y_name}")
    xs_code, ys_code = _scale_code(x_scale), _scale_code(y_scale)
    xs_name = _SCALE_NAME.get(xs_code, _dtype_name(x_scale.dtype))
    ys_name = _SCALE_NAME.get(ys_code, _dtype_name(y_scale.dtype))
    if xs_name != ys_name:
        raise TileTypeError(f"x_scale and y_scale must have the same dtype, got {xs_name} and {ys_name}")
    if xf is None or yf is None:
        raise TileTypeError(f"Unsupported input dtype {x_name if xf is None else y_name} for mma_scaled, "
                            "supported input dtypes are float8_e4m3fn, float8_e5m2, float4_e2m1fn")
    if xs_code not in _SUPPORTED[xf] or xs_code not in _SUPPORTED[yf]:
        names = ", ".join(_SCALE_NAME[c] for c in _SUPPORTED[xf])
        raise TileTypeError(f"Unsupported scale dtype {xs_name} for input dtype {x_name}, "
                            f"supported scale dtypes are {names}")
    if acc.dtype != torch.float32:
        raise TileTypeError(f"Unsupported acc dtype {_dtype_name(acc.dtype)} for mma_scaled, expected float32")

    x_pd = _packed_dim(x, x.dim() - 1, None) if xf == "e2m1" else -1
    y_pd = _packed_dim(y, y.dim() - 2, None) if yf == "e2m1" else -1
    x_shape, y_shape = _logical_shape(x, x_pd), _logical_shape(y, y_pd)

    def verify(shape, scale_shape, k_axis, name, scale_name, fmt, allowed):
        k_axis %= len(shape)
        if len(shape) != len(scale_shape) or any(a != b for i, (a, b) in enumerate(zip(shape, scale_shape))
                                                 if i != k_axis):
            raise TileTypeError(f"{scale_name} shape {tuple(scale_shape)} is not compatible with {name} shape "
                                f"{tuple(shape)}. All dimensions except K axis {k_axis} must match")
        bs, rem = divmod(shape[k_axis], scale_shape[k_axis]) if scale_shape[k_axis] else (0, 1)
        if rem != 0 or bs not in allowed:
            raise TileTypeError(
                f"For mma_scaled with dtype={_FMT_NAME[fmt]}, scale_dtype={xs_name}: "
                f"{name}.shape[{k_axis}] must be an exact multiple of {scale_name}.shape[{k_axis}] "
                f"with scaling block size B = K // K_s in {set(allowed)}, "
                f"got {name}.shape[{k_axis}] = {shape[k_axis]} and "
                f"{scale_name}.shape[{k_axis}] = {scale_shape[k_axis]}")
        return bs

    bx = verify(x_shape, tuple(x_scale.shape), -1, "x", "x_scale", xf, _SUPPORTED[xf][xs_code])
    by = verify(y_shape, tuple(y_scale.shape), -2, "y", "y_scale", yf, _SUPPORTED[yf][xs_code])
    if x_shape[-1] != y_shape[-2]:
        raise TileTypeError(f"Incompatible shapes for matrix mul on tiles: {x_shape}, {y_shape}.")
    if bx != by:
        raise TileTypeError(f"x and y use different scaling block sizes ({bx} and {by})")
    try:
        batch = torch.broadcast_shapes(x_shape[:-2], y_shape[:-2])
    except RuntimeError:
        raise TileTypeError(f"Incompatible shapes for matrix mul on tiles: {x_shape}, {y_shape}.") from None
    out_shape = tuple(batch) + (x_shape[-2], y_shape[-1])
    if tuple(acc.shape) != out_shape:
        raise TileTypeError(f"Expect acc shape to be {out_shape}, got {tuple(acc.shape)}")
    devs = {t.device for t in (x, x_scale, y, y_scale, acc)}
    if len(devs) != 1:
        raise ValueError("Input tensors must be on the same device.")
    if not x.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")

    out = acc.clone(memory_format=torch.contiguous_format)
    return _launch_gemm(x, xf, x_pd, x_scale, y, yf, y_pd, y_scale, out, accumulate=True, kernel=kernel,
                        block=bx)


# ==================================================================================================
# Quantiser and scale layouts  (test/kernels/kernel_utils.py:38-112)
# ==================================================================================================
def block_quantize(x: torch.Tensor, block_size: int = 32, dtype=torch.float8_e4m3fn, *,
                   scale_mode: str = "ceil"):
    """MX-quantises the last axis of ``x`` on the GPU.  Returns ``(x_q, scale)``.

    ``dtype``: ``torch.float8_e4m3fn`` / ``torch.float8_e5m2`` (x_q has that dtype and x's shape, last axis
    zero-padded to a multiple of the block) or ``"e2m1"`` / ``torch.float4_e2m1fn_x2`` (x_q is ``uint8``,
    two elements per byte along the last axis, low nibble first).  ``scale`` is ``float8_e8m0fnu`` with
    shape [..., K/block].
    scale_mode "ceil": the reference's rule 2^ceil(log2(max(amax/448, 1e-12))) with a non-saturating
    cast; "floor": the OCP MX rule 2^(floor(log2 amax) - emax_elem) with a saturating cast.
    """
    if block_size != 32:
        raise TileValueError(f"only the MX block size 32 is supported by the quantiser, got {block_size}")
    if x.shape[-1] < block_size:
        raise ValueError(f'The requested block size {block_size} is larger than the inner most '
                         f'dimension of the input tensor {x.shape[-1]}')
    if scale_mode not in ("ceil", "floor"):
        raise TileValueError(f"scale_mode must be 'ceil' or 'floor', got {scale_mode!r}")
    if isinstance(dtype, str):
        fmt = dtype
    else:
        fmt = _DTYPE_FMT.get(dtype)
    if fmt not in _FMT_CODE:
        raise TileTypeError(f"Unsupported quantisation dtype {dtype}")
    if x.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TileTypeError(f"Unsupported input dtype {_dtype_name(x.dtype)} for block_quantize")
    if not x.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")
    K = x.shape[-1]
    if K % block_size != 0:
        print('[WARNING] block size is not a multiple of the inner most '
              'dimension of the input tensor')
        print('          padding the input tensor...')
    Kpad = (K + block_size - 1) // block_size * block_size
    lead = tuple(x.shape[:-1])
    x2 = x.reshape(-1, K)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    if fmt == "e2m1":
        xq = torch.empty((rows, Kpad // 2), dtype=torch.uint8, device=x.device)
        dq = L.desc(xq, L.MX_E2M1, 1)
    else:
        xq = torch.empty((rows, Kpad), dtype=torch.uint8, device=x.device)
        dq = L.desc(xq, _FMT_CODE[fmt])
    sc = torch.empty((rows, Kpad // block_size), dtype=torch.uint8, device=x.device)
    dx = L.desc(x2, L._TORCH_TO_MX[x2.dtype])
    ds = L.desc(sc, L.MX_E8M0)
    with torch.cuda.device(x.device):
        rc = L.lib().mx_quantize(ctypes.byref(dx), ctypes.byref(dq), ctypes.byref(ds),
                                 0 if scale_mode == "ceil" else 1, L.stream_ptr(x.device))
    _check(rc)
    if fmt == "e2m1":
        out = xq.reshape(*lead, Kpad // 2)
    else:
        out = xq.view(torch.float8_e4m3fn if fmt == "e4m3" else torch.float8_e5m2).reshape(*lead, Kpad)
    return out, sc.view(torch.float8_e8m0fnu).reshape(*lead, Kpad // block_size)


def swizzle_32_4_4(scale: torch.Tensor) -> torch.Tensor:
    """(M, K_s) -> (M/128, K_s/4, 32, 16), the layout the reference's Blackwell kernels read
    (test/kernels/kernel_utils.py:83-98).  Pure data movement; accepted as-is by block_scaled_matmul."""
    m1, m2, k1 = 32, 4, 4
    M, K_s = scale.shape
    m0, k0 = M // (m1 * m2), K_s // k1
    s = scale.reshape(m0, m2, m1, k0, k1).permute(0, 3, 2, 1, 4).contiguous()
    return s.reshape(m0, k0, 32, 16)


def unswizzle_32_4_4(sw: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`swizzle_32_4_4` (test/kernels/kernel_utils.py:101-112)."""
    m1, m2, k1 = 32, 4, 4
    m0, k0 = sw.shape[0], sw.shape[1]
    return sw.reshape(m0, k0, m1, m2, k1).permute(0, 3, 2, 1, 4).reshape(m0 * m2 * m1, k0 * k1)


def pack_scales(scale: torch.Tensor, *, transposed: bool = False, operand: Optional[str] = None,
                kernel: str = "auto") -> PackedScales:
    """Re-lays E8M0 scales once into the layout the MFMA kernels read directly, so repeated GEMMs with
    the same operand (weights) skip the per-call re-layout.  ``scale`` is [rows, K/32] (``transposed``:
    [K/32, rows], as B_scale is passed), optionally with a leading batch (experts) dimension, or the
    4-D swizzle_32_4_4 tensor.  ``operand``: "a" for the left operand (activations), "b" for the right one
    (weights, expert weights); the two are packed differently.  Default: "b" for a transposed or batched
    tensor, else "a".  ``kernel``: the kernel the scales are for; only "pingpong32" and "w4p" differ from the rest."""
    if not scale.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")
    if operand is None:
        operand = "b" if (transposed or scale.dim() == 3) else "a"
    if operand not in ("a", "b"):
        raise TileValueError(f"operand must be 'a' or 'b', got {operand!r}")
    native = L.MX_SCALE_NATIVE32 if kernel in L.NATIVE32_KERNELS else L.MX_SCALE_NATIVE
    s = _as_u8(scale)
    lib = L.lib()
    if s.dim() == 4:
        rows, K = s.shape[0] * 128, s.shape[1] * 128
        layout, batch = L.MX_SCALE_SWIZZLE_32_4_4, 1
    else:
        if transposed:
            s = s.transpose(-1, -2)
        rows, K = s.shape[-2], s.shape[-1] * 32
        layout, batch = L.MX_SCALE_2D, (s.shape[0] if s.dim() == 3 else 1)
    nbytes = lib.mx_packed_scale_bytes(rows, K)
    out = torch.empty(batch * nbytes, dtype=torch.uint8, device=s.device)
    d = L.desc(s, L.MX_E8M0)
    with torch.cuda.device(s.device):
        rc = lib.mx_pack_scales(ctypes.byref(d), layout, rows, K, native,
                                L.MX_OPERAND_B if operand == "b" else L.MX_OPERAND_A, out.data_ptr(),
                                L.stream_ptr(s.device))
    _check(rc)
    return PackedScales(out, rows, K, batch, operand, native)


# ==================================================================================================
# MoE grouping  (test/kernels/fused_moe.py:113-173, samples/MoE.py:338-375)
# ==================================================================================================
def moe_align_tile_size(topk_ids: torch.Tensor, tile_m: int, num_experts: int, *, exact: bool = True):
    """Device-side equivalent of ``moe_align_tile_size_torch``: returns (sorted_token_ids int32,
    sorted_expert_ids int32).  With ``exact`` (the default) the outputs are trimmed to the used length,
    which costs one host synchronisation, exactly like the reference; with ``exact=False`` nothing
    synchronises and the outputs keep their worst-case length, padded with the sentinel
    ``num_tokens * topk`` (and expert 0), which the grouped GEMM skips."""
    if not topk_ids.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")
    flat = topk_ids.reshape(-1).to(torch.int32).contiguous()
    n = flat.numel()
    lib = L.lib()
    max_slots = lib.mx_moe_align_max_slots(n, num_experts, tile_m)
    ids = torch.empty(max_slots, dtype=torch.int32, device=flat.device)
    eids = torch.empty(max_slots // tile_m, dtype=torch.int32, device=flat.device)
    used = torch.zeros(1, dtype=torch.int32, device=flat.device)
    need = lib.mx_moe_align_workspace_bytes(n, num_experts)
    ws = _workspace(flat.device, need)
    with torch.cuda.device(flat.device):
        rc = lib.mx_moe_align(flat.data_ptr(), n, num_experts, tile_m, ids.data_ptr(), eids.data_ptr(),
                              used.data_ptr(), ws.data_ptr() if ws is not None else None, need,
                              L.stream_ptr(flat.device))
    _check(rc)
    if exact:
        u = int(used.item())
        return ids[:u], eids[:u // tile_m]
    return ids, eids


def invoke_fused_moe_scaled(A: torch.Tensor, A_scale: torch.Tensor, B: torch.Tensor, B_scale,
                            C: torch.Tensor, topk_weights: Optional[torch.Tensor],
                            sorted_token_ids: torch.Tensor, sorted_expert_ids: torch.Tensor,
                            mul_routed_weight: bool, num_token_replicas: int, tile_m: int, *,
                            a_format: Optional[str] = None, b_format: Optional[str] = None,
                            kernel: str = "auto") -> None:
    """Grouped block-scaled GEMM with the calling convention of ``invoke_fused_moe_kernel``
    (samples/MoE.py:338-375): for every slot of ``sorted_token_ids`` holding id < num_tokens*topk,
    ``C[id] = (A[id // num_token_replicas] * A_scale) @ (B[e] * B_scale[e]).T`` (times
    ``topk_weights[id]`` if ``mul_routed_weight``), e = sorted_expert_ids[slot // tile_m].
    A (tokens, K) MX elements with A_scale (tokens, K/32); B (experts, N, K) with B_scale
    (experts, N, K/32) or PackedScales; C (tokens, topk, N) or (tokens*topk, N), fp32 or bf16."""
    a_fmt, b_fmt = _elem_format(A, a_format), _elem_format(B, b_format)
    if a_fmt is None or b_fmt is None:
        raise TileTypeError("Unsupported input dtype for mma_scaled, supported input dtypes are "
                            "float8_e4m3fn, float8_e5m2, float4_e2m1fn")
    if A.dim() != 2 or B.dim() != 3:
        raise TileTypeError(f"Expect A to be 2D and B 3D, got {tuple(A.shape)} and {tuple(B.shape)}")
    if not A.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")
    C2 = C.view(-1, C.shape[-1])
    num_valid = C2.shape[0]
    dev = A.device
    dA = L.desc(_as_u8(A), _FMT_CODE[a_fmt], 1 if a_fmt == "e2m1" else -1)
    dB = L.desc(_as_u8(B), _FMT_CODE[b_fmt], 2 if b_fmt == "e2m1" else -1)
    K, N, E = dA.shape[1], dB.shape[1], dB.shape[0]
    dAs = L.desc(_as_u8(A_scale), L.MX_E8M0)
    if isinstance(B_scale, PackedScales):
        if B_scale.rows != N or B_scale.K != K or B_scale.batch != E:
            raise ValueError("packed B_scale does not match B")
        if B_scale.operand != "b":
            raise ValueError("expert scales must be packed with operand='b'")
        dBs = L.MxTensor()
        dBs.ptr = B_scale.data.data_ptr()
        dBs.dtype, dBs.ndim = L.MX_E8M0, 3
        dBs.shape[0], dBs.shape[1], dBs.shape[2] = E, N, K // 32
        dBs.stride[0], dBs.stride[1], dBs.stride[2] = N * (K // 32), K // 32, 1
        dBs.packed_dim = -1
        lb = B_scale.layout
    else:
        dBs, lb = L.desc(_as_u8(B_scale), L.MX_E8M0), L.MX_SCALE_2D
    dC = L.desc(C2, L._TORCH_TO_MX[C2.dtype])
    o = _opts(False, L.MX_SCALE_2D, lb, kernel, 32)
    w = None
    if mul_routed_weight:
        w = topk_weights.reshape(-1).to(torch.float32).contiguous()
    ids = sorted_token_ids.to(torch.int32).contiguous()
    eids = sorted_expert_ids.to(torch.int32).contiguous()
    lib = L.lib()
    need = lib.mx_gemm_grouped_workspace_bytes(ids.numel(), N, K, E, ctypes.byref(o))
    ws = _workspace(dev, max(need, 1))
    with torch.cuda.device(dev):
        rc = lib.mx_gemm_grouped(ctypes.byref(dA), ctypes.byref(dAs), ctypes.byref(dB), ctypes.byref(dBs),
                                 ctypes.byref(dC), w.data_ptr() if w is not None else None, ids.data_ptr(),
                                 ids.numel(), eids.data_ptr(), tile_m, num_token_replicas, num_valid,
                                 ctypes.byref(o), ws.data_ptr(), need, L.stream_ptr(dev))
    _check(rc)


def silu_and_mul_quantize(gate_up: torch.Tensor, dtype=torch.float8_e4m3fn, *, scale_mode: str = "floor"):
    """``silu(gate_up[..., :F]) * gate_up[..., F:]`` MX-quantised along F in blocks of 32, in one pass
    (the reference runs silu_and_mul_kernel, test/kernels/fused_moe.py:85-108, into a bf16 buffer; here the
    product never leaves registers before it is quantised).  Returns ``(x_q, scale)`` like
    :func:`block_quantize`."""
    if scale_mode not in ("ceil", "floor"):
        raise TileValueError(f"scale_mode must be 'ceil' or 'floor', got {scale_mode!r}")
    fmt = dtype if isinstance(dtype, str) else _DTYPE_FMT.get(dtype)
    if fmt not in _FMT_CODE:
        raise TileTypeError(f"Unsupported quantisation dtype {dtype}")
    if gate_up.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TileTypeError(f"Unsupported input dtype {_dtype_name(gate_up.dtype)} for silu_and_mul_quantize")
    if not gate_up.is_cuda:
        raise ValueError("Input tensors must be on a CUDA device.")
    if gate_up.shape[-1] % 2 != 0:
        raise ValueError("gate_up must have 2 * intermediate_size columns (gate + up projection)")
    F = gate_up.shape[-1] // 2
    if F < 32:
        raise ValueError(f'The requested block size 32 is larger than the inner most '
                         f'dimension of the input tensor {F}')
    lead = tuple(gate_up.shape[:-1])
    x2 = gate_up.reshape(-1, 2 * F)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    Fpad = (F + 31) // 32 * 32
    if fmt == "e2m1":
        xq = torch.empty((rows, Fpad // 2), dtype=torch.uint8, device=x2.device)
        dq = L.desc(xq, L.MX_E2M1, 1)
    else:
        xq = torch.empty((rows, Fpad), dtype=torch.uint8, device=x2.device)
        dq = L.desc(xq, _FMT_CODE[fmt])
    sc = torch.empty((rows, Fpad // 32), dtype=torch.uint8, device=x2.device)
    dx = L.desc(x2, L._TORCH_TO_MX[x2.dtype])
    ds = L.desc(sc, L.MX_E8M0)
    with torch.cuda.device(x2.device):
        rc = L.lib().mx_silu_mul_quantize(ctypes.byref(dx), ctypes.byref(dq), ctypes.byref(ds),
                                          0 if scale_mode == "ceil" else 1, L.stream_ptr(x2.device))
    _check(rc)
    if fmt == "e2m1":
        out = xq.reshape(*lead, Fpad // 2)
    else:
        out = xq.view(torch.float8_e4m3fn if fmt == "e4m3" else torch.float8_e5m2).reshape(*lead, Fpad)
    return out, sc.view(torch.float8_e8m0fnu).reshape(*lead, Fpad // 32)


def cutile_moe_scaled(hidden_states: torch.Tensor, hidden_scale: torch.Tensor,
                      w1: torch.Tensor, w1_scale, w2: torch.Tensor, w2_scale,
                      topk_weights: torch.Tensor, topk_ids: torch.Tensor, tile_m: int = 256, *,
                      out_dtype: torch.dtype = torch.bfloat16, scale_mode: str = "floor",
                      w_format: Optional[str] = None, kernel: str = "auto") -> torch.Tensor:
    """Block-scaled Mixture-of-Experts forward with the structure of ``cutile_moe``
    (samples/MoE.py:197-288): align -> grouped gate+up GEMM -> SiLU(gate) * up -> grouped down GEMM
    with the routed-weight multiply -> sum over the top-k copies.

    hidden_states (tokens, H) MX elements with hidden_scale (tokens, H/32); w1 (E, 2F, H) and w2 (E, H, F)
    MX elements (FP4 packed along the last axis, ``w_format="e2m1"``) with scales (E, rows, K/32) or
    :class:`PackedScales`; topk_weights / topk_ids (tokens, topk).  The intermediate activation is
    re-quantised to E4M3 on the device (one fused pass) so that both GEMMs run block-scaled.  Nothing in the
    call synchronises with the host.  Returns (tokens, H) in ``out_dtype``."""
    if hidden_states.dim() != 2 or w1.dim() != 3 or w2.dim() != 3:
        raise TileTypeError("hidden_states must be 2D, w1 and w2 3D")
    T = hidden_states.shape[0]
    E = w1.shape[0]
    topk = topk_ids.shape[1]
    two_f = w1.shape[1]
    H_out = w2.shape[1]
    if two_f % 2 != 0:
        raise ValueError("w1 must have 2 * intermediate_size rows (gate + up projection)")
    dev = hidden_states.device
    ids, eids = moe_align_tile_size(topk_ids, tile_m, E, exact=False)
    cache1 = torch.empty((T * topk, two_f), dtype=torch.bfloat16, device=dev)
    invoke_fused_moe_scaled(hidden_states, hidden_scale, w1, w1_scale, cache1, None, ids, eids, False, topk,
                            tile_m, b_format=w_format, kernel=kernel)
    a2, a2s = silu_and_mul_quantize(cache1, torch.float8_e4m3fn, scale_mode=scale_mode)
    # rows of ids that no expert claimed (ids outside [0, E)) stay zero, as in the reference's zeros() caches
    cache3 = torch.zeros((T, topk, H_out), dtype=torch.float32, device=dev)
    invoke_fused_moe_scaled(a2, a2s, w2, w2_scale, cache3, topk_weights, ids, eids, True, 1, tile_m,
                            b_format=w_format, kernel=kernel)
    return cache3.sum(dim=1).to(out_dtype)
