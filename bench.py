#!/usr/bin/env python3
"""Benchmark of the block-scaled (MX) matmul path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only c2,c3,c4,c5,r4096] [--kernel NAME] [--no-cpu]

A "step" is one call of the hot path -- block_scaled_matmul(A, A_scale, B, B_scale, out_dtype=bf16) with
the reference's tensor layouts (plain (M, K/32) / (K/32, N) E8M0 scales, so the per-call scale re-layout
is inside the step) -- on synthetic operands already resident in HBM.  The headline workload is the
configuration the metric is quoted on: MXFP8 E4M3 x E4M3, M = N = K = 8192, bf16 output.  The other
single-GPU configurations of the metric (MXFP4 8192^3, the M = 32 decode GEMM, the MoE grouped GEMM) are
timed the same way and reported under "extra".

Prints ONE JSON line.  `roofline` describes the dominant kernel of the headline workload: algorithmic
flops per launch divided by the kernel's average duration, measured with one pair of HIP events per launch on
the launch stream around launches of the GEMM kernel alone (scales pre-packed, so no other kernel runs between
the events).  The samples follow the reference tuner's protocol (src/cuda/tile/tune/_tune.py:339-395): batches
of 5 until the 95 % confidence half-width is below 1 % of the mean (or 0.5 us), at least 20 samples; n, mean,
min and the half-width are reported.  Every configuration under `extra` carries the same kind of object.
`traffic` (HBM bytes per launch) comes from rocprofv3 --pmc runs of this file; it is read from the summary
under profiles/ so that it cannot outlive the kernel it was measured on (null if no figure is kept there).
`cpu_baseline` times the oracle's dequantize + fp32 matmul on this host's cores on an N-slice of the same
workload.  Operand sets are rotated so that no launch finds its inputs in L2 / Infinity Cache.  Every timed
region is preceded by an untimed settle period of the same steps (see _settle) and the W warm-up steps.
"""
from __future__ import annotations

import argparse
import json
import os
import pathlib
import re
import sys
import time

ROOT = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT / "cutile-python_amd"))
sys.path.insert(0, str(ROOT))

import numpy as np  # noqa: E402
import torch  # noqa: E402

PEAK_TFLOPS = {"mxfp8": 5033.0, "mxfp4": 10066.0}   # MI355X dense MFMA peaks (vendor figures)
PEAK_HBM_GBS = 8000.0
PROFILE_TRAFFIC = ROOT / "profiles" / "hbm_traffic_pmc.md"
METRIC = "MX GEMM TFLOP/s (+% MFMA peak) 8192^3 MXFP8/MXFP4; GB/s at M=32 decode"


def _sync():
    torch.cuda.synchronize()


SETTLE_S = 0.06


def _settle(fn):
    """Untimed: repeats the step for SETTLE_S seconds.  When load arrives after an idle period the GPU's power
    management first boosts, then throttles (steps 5 - 40 of the MXFP8 GEMM run up to 35 % longer), and
    reaches its steady clock after about 35 ms; a measurement that starts earlier times that transient."""
    _sync()
    t0 = time.perf_counter()
    i = 0
    while time.perf_counter() - t0 < SETTLE_S:
        fn(i)
        i += 1
        if i % 8 == 0:
            _sync()
    _sync()


def _time_wall(fn, steps, warmup):
    """Contract timing: W untimed warm-up steps, then exactly K steps between synchronisations."""
    _settle(fn)
    for i in range(warmup):
        fn(i)
    _sync()
    t0 = time.perf_counter()
    for i in range(steps):
        fn(warmup + i)
    _sync()
    return (time.perf_counter() - t0) / steps


def _time_events(fn, steps, warmup):
    """Average duration of one launch from HIP events recorded on the launch stream."""
    _settle(fn)
    for i in range(warmup):
        fn(i)
    _sync()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        fn(warmup + i)
    stop.record()
    _sync()
    return start.elapsed_time(stop) * 1e-3 / steps


class Welford:
    """Running mean / variance of per-launch durations and the stopping rule of the reference's tuner
    (src/cuda/tile/tune/_tune.py:339-395)."""

    def __init__(self):
        self.n, self.mean, self.m2, self.min, self.max = 0, 0.0, 0.0, float("inf"), 0.0

    def add(self, x):
        self.n += 1
        d = x - self.mean
        self.mean += d / self.n
        self.m2 += d * (x - self.mean)
        self.min, self.max = min(self.min, x), max(self.max, x)

    @property
    def margin(self):   # 95 % confidence half-width of the mean
        return 1.96 * (self.m2 / (self.n - 1) / self.n) ** 0.5 if self.n > 1 else float("inf")

    def converged(self, min_samples):
        return self.n >= min_samples and (self.margin <= 0.01 * self.mean or self.margin <= 0.5 or self.n >= 1000
                                          or self.mean * self.n > 5e6)

    def stats(self):
        return {"n": self.n, "mean_us": self.mean, "min_us": self.min, "max_us": self.max, "ci95_us": self.margin}


def measure(batch_fn, min_samples=20, batch=5):
    """batch_fn(k) -> k per-launch durations in microseconds (it does its own warm-up on the first call)."""
    w = Welford()
    while not w.converged(min_samples):
        for t in batch_fn(batch):
            w.add(t)
    return w


def profile_traffic(tag):
    """HBM bytes per launch of configuration `tag`, from the line `traffic_bytes[tag] = N` of the rocprofv3
    summary under profiles/ (None if there is none)."""
    try:
        m = re.search(rf"traffic_bytes\[{tag}\]\s*=\s*(\d+)", PROFILE_TRAFFIC.read_text())
        return int(m.group(1)) if m else None
    except OSError:
        return None


def profile_clock(tag):
    """Shader clock (GHz) the kernel of configuration `tag` sustained in the rocprofv3 counter run kept under
    profiles/ (line `clock_ghz[tag] = X`: kernel cycles from SQ_BUSY_CYCLES over the kernel's duration); None if
    no figure is kept there."""
    try:
        m = re.search(rf"clock_ghz\[{tag}\]\s*=\s*([0-9.]+)", PROFILE_TRAFFIC.read_text())
        return float(m.group(1)) if m else None
    except OSError:
        return None


NOMINAL_CLOCK_GHZ = 2.4   # the clock the dense MFMA peaks are quoted at


def roofline(bound, achieved, peak, unit, tag, kernel, w, work):
    r = {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
         "traffic": profile_traffic(tag), "kernel": kernel, "kernel_ms": w.mean * 1e-3,
         ("flops_per_launch" if bound == "mfma" else "bytes_per_launch"): work, **w.stats()}
    if bound == "mfma":
        # the chip lowers its clock under this load: the fraction of the peak at the clock the kernel actually ran at
        # (from the counter run under profiles/, like `traffic`) is the share of cycles the matrix pipe was fed
        clk = profile_clock(tag)
        r["clock_ghz"] = clk
        r["frac_at_clock"] = achieved / (peak * clk / NOMINAL_CLOCK_GHZ) if clk else None
    return r


def _quantized(ct, rows, K, fmt, seed, dev, dist, std=1.0, cpu_seeded=True):
    """(storage, scale) on the device.  The first operand set of every workload comes from a seeded CPU
    generator (the workload definition); rotation copies are drawn on the device."""
    if cpu_seeded:
        g = torch.Generator().manual_seed(seed)
        x = torch.randn((rows, K), generator=g) if dist == "randn" else torch.rand((rows, K), generator=g) * 12 - 6
        x = (x * std).to(dev)
    else:
        g = torch.Generator(device=dev).manual_seed(seed)
        x = torch.randn((rows, K), generator=g, device=dev) if dist == "randn" else \
            torch.rand((rows, K), generator=g, device=dev) * 12 - 6
        x = x * std
    q, s = ct.block_quantize(x, 32, fmt, scale_mode="floor")
    del x
    return q, s


def _oracle_rows(O, a_q, a_s, b_q, b_s, rows, a_fmt, b_fmt):
    """CPU oracle of C[rows, :] for K-contiguous operands a (M, K) and b (N, K)."""
    def codes(t, fmt):
        u = t.view(torch.uint8).cpu().numpy()
        return O.unpack_fp4(u) if fmt == O.E2M1 else u
    a = O.dequantize(codes(a_q[rows], a_fmt), a_s[rows].view(torch.uint8).cpu().numpy(), a_fmt)
    b = O.dequantize(codes(b_q, b_fmt), b_s.view(torch.uint8).cpu().numpy(), b_fmt)
    return a @ b.T


def _check_rows(O, c, ref, rows, tol, what):
    err = O.rel_fro(c[rows].float().cpu(), ref)
    if not err <= tol:
        raise SystemExit(f"bench: {what}: relative Frobenius error {err:.3e} exceeds {tol}")
    return err


def _events_batch(fn, settle=True):
    """batch_fn for `measure`: each call of fn(i) between its own pair of events on the current stream."""
    state = {"i": 0, "warm": False}

    def batch(k):
        if not state["warm"]:
            if settle:
                _settle(fn)
            for _ in range(3):
                fn(state["i"])
                state["i"] += 1
            state["warm"] = True
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(k)]
        for e0, e1 in ev:
            e0.record()
            fn(state["i"])
            e1.record()
            state["i"] += 1
        _sync()
        return [e0.elapsed_time(e1) * 1e3 for e0, e1 in ev]
    return batch


def bench_gemm(ct, O, dev, M, N, K, fmt, dist, steps, warmup, check, kernel="auto", nsets=3):
    """Square / large GEMM configurations (MXFP8 or MXFP4, bf16 out)."""
    tfmt = torch.float8_e4m3fn if fmt == O.E4M3 else "e2m1"
    kw = {} if fmt == O.E4M3 else {"a_format": "e2m1", "b_format": "e2m1"}
    sets = []
    for i in range(nsets):
        a_q, a_s = _quantized(ct, M, K, tfmt, 1234 + 2 * i, dev, dist, cpu_seeded=(i == 0))
        b_q, b_s = _quantized(ct, N, K, tfmt, 1235 + 2 * i, dev, dist, cpu_seeded=(i == 0))
        sets.append((a_q, a_s, b_q, b_s, torch.empty((M, N), dtype=torch.bfloat16, device=dev)))
    err = None
    if check:
        a_q, a_s, b_q, b_s, c = sets[0]
        ct.block_scaled_matmul(a_q, a_s, b_q.T, b_s.T, C=c, kernel=kernel, **kw)
        rows = torch.arange(0, M, max(1, M // 32))[:32]
        err = _check_rows(O, c, _oracle_rows(O, a_q, a_s, b_q, b_s, rows, fmt, fmt), rows, 8e-3, f"{fmt} {M}x{N}x{K}")

    def step(i):
        a_q, a_s, b_q, b_s, c = sets[i % nsets]
        ct.block_scaled_matmul(a_q, a_s, b_q.T, b_s.T, C=c, kernel=kernel, **kw)

    t_step = _time_wall(step, steps, warmup)
    # kernel alone: scales pre-packed, one pair of HIP events per launch recorded by the library's own timing
    # entry point (mx_bench_gemm) on the launch stream, operand sets rotated
    packed = [(s[0], ct.pack_scales(s[1], operand="a", kernel=kernel), s[2].T, ct.pack_scales(s[3], operand="b", kernel=kernel),
               s[4]) for s in sets]
    state = {"warm": False}

    def batch(k):
        if not state["warm"]:
            _settle(lambda i: ct.block_scaled_matmul(*packed[i % nsets][:4], C=packed[i % nsets][4], kernel=kernel, **kw))
            state["warm"] = True
        return [t * 1e3 for t in ct.bench_block_scaled_matmul(packed, warmup=3, iters=k, kernel=kernel, **kw)]

    w = measure(batch, batch=10)
    flops = 2.0 * M * N * K
    return {"ms_per_step": t_step * 1e3, "tflops": flops / t_step * 1e-12, "kernel": w,
            "kernel_tflops": flops / (w.mean * 1e-6) * 1e-12, "rel_fro_vs_oracle": err, "flops": flops, "sets": sets}


def vendor_scaled_mm(sets, steps, warmup):
    """Context only, not part of the product path: the vendor library's MXFP8 GEMM (torch._scaled_mm with
    E8M0 scales, hipBLASLt underneath) on the same operands, timed like the kernel-only leg."""
    def run(i):
        a_q, a_s, b_q, b_s, _ = sets[i % len(sets)]
        return torch._scaled_mm(a_q, b_q.T, scale_a=a_s, scale_b=b_s, out_dtype=torch.bfloat16)
    try:
        run(0)
        _sync()
        t = _time_events(run, steps, warmup)
    except Exception as e:   # an image without MX support in its BLAS: report that, the bench goes on
        return {"error": f"{type(e).__name__}: {str(e)[:160]}"}
    M, K = sets[0][0].shape
    N = sets[0][2].shape[0]
    return {"kernel_ms": t * 1e3, "tflops": 2.0 * M * N * K / t * 1e-12}


def bench_recorded_4096(ct, O, dev, steps, warmup, check, nsets=4):
    """The one problem the reference keeps a measurement of (test/benchmark_tuning.json:549-561, problem in
    test/bench_matmul.py:467-495): MXFP8 E4M3, M = N = K = 4096, scales in the swizzle_32_4_4 form, fp32 output;
    71.379 us mean kernel time on a B200.  Reported beside it, not as vs_baseline: the headline metric is
    quoted on 8192^3."""
    M = N = K = 4096
    sets = []
    for i in range(nsets):
        a_q, a_s = _quantized(ct, M, K, torch.float8_e4m3fn, 4001 + 2 * i, dev, "randn", cpu_seeded=(i == 0))
        b_q, b_s = _quantized(ct, N, K, torch.float8_e4m3fn, 4002 + 2 * i, dev, "randn", cpu_seeded=(i == 0))
        sets.append((a_q, a_s, b_q, b_s, ct.swizzle_32_4_4(a_s), ct.swizzle_32_4_4(b_s),
                     torch.empty((M, N), dtype=torch.float32, device=dev)))
    err = None
    if check:
        a_q, a_s, b_q, b_s, a_sw, b_sw, c = sets[0]
        ct.block_scaled_matmul(a_q, a_sw, b_q.T, b_sw, C=c)
        rows = torch.arange(0, M, M // 32)[:32]
        err = _check_rows(O, c, _oracle_rows(O, a_q, a_s, b_q, b_s, rows, O.E4M3, O.E4M3), rows, 1e-3, "4096^3 swizzled")

    def step(i):
        a_q, _, b_q, _, a_sw, b_sw, c = sets[i % nsets]
        ct.block_scaled_matmul(a_q, a_sw, b_q.T, b_sw, C=c)

    t_call = _time_events(step, steps, warmup)

    # the same calls with the wrapper's scale cache: like the reference, which reads the swizzled scales in place,
    # a call then launches the GEMM kernel only (the first call per scale tensor re-lays it once)
    def step_cached(i):
        a_q, _, b_q, _, a_sw, b_sw, c = sets[i % nsets]
        ct.block_scaled_matmul(a_q, a_sw, b_q.T, b_sw, C=c, cache_scales=True)

    t_call_cached = _time_events(step_cached, steps, max(warmup, 2 * nsets))

    # the reference's own signature, cutile_block_scaled_matmul(A, A_scale, B, B_scale) -> C (it allocates the fp32
    # result like the sample does, and keeps the scale re-layout between calls)
    def step_drop_in(i):
        a_q, _, b_q, _, a_sw, b_sw, _ = sets[i % nsets]
        ct.cutile_block_scaled_matmul(a_q, a_sw, b_q.T, b_sw)

    t_call_drop_in = _time_events(step_drop_in, steps, max(warmup, 2 * nsets))
    packed = [(s[0], ct.pack_scales(s[1], operand="a"), s[2].T, ct.pack_scales(s[3], operand="b"), s[6]) for s in sets]
    w = measure(lambda k: [t * 1e3 for t in ct.bench_block_scaled_matmul(packed, warmup=3, iters=k)], batch=10)
    flops = 2.0 * M * N * K
    return {"call_us_incl_scale_relayout": t_call * 1e6, "tflops": flops / t_call * 1e-12,
            "call_us_cached_scales": t_call_cached * 1e6, "call_us_drop_in_signature": t_call_drop_in * 1e6,
            "gemm_kernel_us": w.mean, "gemm_kernel_tflops": flops / w.mean * 1e-6, **w.stats(),
            "reference_recorded_us_b200": 71.379, "reference_recorded_ci_us_b200": 0.294,
            "rel_fro_vs_oracle": err}


def bench_shape(ct, O, dev, M, N, K, check, kernels=("auto", "mfma128", "pingpong"), swizzled=True, nsets=3):
    """One problem of the reference's own benchmark list (test/bench_matmul.py:419-425 shapes, :98-112 check): MXFP8
    E4M3, scales in the swizzle_32_4_4 form, fp32 output, checked against the oracle before timing.  Reports a call
    through the drop-in signature (scale re-layout inside) and the GEMM kernel alone for the kernel MX_KERNEL_AUTO
    picks and for each candidate kernel, so that the cost of the selection rule is on record."""
    nsets = max(nsets, min(8, -(-(300 << 20) // (M * K + N * K + M * N * 4))))   # rotate more than the Infinity Cache
    sets = []
    for i in range(nsets):
        a_q, a_s = _quantized(ct, M, K, torch.float8_e4m3fn, 5001 + 2 * i, dev, "randn", cpu_seeded=(i == 0))
        b_q, b_s = _quantized(ct, N, K, torch.float8_e4m3fn, 5002 + 2 * i, dev, "randn", cpu_seeded=(i == 0))
        sw = swizzled and M % 128 == 0 and N % 128 == 0 and (K // 32) % 4 == 0
        sets.append((a_q, a_s, b_q, b_s, ct.swizzle_32_4_4(a_s) if sw else a_s, ct.swizzle_32_4_4(b_s) if sw else b_s.T,
                     torch.empty((M, N), dtype=torch.float32, device=dev)))
    err = None
    if check:
        a_q, a_s, b_q, b_s, a_sw, b_sw, c = sets[0]
        ct.block_scaled_matmul(a_q, a_sw, b_q.T, b_sw, C=c)
        rows = torch.arange(0, M, max(1, M // 32))[:32]
        err = _check_rows(O, c, _oracle_rows(O, a_q, a_s, b_q, b_s, rows, O.E4M3, O.E4M3), rows, 1e-3, f"{M}x{N}x{K}")

    def step(i):
        a_q, _, b_q, _, a_sw, b_sw, c = sets[i % nsets]
        ct.block_scaled_matmul(a_q, a_sw, b_q.T, b_sw, C=c)

    t_call = _time_events(step, 50, 10)
    flops = 2.0 * M * N * K
    out = {"M": M, "N": N, "K": K, "call_us_incl_scale_relayout": t_call * 1e6, "rel_fro_vs_oracle": err, "kernel_us": {}}
    packed = [(s[0], ct.pack_scales(s[1], operand="a"), s[2].T, ct.pack_scales(s[3], operand="b"), s[6]) for s in sets]
    for kern in kernels:
        try:
            w = measure(lambda k: [t * 1e3 for t in ct.bench_block_scaled_matmul(packed, warmup=3, iters=k, kernel=kern)], batch=10)
        except (ValueError, TypeError, RuntimeError) as e:      # a kernel that does not take this shape
            out["kernel_us"][kern] = {"error": str(e)[:120]}
            continue
        out["kernel_us"][kern] = {**w.stats(), "tflops": flops / w.mean * 1e-6}
        if kern == "auto":
            out["roofline"] = roofline("mfma", flops / w.mean * 1e-6, PEAK_TFLOPS["mxfp8"], "TFLOP/s", "none",
                                       "kernel chosen by MX_KERNEL_AUTO", w, flops)
    best = min((v["mean_us"] for v in out["kernel_us"].values() if "mean_us" in v), default=None)
    auto = out["kernel_us"].get("auto", {}).get("mean_us")
    out["auto_over_best"] = auto / best if auto and best else None
    return out


def probe_mfma(ct, dev, reps=6):
    """What the chip sustains on the scaled MFMA instruction out of registers alone (mx_probe_mfma_rate: the GEMM
    kernel's register tile, two waves per SIMD, no LDS or memory traffic), for several kinds of operand bits.  The
    chip lowers its clock as operand bits toggle, so the rate on real data is the ceiling of any GEMM schedule on that
    data.  Each kind is run `reps` times back to back (about 20 ms each) and the last run is reported: by then the
    power management has settled.  (The clock each kind ran at is in the rocprofv3 summary of this probe under
    profiles/: SQ_BUSY_CYCLES over the launch's duration.)"""
    import ctypes
    lib = ct.lib()
    n_cu = torch.cuda.get_device_properties(dev).multi_processor_count
    nbytes = 12 * 512 * 32
    g = torch.Generator(device=dev).manual_seed(7)

    def fp8_real():
        q, _ = ct.block_quantize(torch.randn((192, 1024), generator=g, device=dev), 32, torch.float8_e4m3fn, scale_mode="floor")
        return q.view(torch.uint8).reshape(-1)

    def fp4_real():
        q, _ = ct.block_quantize(torch.rand((96, 2048), generator=g, device=dev) * 12 - 6, 32, "e2m1", scale_mode="floor")
        f = torch.zeros((12 * 512, 32), dtype=torch.uint8, device=dev)
        f[:, :16] = q.reshape(12 * 512, 16)
        return f.reshape(-1)

    def fp4_random():
        f = torch.zeros((12 * 512, 32), dtype=torch.uint8, device=dev)
        f[:, :16] = torch.randint(0, 256, (12 * 512, 16), generator=g, device=dev, dtype=torch.uint8)
        return f.reshape(-1)

    kinds = [("mxfp8", "zeros", ct._lib.MX_E4M3, lambda: torch.zeros(nbytes, dtype=torch.uint8, device=dev)),
             ("mxfp8", "uniform random bytes", ct._lib.MX_E4M3,
              lambda: torch.randint(0, 256, (nbytes,), generator=g, device=dev, dtype=torch.uint8)),
             ("mxfp8", "E4M3 of N(0,1), floor-rule block scales (the headline workload's data)", ct._lib.MX_E4M3, fp8_real),
             ("mxfp4", "zeros", ct._lib.MX_E2M1, lambda: torch.zeros(nbytes, dtype=torch.uint8, device=dev)),
             ("mxfp4", "uniform random nibbles", ct._lib.MX_E2M1, fp4_random),
             ("mxfp4", "E2M1 of uniform(-6, 6), floor-rule block scales (the MXFP4 workload's data)", ct._lib.MX_E2M1, fp4_real)]
    sink = torch.empty(n_cu * 512, dtype=torch.float32, device=dev)
    out = []
    for peak_key, name, fmt, make in kinds:
        frags = make()
        iters = 20000 if peak_key == "mxfp8" else 40000
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(reps):
            e0.record()
            rc = lib.mx_probe_mfma_rate(fmt, frags.data_ptr(), n_cu, iters, sink.data_ptr(),
                                        torch.cuda.current_stream(dev).cuda_stream)
            if rc != 0:
                raise SystemExit("bench: " + ct._lib.last_error())
            e1.record()
            _sync()
        ms = e0.elapsed_time(e1)
        flop = n_cu * 8 * iters * 32 * 65536.0
        tf = flop / ms * 1e-9
        out.append({"format": peak_key, "data": name, "ms": ms, "tflops": tf, "frac_of_nominal_peak": tf / PEAK_TFLOPS[peak_key]})
    return out


def bench_decode(ct, O, dev, steps, warmup, check, M=32, N=28672, K=8192, nsets=8):
    """Decode-shaped mixed GEMM: X MXFP8 (M, K) x W MXFP4 (N, K)^T, bf16 out; the headline shape is 32 x 28672 x 8192.
    HBM bound; its 121 MiB working set fits in the Infinity Cache, so several weight sets are rotated.  Shapes the
    skinny-M kernel is not chosen for (M > 64) run on what MX_KERNEL_AUTO picks, with the weight scales packed once."""
    x_q, x_s = _quantized(ct, M, K, torch.float8_e4m3fn, 2001, dev, "randn")
    nsets = max(nsets, -(-(300 << 20) // (N * K // 2)))
    ws = []
    for i in range(nsets):
        w_q, w_s = _quantized(ct, N, K, "e2m1", 2002 + i, dev, "randn", std=0.02, cpu_seeded=(i == 0))
        ws.append((w_q, w_s, torch.empty((M, N), dtype=torch.bfloat16, device=dev),
                   w_s.T if M <= 64 else ct.pack_scales(w_s, operand="b")))
    err = None
    if check:
        w_q, w_s, c, w_sc = ws[0]
        ct.block_scaled_matmul(x_q, x_s, w_q.T, w_sc, b_format="e2m1", C=c)
        rows = torch.arange(min(M, 32))
        ref = _oracle_rows(O, x_q, x_s, w_q, w_s, rows, O.E4M3, O.E2M1)
        err = _check_rows(O, c, ref, rows, 8e-3, f"decode {M}x{N}x{K}")

    def step(i):
        w_q, w_s, c, w_sc = ws[i % nsets]
        ct.block_scaled_matmul(x_q, x_s, w_q.T, w_sc, b_format="e2m1", C=c)

    t_wall = _time_wall(step, steps, warmup)
    # The kernel runs ~20 us, less than the host needs to issue a launch from Python, so the kernel's own
    # duration is taken from a captured graph of one launch per weight set, replayed between HIP events.
    # (four passes over the weight sets per graph: the start of a replay, a few microseconds between the first
    # event and the first kernel, is shared by 32 launches)
    per_graph = 4 * nsets
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(per_graph):
            step(i)
    # one sample = one replay (per_graph launches back to back on the stream) between a pair of events, / per_graph
    rb = _events_batch(lambda i: graph.replay())
    w = measure(lambda k: [t / per_graph for t in rb(k)])
    nbytes = M * K + M * K // 32 + N * K // 2 + N * K // 32 + M * N * 2     # 126 885 888 for the headline shape
    return {"ms_per_step": t_wall * 1e3, "kernel": w, "gbs": nbytes / (w.mean * 1e-6) * 1e-9,
            "gbs_wall": nbytes / t_wall * 1e-9, "bytes": nbytes, "rel_fro_vs_oracle": err}


def bench_moe(ct, O, dev, steps, warmup, check, full_forward=True):
    """MoE grouped MXFP8 GEMM: 4096 tokens, hidden 4096, 8 experts x 14336, top-2 (8192 routed rows)."""
    T, K, N, E, topk, tile = 4096, 4096, 14336, 8, 2, 256
    x_q, x_s = _quantized(ct, T, K, torch.float8_e4m3fn, 3001, dev, "randn")
    w_q, w_s = _quantized(ct, E * N, K, torch.float8_e4m3fn, 3002, dev, "randn", std=0.02, cpu_seeded=False)
    W, Ws = w_q.view(E, N, K), w_s.view(E, N, K // 32)
    g = torch.Generator().manual_seed(3003)
    ids = torch.topk(torch.rand((T, E), generator=g), topk, dim=1).indices.to(dev)
    sid, eid = ct.moe_align_tile_size(ids, tile, E)
    C = torch.empty((T, topk, N), dtype=torch.bfloat16, device=dev)
    err = None
    if check:
        ct.invoke_fused_moe_scaled(x_q, x_s, W, Ws, C, None, sid, eid, False, topk, tile)
        # oracle on the rows of 16 tokens, one weight dequantisation per expert
        toks = torch.arange(0, T, T // 16)[:16]
        a = O.dequantize(x_q[toks].view(torch.uint8).cpu().numpy(), x_s[toks].view(torch.uint8).cpu().numpy(), O.E4M3)
        ids_cpu = ids.cpu()
        num = den = 0.0
        for e in sorted(set(ids_cpu[toks].reshape(-1).tolist())):
            w = O.dequantize(W[e].view(torch.uint8).cpu().numpy(), Ws[e].view(torch.uint8).cpu().numpy(), O.E4M3)
            for ti, t in enumerate(toks.tolist()):
                for j in range(topk):
                    if int(ids_cpu[t, j]) != e:
                        continue
                    ref = a[ti] @ w.T
                    got = C[t, j].float().cpu()
                    num += float(((got - ref).double() ** 2).sum())
                    den += float((ref.double() ** 2).sum())
        err = (num / den) ** 0.5
        if not err <= 8e-3:
            raise SystemExit(f"bench: MoE grouped GEMM: relative Frobenius error {err:.3e} exceeds 8e-3")

    def step(i):
        ct.invoke_fused_moe_scaled(x_q, x_s, W, Ws, C, None, sid, eid, False, topk, tile)

    t_step = _time_wall(step, steps, warmup)
    pW = ct.pack_scales(Ws, operand="b")

    def kernel_mostly(i):
        ct.invoke_fused_moe_scaled(x_q, x_s, W, pW, C, None, sid, eid, False, topk, tile)

    # the grouped GEMM kernel with the expert scales pre-packed: the only other kernel between the events is the
    # re-layout of the (gathered) activation scales, 0.5 MiB
    w = measure(_events_batch(kernel_mostly))
    flops = 2.0 * T * topk * K * N
    out = {"ms_per_step": t_step * 1e3, "tflops": flops / t_step * 1e-12, "kernel": w,
           "kernel_tflops": flops / (w.mean * 1e-6) * 1e-12, "rel_fro_vs_oracle": err, "padded_rows": int(sid.numel()),
           "flops": flops}
    if not full_forward:
        return out
    # Informational: the whole block-scaled MoE forward the up-projection belongs to (alignment, gate+up GEMM,
    # SiLU * up with re-quantisation, down GEMM with the routed weights, sum over the top-k copies), N = 2 F.
    F = N // 2
    w2_q, w2_s = _quantized(ct, E * K, F, torch.float8_e4m3fn, 3004, dev, "randn", std=0.02, cpu_seeded=False)
    W2, W2s = w2_q.view(E, K, F), w2_s.view(E, K, F // 32)
    tw = torch.rand((T, topk), generator=g).to(dev)

    def forward(i):
        ct.cutile_moe_scaled(x_q, x_s, W, Ws, W2, W2s, tw, ids, tile)

    t_fwd = _time_events(forward, max(steps // 4, 5), max(warmup // 4, 2))
    out["full_forward_ms"] = t_fwd * 1e3
    out["full_forward_tflops"] = (flops + 2.0 * T * topk * F * K) / t_fwd * 1e-12
    return out


def cpu_baseline_c2(O, sets, budget_s=12.0):
    """The reference's check (dequantize to fp32, torch matmul; samples/BlockScaledMatMul.py:358-364) timed on
    the host cores on the leading m x m x K corner of the headline workload, m sized from a probe so that the
    timed run takes about `budget_s` (the whole workload when the host is fast enough)."""
    a_q, a_s, b_q, b_s, _ = sets[0]
    M, K = a_q.shape
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    torch.set_num_threads(cores)
    a_all, as_all = a_q.view(torch.uint8).cpu().numpy(), a_s.view(torch.uint8).cpu().numpy()
    b_all, bs_all = b_q.view(torch.uint8).cpu().numpy(), b_s.view(torch.uint8).cpu().numpy()

    def run(m):
        t0 = time.perf_counter()
        a = O.dequantize(a_all[:m], as_all[:m], O.E4M3)
        b = O.dequantize(b_all[:m], bs_all[:m], O.E4M3)
        c = a @ b.T
        dt = time.perf_counter() - t0
        return dt, float(c[0, 0])

    run(256)                      # first-touch / thread-pool warm-up
    t_probe, _ = run(1024)
    m = int(1024 * (budget_s / max(t_probe, 1e-4)) ** 0.5) // 64 * 64
    m = max(1024, min(M, m))
    # repeat the sample until about budget_s of CPU work has been timed (the probe overestimates large
    # sizes, where the matmul dominates the dequantisation)
    total, runs = 0.0, 0
    while total < budget_s * 0.8 and runs < 16:
        dt, _ = run(m)
        total += dt
        runs += 1
    tflops = runs * 2.0 * m * m * K / total * 1e-12
    return {"value": tflops, "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"oracle dequantize + fp32 matmul of the leading {m} x {m} x {K} corner of the workload "
                      f"({2.0 * m * m * K * 1e-12:.2f} TFLOP), {runs} runs, {total:.1f} s wall in total"}


def main():
    global SETTLE_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", default="", help="comma list of c2,c3,c4,c5,r4096,shapes (default: all)")
    ap.add_argument("--kernel", default="auto",
                    help="kernel of the square GEMM legs: auto, pingpong, pingpong32, w4p, mfma256, mfma256w4, mfma128 "
                         "(the counter comparisons under profiles/ are runs of this file with this option)")
    ap.add_argument("--no-moe-forward", action="store_true",
                    help="c5: only the up-projection grouped GEMM (a kernel trace of the run then holds one shape of "
                         "the grouped kernel), not the whole MoE forward")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-check", action="store_true", help="skip the correctness check before timing")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_S * 1e3,
                    help="untimed settle period before every timed region (0 for counter-collection runs)")
    ap.add_argument("--no-vendor", action="store_true",
                    help="skip the context leg that times torch._scaled_mm on the headline operands")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy kernel (a known-size reference for "
                         "scaling the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--probe-mfma", action="store_true",
                    help="only run the register-only MFMA rate probe (what the chip sustains on zeros / random / real "
                         "operand bits with nothing but the matrix pipe working) and print its JSON line")
    a = ap.parse_args()
    SETTLE_S = a.settle_ms * 1e-3
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py: this build measures ONE GPU (the path has no cross-GPU exchange; a larger "
                         "job would shard the weights along N and run this same kernel per GPU); run with --gpus 1")
    if not torch.cuda.is_available():
        raise SystemExit("bench.py: no GPU visible")
    import cutile_amd as ct
    from oracle import mx_oracle as O   # checker + cpu_baseline leg only
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if ct.lib().mx_device_check() != 0:
        raise SystemExit("bench.py: " + ct._lib.last_error())
    if a.probe_mfma:
        print(json.dumps({"probe": "mx_probe_mfma_rate: v_mfma_scale_f32_16x16x128_f8f6f4 out of registers, 8 waves per CU",
                          "results": probe_mfma(ct, dev)}))
        return
    if a.calib_copy:
        src = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)          # 256 MiB read + 256 MiB written by one elementwise copy kernel
        _sync()
        del src, dst
    want = set(filter(None, a.only.split(","))) or {"c2", "c3", "c4", "c5", "r4096", "shapes"}
    check = not a.no_check
    kname = {"auto": "gemm_pp_kernel", "pingpong": "gemm_pp_kernel", "pingpong32": "gemm_pp32_kernel",
             "w4p": "gemm_w4_kernel", "mfma256": "gemm_kernel<256x256,8 waves>", "mfma256w4": "gemm_kernel<256x256,4 waves>",
             "mfma128": "gemm_kernel<128x128>"}.get(a.kernel, a.kernel)
    extra = {}
    if "c4" in want:
        r = bench_gemm(ct, O, dev, 8192, 8192, 8192, O.E2M1, "uniform6", a.steps, a.warmup, check,
                       kernel=a.kernel if a.kernel != "pingpong32" and a.kernel != "w4p" else "auto")
        extra["c4_mxfp4_8192"] = {"tflops": r["tflops"], "ms_per_step": r["ms_per_step"],
                                  "rel_fro_vs_oracle": r["rel_fro_vs_oracle"],
                                  "roofline": roofline("mfma", r["kernel_tflops"], PEAK_TFLOPS["mxfp4"], "TFLOP/s", "c4",
                                                       "gemm_pp_kernel<Cfg<e2m1,e2m1,256,256,2,4>,bf16>", r["kernel"], r["flops"])}
        del r
        torch.cuda.empty_cache()
    if "r4096" in want:
        extra["recorded_problem_mxfp8_4096_swizzled_fp32"] = bench_recorded_4096(ct, O, dev, a.steps, a.warmup, check)
        torch.cuda.empty_cache()
    if "shapes" in want:
        # the reference benchmark's other two problems (test/bench_matmul.py:419-425) and two mid-size points: one
        # with few tiles and a long K, one with 400 tiles of 256 x 256 (1.56 rounds of the 256 CUs)
        for name, (M, N, K) in (("ref_bench_1024", (1024, 1024, 1024)),
                                ("ref_bench_12288x4096x2560", (12288, 4096, 2560)),
                                ("mid_2048x2048x8192", (2048, 2048, 8192)),
                                ("mid_5120", (5120, 5120, 5120))):
            extra[name] = bench_shape(ct, O, dev, M, N, K, check)
            torch.cuda.empty_cache()
    if "c3" in want:
        r = bench_decode(ct, O, dev, max(a.steps, 50), a.warmup, check)
        extra["c3_decode_m32"] = {"gbs_wall_clock": r["gbs_wall"], "ms_per_step": r["ms_per_step"],
                                  "rel_fro_vs_oracle": r["rel_fro_vs_oracle"],
                                  "roofline": roofline("hbm", r["gbs"], PEAK_HBM_GBS, "GB/s", "c3",
                                                       "decode_kernel<e4m3,16,bf16>", r["kernel"], r["bytes"])}
        torch.cuda.empty_cache()
        # beyond the headline shape: K longer than one launch of the skinny-M kernel takes (the down-projection
        # of the MoE layer of the grouped workload), and 32 < M <= 128 on the same weights (tiled kernels)
        for name, (M, N, K) in (("decode_m32_k14336", (32, 4096, 14336)), ("decode_m64", (64, 28672, 8192)),
                                ("decode_m128", (128, 28672, 8192))):
            r = bench_decode(ct, O, dev, 50, a.warmup, check, M=M, N=N, K=K)
            extra[name] = {"M": M, "N": N, "K": K, "rel_fro_vs_oracle": r["rel_fro_vs_oracle"],
                           "call_us": r["kernel"].mean, "gbs": r["gbs"], "frac_of_hbm_peak": r["gbs"] / PEAK_HBM_GBS,
                           "bytes_per_launch": r["bytes"], **r["kernel"].stats()}
            del r
            torch.cuda.empty_cache()
    if "c5" in want:
        r = bench_moe(ct, O, dev, a.steps, a.warmup, check, full_forward=not a.no_moe_forward)
        e5 = {"tflops": r["tflops"], "ms_per_step": r["ms_per_step"], "padded_rows": r["padded_rows"],
              "rel_fro_vs_oracle": r["rel_fro_vs_oracle"],
              "roofline": roofline("mfma", r["kernel_tflops"], PEAK_TFLOPS["mxfp8"], "TFLOP/s", "c5",
                                   "gemm_pp_kernel<Cfg<e4m3,e4m3,256,256,2,4>,bf16,grouped>", r["kernel"], r["flops"])}
        if "full_forward_ms" in r:
            e5["full_forward_ms"], e5["full_forward_tflops"] = r["full_forward_ms"], r["full_forward_tflops"]
        extra["c5_moe_grouped_mxfp8"] = e5
        torch.cuda.empty_cache()
    out = {"metric": METRIC, "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "mxfp8_e4m3 (e8m0 scales, fp32 accumulate, bf16 out)",
           "data": "synthetic", "settle_ms": SETTLE_S * 1e3, "extra": extra}
    if "c2" in want:
        r = bench_gemm(ct, O, dev, 8192, 8192, 8192, O.E4M3, "randn", a.steps, a.warmup, check, kernel=a.kernel)
        out.update({
            "value": r["tflops"], "ms_per_step": r["ms_per_step"],
            "config": {"workload": "MXFP8 E4M3 x E4M3 block-scaled GEMM, M=N=K=8192, E8M0 scale per 32 along K "
                                   "(floor rule), A row-major MxK, B column-major KxN, fp32 accumulate, bf16 output; "
                                   "one step = one block_scaled_matmul call incl. scale re-layout",
                       "M": 8192, "N": 8192, "K": 8192, "operand_sets_rotated": 3, "kernel": a.kernel},
            "rel_fro_vs_oracle": r["rel_fro_vs_oracle"],
            "roofline": roofline("mfma", r["kernel_tflops"], PEAK_TFLOPS["mxfp8"], "TFLOP/s",
                                 "c2" if a.kernel in ("auto", "pingpong") else "c2_" + a.kernel,
                                 f"{kname}<e4m3,e4m3,256x256,bf16>", r["kernel"], r["flops"]),
        })
        if not a.no_vendor:
            extra["context_torch_scaled_mm_mxfp8_8192"] = vendor_scaled_mm(r["sets"], a.steps, a.warmup)
        if not a.no_cpu:
            out["cpu_baseline"] = cpu_baseline_c2(O, r["sets"])
    else:
        out.update({"value": None, "ms_per_step": None, "config": {"workload": "partial run: " + ",".join(sorted(want))}})
    print(json.dumps(out))


if __name__ == "__main__":
    main()
