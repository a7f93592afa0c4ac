#!/usr/bin/env python3
"""Benchmark of the packed-int4 linear-layer GEMM on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-decode] [--no-extra] [--no-vendor]
                    [--no-ceiling] [--calibrate-copy]

A step is one GEMM launch C[MxN] = A[MxK] * B[NxK]^T through the library's C ABI
(int4linear_gemm_s4s4s32, asynchronous, on torch's current stream).  The workload is
the square M = N = K = 8192 case the headline metric is quoted on; inputs are synthetic
seeded s4 values already resident in HBM when the clock starts.  Operand sets rotate
through more memory than L2 plus the 256 MB Infinity Cache, so no launch finds its
operands cached by the previous one (the reference flushes L2 before every timed launch,
test/benchmark.cu:77-96).  Throughput = 2*M*N*K / time (test/benchmark.cu:112-115).

One JSON line is printed.  Besides the whole-run figure it carries
  roofline      the dominant kernel's own rate (HIP events around launches of the GEMM
                kernel alone, on the launch stream) against the dense peak of the MFMA
                type it issues,
  decode        the skinny-M weight-streaming kernel at M = 16 against HBM bandwidth,
  cpu_baseline  the CPU oracle's loop nest timed on this host's cores on a row sample,
  static_weights  the same problem with W converted once beforehand, as a linear layer with static
                weights would run it (per step: convert X, then the GEMM on converted operands),
  int8_kernel   the same 8192^3 problem on the library's int8-MFMA kernel (the path that
                needs no workspace), against the int8 MFMA dense peak,
  vendor        hipBLASLt's int8 GEMM on the widened operands, timed by the C++ harness
                tests/host/vendor_compare (which also checks both results agree bit for bit).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

INT8_MFMA_PEAK_TOPS = 5000.0   # MI355X dense int8, published
FP6_MFMA_PEAK_TOPS = 10100.0   # MI355X dense fp6/fp4, published
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published

M = N = K = 8192
DECODE_SHAPES = [(16, 4096, 4096), (16, 14336, 4096), (16, 4096, 14336)]
DECODE_OTHER_M = [(m, n, k) for m in (1, 64) for (n, k) in ((4096, 4096), (14336, 4096), (4096, 14336))]
# Weight matrices large enough that the per-kernel launch floor (2.5-2.8 us on this device) stops
# mattering: the MLP up-projection and the vocabulary projection of a model with hidden size 8192.
DECODE_LARGE_W = [(16, 28672, 8192), (16, 128256, 8192)]


def packed_random(torch, rows: int, k: int, seed: int):
    """rows x k/2 bytes of uniform s4 pairs: every byte value 0..255 equally likely is
    exactly two independent uniform nibbles in [-8, 7]."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randint(0, 256, (rows, k // 2), dtype=torch.uint8, device="cuda", generator=g)


def packed_normal(torch, rows: int, k: int, seed: int, sigma: float = 2.0):
    """rows x k/2 bytes of decode-style activations: normal(0, sigma) rounded to nearest and
    clamped to [-8, 7], packed on the device in the packer's byte layout (element e of a row in
    byte e/2, even e in the low nibble: utils/packer.cpp:3-18)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    v = torch.randn((rows, k), device="cuda", generator=g).mul_(sigma).round_().clamp_(-8, 7).to(torch.int16)
    nib = (v & 0xF).to(torch.uint8)
    return (nib[:, 0::2] | (nib[:, 1::2] << 4)).contiguous()


RAMP_MS = 60.0   # untimed load before the first timed leg, see ramp_clocks


def ramp_clocks(torch, launch, sets, min_ms: float = RAMP_MS):
    """Runs the workload untimed for min_ms.  After an idle period this device needs some
    tens of milliseconds of load before it runs at its sustained speed (the first ~60 calls
    of the 8192^3 GEMM take 360-400 us, later ones 315-330 us); a short warm-up of a few
    steps would time that ramp instead of the kernel."""
    t0 = time.perf_counter()
    i = 0
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        for _ in range(10):
            launch(sets[i % len(sets)])
            i += 1
        torch.cuda.synchronize()
    return i


def time_launches(torch, launch, sets, steps: int, warmup: int):
    """Average milliseconds per launch: `warmup` untimed, then exactly `steps` timed
    launches bracketed by a device synchronisation and a HIP event pair on the stream.
    `launch` is either a Python callable taking one argument set, or a (C function, name)
    pair: then the timed loop is nothing but the calls themselves (a few microseconds of
    host work per launch matter next to a 5 microsecond kernel) and the returned status
    codes are checked after the loop."""
    if isinstance(launch, tuple):
        fn, name = launch
        order = [sets[i % len(sets)] for i in range(max(steps, warmup))]
        bad = 0
        for t in order[:warmup]:
            bad |= fn(*t)
        torch.cuda.synchronize()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        timed = order[:steps]
        t0 = time.perf_counter()
        start.record()
        for t in timed:
            bad |= fn(*t)
        stop.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        if bad != 0:
            raise RuntimeError(f"{name} failed (status bits {bad})")
        return start.elapsed_time(stop) / steps, wall_ms / steps
    for i in range(warmup):
        launch(sets[i % len(sets)])
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        launch(sets[i % len(sets)])
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def raw_entry(name: str):
    """The C-ABI function itself (ctypes), so the timed loops carry no wrapper overhead."""
    from int4linear_amd import _lib

    return getattr(_lib.load(), name)


def bench_gemm(torch, lib, steps: int, warmup: int):
    """The drop-in call (packed s4 in, int32 out) and, separately, its dominant kernel."""
    import ctypes

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # 3 operand sets x (32 + 32 + 256 MiB) = 960 MiB > L2 + Infinity Cache.
    sets = []
    for s in range(3):
        a = packed_random(torch, M, K, 1000 + s)
        b = packed_random(torch, N, K, 2000 + s)
        c = torch.empty((M, N), dtype=torch.int32, device="cuda")
        sets.append((a, b, c))
    gemm = raw_entry("int4linear_gemm_s4s4s32")
    args = [(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, stream) for (a, b, c) in sets]

    def launch(t):
        st = gemm(*t)
        if st != 0:
            raise RuntimeError(f"int4linear_gemm_s4s4s32 failed with status {st}")

    ramp_clocks(torch, launch, args)
    ev_ms, wall_ms = time_launches(torch, launch, args, steps, warmup)
    # The reference's own statistic (test/benchmark.cu:93-111): an event pair around every
    # launch, median over the launches (here without a flush in between: the rotation keeps
    # the operands cold).
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for i, (e0, e1) in enumerate(pairs):
        e0.record()
        launch(args[i % len(args)])
        e1.record()
    torch.cuda.synchronize()
    per_launch = sorted(e0.elapsed_time(e1) for (e0, e1) in pairs)
    median_ms = per_launch[len(per_launch) // 2]

    # The dominant kernel's own duration inside the same sequence of kernels as the timed
    # region: each step converts both operands into caller-owned buffers (what the call above
    # does into the library's workspace) and then runs the FP6 GEMM between a pair of HIP
    # events on the stream it is launched on.  (Timed in a loop of nothing but GEMMs on
    # operands converted beforehand the kernel runs 8-10 % slower: rotating operand sets then
    # come from HBM instead of the memory-side cache the converter has just left them in, and
    # without the memory-bound converter between two GEMMs the power limit holds the clock lower.)
    kernel = lib.kernel_for_shape(M, N, K)
    kern_ms = ev_ms
    if kernel == "fp6":
        conv = []
        for (a, b, c) in sets:
            ac = torch.empty(lib.fp6_operand_bytes(M, K), dtype=torch.uint8, device="cuda")
            bc = torch.empty(lib.fp6_operand_bytes(N, K), dtype=torch.uint8, device="cuda")
            conv.append((a, b, ac, bc, c))
        convert = raw_entry("int4linear_fp6_convert")
        gemm6 = raw_entry("int4linear_gemm_fp6_converted")
        steps6 = [conv[i % len(conv)] for i in range(warmup + steps)]
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in steps6]
        bad = 0
        for (a, b, ac, bc, c), (e0, e1) in zip(steps6, events):
            bad |= convert(a.data_ptr(), ac.data_ptr(), M, K, stream)
            bad |= convert(b.data_ptr(), bc.data_ptr(), N, K, stream)
            e0.record()
            bad |= gemm6(ac.data_ptr(), bc.data_ptr(), c.data_ptr(), M, N, K, stream)
            e1.record()
        torch.cuda.synchronize()
        if bad != 0:
            raise RuntimeError(f"the caller-owned FP6 entry points failed (status bits {bad})")
        kern_ms = sum(e0.elapsed_time(e1) for (e0, e1) in events[warmup:]) / steps
    return ev_ms, wall_ms, kernel, kern_ms, median_ms


def bench_decode(torch, lib, steps: int, warmup: int, shapes=None, activations: str = "normal", runs: int = 3):
    """Per-launch time of back-to-back launches over rotating weights.  `activations`: "normal"
    (clamp(round(N(0, 2))), the decode configuration) or "uniform"; `runs`: how many runs of
    (warm-up, 300 timed launches), the median one being the figure."""
    import ctypes

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gemm = raw_entry("int4linear_gemm_s4s4s32")
    out = []
    for (m, n, k) in (shapes or DECODE_SHAPES):
        wbytes = n * k // 2
        nsets = max(4 if wbytes < (256 << 20) else 2, (768 << 20) // wbytes + 1)   # rotate through > 768 MiB of weights
        # activations: clamp(round(normal(0, 2))) unless asked otherwise; weights uniform
        x = packed_normal(torch, m, k, 31) if activations == "normal" else packed_random(torch, m, k, 31)
        sets = [(x, packed_random(torch, n, k, 40 + i), torch.empty((m, n), dtype=torch.int32, device="cuda"))
                for i in range(nsets)]
        args = [(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, n, k, stream) for (a, b, c) in sets]

        # runs of (warm-up, 300 timed launches); the median run is the figure, all are listed
        times = sorted(time_launches(torch, (gemm, "int4linear_gemm_s4s4s32"), args, max(steps, 300), max(warmup, 20))[0]
                       for _ in range(runs))
        ev_ms = times[len(times) // 2]
        algo_bytes = m * k // 2 + n * k // 2 + 4 * m * n
        gbs = algo_bytes / (ev_ms * 1e-3) / 1e9
        out.append({"shape": [m, n, k], "kernel": lib.kernel_for_shape(m, n, k), "us_per_launch": ev_ms * 1e3,
                    "us_per_launch_runs": [round(r * 1e3, 3) for r in times],
                    "bytes": algo_bytes, "GB/s": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS})
        del sets
        torch.cuda.empty_cache()
    return out


def stream_ceilings(shapes):
    """Per-launch time of a bare streaming kernel (same read pattern as the decode kernel, no
    arithmetic, 4*M*N bytes written) for each shape, from tests/host/bin/stream_ceiling: what
    the device gives a kernel that only streams, launch cost included.  {} when the harness
    is not built."""
    import re
    import subprocess

    exe = ROOT / "tests" / "host" / "bin" / "stream_ceiling"
    if not exe.exists():
        return {}
    try:
        r = subprocess.run([str(exe)] + [f"{m}x{n}x{k}" for (m, n, k) in shapes], capture_output=True, text=True, timeout=180)
    except (OSError, subprocess.TimeoutExpired):
        return {}
    out = {}
    for mm in re.finditer(r"\[CEILING\] (\d+)x(\d+)x(\d+) ([\d.]+) us ([\d.]+) GB/s", r.stdout):
        out[(int(mm.group(1)), int(mm.group(2)), int(mm.group(3)))] = (float(mm.group(4)), float(mm.group(5)))
    return out


def add_ceilings(entries, ceilings):
    for d in entries:
        c = ceilings.get(tuple(d["shape"]))
        if c:
            d["bare_stream_us_per_launch"] = c[0]
            d["bare_stream_GB/s"] = c[1]
            d["frac_of_bare_stream"] = c[0] / d["us_per_launch"]


def bench_int8_kernel(torch, lib, steps: int, warmup: int):
    """8192^3 on the int8 MFMA kernel (kernel id 2), same rotation and timing as the headline."""
    import ctypes

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sets = []
    for s in range(3):
        sets.append((packed_random(torch, M, K, 1000 + s), packed_random(torch, N, K, 2000 + s),
                     torch.empty((M, N), dtype=torch.int32, device="cuda")))
    fn = raw_entry("int4linear_gemm_s4s4s32_ex")
    args = [(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, 2, stream) for (a, b, c) in sets]

    def launch(t):
        st = fn(*t)
        if st != 0:
            raise RuntimeError(f"int4linear_gemm_s4s4s32_ex failed with status {st}")

    ramp_clocks(torch, launch, args)   # the legs before this one leave the device in a low clock state
    ev_ms, _ = time_launches(torch, launch, args, steps, warmup)
    tops = 2.0 * M * N * K / (ev_ms * 1e-3) / 1e12
    return {"kernel": "mfma_gemm_kernel (v_mfma_i32_32x32x32_i8)", "kernel_ms": ev_ms, "TOPS": tops,
            "frac_of_int8_peak": tops / INT8_MFMA_PEAK_TOPS}


def bench_static_weights(torch, lib, steps: int, warmup: int):
    """The 8192^3 problem the way a linear layer with static weights would run it: W converted
    once before the timed region (int4linear_fp6_convert), every step converts the activations
    X and multiplies (int4linear_gemm_fp6_converted).  Reported beside `value`, never as it:
    `value` converts both operands in every call, as the reference's entry point implies."""
    import ctypes

    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    convert = raw_entry("int4linear_fp6_convert")
    gemm6 = raw_entry("int4linear_gemm_fp6_converted")
    sets = []
    for s in range(3):
        a = packed_random(torch, M, K, 3000 + s)
        b = packed_random(torch, N, K, 4000 + s)
        ac = torch.empty(lib.fp6_operand_bytes(M, K), dtype=torch.uint8, device="cuda")
        bc = torch.empty(lib.fp6_operand_bytes(N, K), dtype=torch.uint8, device="cuda")
        c = torch.empty((M, N), dtype=torch.int32, device="cuda")
        if convert(b.data_ptr(), bc.data_ptr(), N, K, stream) != 0:
            raise RuntimeError("int4linear_fp6_convert failed")
        sets.append((a, ac, bc, c))
        del b
    torch.cuda.synchronize()

    def launch(t):
        a, ac, bc, c = t
        st = convert(a.data_ptr(), ac.data_ptr(), M, K, stream)
        st |= gemm6(ac.data_ptr(), bc.data_ptr(), c.data_ptr(), M, N, K, stream)
        if st != 0:
            raise RuntimeError(f"the caller-owned FP6 entry points failed (status bits {st})")

    ramp_clocks(torch, launch, sets)
    ev_ms, _ = time_launches(torch, launch, sets, steps, warmup)
    return {"what": "W converted once beforehand (int4linear_fp6_convert), per step: convert X, int4linear_gemm_fp6_converted",
            "ms_per_step": ev_ms, "TOPS": 2.0 * M * N * K / (ev_ms * 1e-3) / 1e12,
            "note": "three sets of operands rotate, so the converted W comes from HBM in every step; the per-call "
                    "converter of the default path leaves it in the memory-side cache instead, which at this size is "
                    "worth about what the conversion costs"}


def vendor_line():
    """hipBLASLt int8 at 8192^3 through the C++ harness; None when the harness is not built."""
    import re
    import subprocess

    exe = ROOT / "tests" / "host" / "bin" / "vendor_compare"
    if not exe.exists():
        return None
    try:
        r = subprocess.run([str(exe), "--iters", "20", f"{M}x{N}x{K}"], capture_output=True, text=True, timeout=120)
    except (OSError, subprocess.TimeoutExpired):
        return None
    m = re.search(r"hipBLASLt int8 ([\d.]+) ms ([\d.]+) TOPS \| int4linear \((\w+)\) ([\d.]+) ms ([\d.]+) TOPS \| "
                  r"ratio ([\d.]+)x \| results (\w+)", r.stdout)
    if not m:
        return None
    return {"library": "hipBLASLt int8 x int8 -> int32 on operands widened beforehand", "ms": float(m.group(1)),
            "TOPS": float(m.group(2)), "int4linear_ms_same_protocol": float(m.group(4)),
            "int4linear_TOPS_same_protocol": float(m.group(5)), "speedup": float(m.group(6)),
            "results": m.group(7), "protocol": "per-launch events, 512 MiB cache-cleaning fill before each, median of 20"}


def cpu_baseline(budget_s: float = 15.0):
    """The oracle's loop nest (oracle_linear_ref_mt) on a row sample of the 8192^3
    problem, all host threads the box grants us."""
    from oracle import loader as oracle

    threads = max(1, min(16, os.cpu_count() or 1))
    rng = np.random.default_rng(7)
    w = rng.integers(-8, 8, size=(N, K), dtype=np.int8).astype(np.int32)
    # calibrate on one row per thread, then size the sample to the budget
    rows = threads
    x = rng.integers(-8, 8, size=(rows, K), dtype=np.int8).astype(np.int32)
    t0 = time.perf_counter()
    oracle.linear_ref(x, w, threads=threads)
    dt = time.perf_counter() - t0
    rows = int(max(threads, min(M, (budget_s / max(dt, 1e-3)) * rows)) // threads * threads)
    x = rng.integers(-8, 8, size=(rows, K), dtype=np.int8).astype(np.int32)
    t0 = time.perf_counter()
    oracle.linear_ref(x, w, threads=threads)
    dt = time.perf_counter() - t0
    tops = 2.0 * rows * N * K / dt / 1e12
    # the reference's own single-threaded loop nest on a smaller sample, for the per-core figure
    rows1 = max(1, rows // (threads * 4))
    t0 = time.perf_counter()
    oracle.linear_ref(x[:rows1], w, threads=1)
    dt1 = time.perf_counter() - t0
    return {"value": tops, "unit": "TOPS", "cores": threads, "kind": "port",
            "sample": f"{rows} of {M} rows of the 8192^3 problem (all {N} columns, full K), "
                      f"{dt:.1f} s, oracle_linear_ref_mt with {threads} threads",
            "single_thread_TOPS": 2.0 * rows1 * N * K / dt1 / 1e12,
            "single_thread_sample": f"{rows1} rows, {dt1:.1f} s, oracle_linear_ref"}


TRAFFIC_PROFILE = ROOT / "profiles" / "fp6_gemm_8192_and_decode_hbm_traffic.md"
KERNEL_SOURCE = {"fp6": ROOT / "int4linear_amd" / "csrc" / "kernels_fp6.hip"}


def source_digest(path: Path) -> str:
    import hashlib

    return hashlib.sha256(path.read_bytes()).hexdigest()


def measured_traffic(kernel: str):
    """(HBM bytes per launch of the GEMM kernel, where the figure comes from).  The figure was
    recorded from rocprofv3 counter runs (FETCH_SIZE and WRITE_SIZE, each scaled by a plain
    copy of known size) together with a digest of the kernel's source file; it is reported only
    while that file is still the one that was measured, otherwise None."""
    if not TRAFFIC_PROFILE.exists() or kernel not in KERNEL_SOURCE:
        return None, "no counter run on record for this kernel"
    value = digest = None
    for line in TRAFFIC_PROFILE.read_text().splitlines():
        if line.startswith(f"bytes_per_launch {kernel}_gemm_8192:"):
            try:
                value = int(line.split(":")[1])
            except ValueError:
                value = None
        if line.startswith(f"source_sha256 {KERNEL_SOURCE[kernel].name}:"):
            digest = line.split(":")[1].strip()
    where = f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs recorded in profiles/{TRAFFIC_PROFILE.name}"
    if value is None:
        return None, "no figure in " + where
    if digest != source_digest(KERNEL_SOURCE[kernel]):
        return None, (f"{KERNEL_SOURCE[kernel].name} has changed since the {where}: "
                      "the recorded figure is withheld until the counters are read again")
    return value, "static: " + where + " for this very source file, not measured by this run"


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode-shape leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the int8-kernel, large-W decode and vendor legs")
    ap.add_argument("--no-vendor", action="store_true", help="skip the vendor-library leg (a child process)")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the bare-stream ceiling leg (a child process)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run four plain 1 GiB device copies first (a kernel of known traffic "
                         "to scale hardware byte counters by when profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only; run with --gpus 1 "
              "(the path would shard over the rows of W with no exchange step)", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no HIP device visible", file=sys.stderr)
        return 1
    import int4linear_amd as lib

    lib.init()
    torch.cuda.set_device(0)

    if args.calibrate_copy:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    ev_ms, wall_ms, kernel, kern_ms, median_ms = bench_gemm(torch, lib, args.steps, args.warmup)
    ops = 2.0 * M * N * K
    tops_kernel = ops / (kern_ms * 1e-3) / 1e12
    tops_wall = ops / (wall_ms * 1e-3) / 1e12
    # The roofline that bounds the dominant kernel is that of the MFMA type it issues.
    peak = FP6_MFMA_PEAK_TOPS if kernel == "fp6" else INT8_MFMA_PEAK_TOPS
    kernel_name = {"fp6": "fp6_gemm_kernel (v_mfma_f32_32x32x64_f8f6f4, E2M3 operands)",
                   "mfma": "mfma_gemm_kernel (v_mfma_i32_32x32x32_i8)"}.get(kernel, kernel)

    traffic, traffic_source = measured_traffic(kernel)
    result = {
        "metric": "INT4 GEMM TOPS at M=N=K=8192 (% int8 MFMA peak); GB/s at M=16 decode",
        "value": tops_wall,
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "median_ms": median_ms,
        "median_TOPS": 2.0 * M * N * K / (median_ms * 1e-3) / 1e12,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp6" if kernel == "fp6" else "int8",
        "dtype_note": ("s4 operands re-encoded exactly as FP6 E2M3, fp32 accumulation of integers below 2^24: "
                       "bit-identical to int32 arithmetic.  pct_of_int8_mfma_peak divides this throughput by the "
                       "int8 MFMA peak the metric names although the kernel issues FP6 MFMAs (peak 10.1 PFLOP/s): "
                       "a ratio across units; roofline.frac is the one against the issued instruction's own peak")
        if kernel == "fp6" else "s4 widened to int8, int32 accumulation",
        "data": "synthetic",
        "config": {"workload": "M=N=K=8192 s4*s4->s32 GEMM, uniform [-8,7], 3 rotating operand sets",
                   "untimed_clock_ramp_ms": RAMP_MS,
                   "kernel": kernel, "M": M, "N": N, "K": K},
        "pct_of_int8_mfma_peak": 100.0 * tops_wall / INT8_MFMA_PEAK_TOPS,
        "roofline": {"bound": "mfma", "achieved": tops_kernel, "peak": peak,
                     "unit": "TFLOP/s", "frac": tops_kernel / peak,
                     "traffic": traffic,
                     "traffic_source": traffic_source,
                     "kernel": kernel_name,
                     "note": "2*M*N*K multiply-adds per launch / mean duration of the GEMM kernel itself: a HIP "
                             "event pair around each of its launches on caller-owned converted operands, in the "
                             "same converter-then-GEMM sequence as the timed region",
                     "kernel_ms": kern_ms, "whole_call_ms": ev_ms,
                     "frac_of_int8_peak": tops_kernel / INT8_MFMA_PEAK_TOPS},
    }
    if not args.no_decode:
        dec = bench_decode(torch, lib, args.steps, args.warmup)
        result["decode"] = dec
        result["decode_GB/s_M16"] = sum(d["GB/s"] for d in dec) / len(dec)
        result["decode_GB/s_M16_min"] = min(d["GB/s"] for d in dec)
        result["decode_M16_shapes"] = [d["shape"] for d in dec]
        result["decode_note"] = ("mean time per launch of 300 back-to-back launches over rotating weights (> 768 MiB), median of three such runs; "
                                 "bare_stream_*: a kernel that only streams the same bytes in the same pattern, "
                                 "launched the same way (tests/host/stream_ceiling.cpp)")
        # The statistic of this benchmark's first version, kept so that figures stay comparable
        # across versions of the kernels: uniform activations, one run, the mean over the two
        # large M = 16 shapes.
        first = bench_decode(torch, lib, args.steps, args.warmup, DECODE_SHAPES[1:], activations="uniform", runs=1)
        result["decode_GB/s_M16_uniform_activations_two_large_shapes"] = sum(d["GB/s"] for d in first) / len(first)
        result["decode_other_M"] = bench_decode(torch, lib, args.steps, args.warmup, DECODE_OTHER_M)
        if not args.no_extra:
            result["decode_large_W"] = bench_decode(torch, lib, args.steps, args.warmup, DECODE_LARGE_W)
        torch.cuda.synchronize()
        all_dec = result["decode"] + result["decode_other_M"] + result.get("decode_large_W", [])
        if not args.no_ceiling:
            add_ceilings(all_dec, stream_ceilings([tuple(d["shape"]) for d in all_dec]))
    if not args.no_extra:
        if kernel == "fp6":
            result["static_weights"] = bench_static_weights(torch, lib, max(10, args.steps // 2), args.warmup)
        result["int8_kernel"] = bench_int8_kernel(torch, lib, max(10, args.steps // 2), args.warmup)
        if not args.no_vendor:
            result["vendor"] = vendor_line()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
