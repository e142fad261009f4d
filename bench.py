#!/usr/bin/env python3
"""Benchmark of the GEMM + broadcast hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-others] [--no-cpu]

Prints ONE JSON line. The headline workload is the float32 GEMM C = A*B at M = N = K = 4096
(row-major, A and B iid uniform[-1, 1) from fixed seeds, resident in HBM before the timed
region). A step is one launch of the GEMM. `value` is TFLOP/s over the K timed steps, wall clock
bracketed by stream synchronisation; `roofline` prices the same kernel against the MFMA fp32
peak using HIP events recorded on the library's stream; `cpu_baseline` times the CPU restatement
of the reference's laser gemm_strided (oracle/, OpenMP, all host cores) on the same workload.
`others` carries the remaining configurations of the path (int32 4096^3, the float64 strided
config, the 8192^2 broadcast ops), each with its own bound.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

# The CPU legs use OpenMP: their worker threads should sleep, not spin, once a parallel region is
# over, or they compete with the thread that launches the GPU kernels timed right afterwards.
os.environ.setdefault("OMP_WAIT_POLICY", "passive")

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_F32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix peak: 256 CU x 256 FLOP/clk x 2.4 GHz
MFMA_F64_PEAK_TFLOPS = 78.6
HBM_PEAK_GBS = 8000.0
MFMA_I8_PEAK_TOPS = 5000.0     # MI355X dense int8 matrix peak (5.0 POP/s)
# Measured separately with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), see profiles/; None = not measured.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def device_info(L):
    name = ctypes.create_string_buffer(128)
    cus, khz, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    hbm = ctypes.c_size_t()
    L.am_hip_device_info(name, 128, ctypes.byref(cus), ctypes.byref(khz), ctypes.byref(hbm), ctypes.byref(lds))
    return dict(name=name.value.decode(), compute_units=cus.value, clock_mhz=khz.value / 1000.0,
                hbm_gib=round(hbm.value / 2**30, 1))


class Timer:
    """HIP events on the library stream + host wall clock around a synchronised region."""

    def __init__(self, am, L):
        self.am, self.L = am, L
        self.e0, self.e1 = ctypes.c_void_p(), ctypes.c_void_p()
        L.am_hip_event_create(ctypes.byref(self.e0))
        L.am_hip_event_create(ctypes.byref(self.e1))

    def run(self, fn, steps, warmup, min_warm_s=0.0):
        """Times `steps` calls of fn after `warmup` untimed ones. While the timed steps run, the matrix-core
        GEMM kernels count shader cycles against the constant-rate counter (am_hip_diag_clock_*):
        self.sclk_mhz is the shader clock they sustained (None when no such kernel ran).
        min_warm_s: go on warming up until the untimed calls have kept the device busy for that long. The
        shader clock needs 20-50 ms under load to climb from about 2.1 GHz to the 2.39 GHz it then holds (and as
        long to recover after a power-limited kernel); a figure taken inside that ramp is 10 % low."""
        self.L.am_hip_event_record(self.e0)
        for _ in range(warmup):
            fn()
        self.L.am_hip_event_record(self.e1)
        self.am.sync()
        if min_warm_s > 0 and warmup > 0:
            ms = ctypes.c_float()
            self.L.am_hip_event_elapsed_ms(self.e0, self.e1, ctypes.byref(ms))
            per_call = max(ms.value / 1e3 / warmup, 1e-6)
            for _ in range(min(int((min_warm_s - ms.value / 1e3) / per_call) + 1, 20000) if ms.value / 1e3 < min_warm_s else 0):
                fn()
            self.am.sync()
        armed = self.L.am_hip_diag_clock_begin() == 0
        t0 = time.perf_counter()
        self.L.am_hip_event_record(self.e0)
        for _ in range(steps):
            fn()
        self.L.am_hip_event_record(self.e1)
        self.am.sync()
        wall = time.perf_counter() - t0
        ms = ctypes.c_float()
        self.L.am_hip_event_elapsed_ms(self.e0, self.e1, ctypes.byref(ms))
        self.sclk_mhz = None
        if armed:
            mhz = ctypes.c_double()
            if self.L.am_hip_diag_clock_end(ctypes.byref(mhz)) == 0 and mhz.value > 0:
                self.sclk_mhz = round(mhz.value, 0)
        return wall, ms.value / 1e3     # seconds: wall clock for all steps, event time for all steps


ROTATE = 5   # buffer sets of the rotating protocol: together far beyond the 256 MB memory-side cache


WARM_S = 0.05   # device-busy time before every timed region of the secondary workloads (see Timer.run)


def run_rotating(timer, fns, rounds, warm_rounds=1):
    """The same operation on len(fns) disjoint buffer sets, issued round robin, so that no byte of an
    input is still in the memory-side cache when it is read again: every byte comes from HBM.
    Returns seconds per launch (HIP events)."""
    state = {"i": 0}

    def step():
        fns[state["i"] % len(fns)]()
        state["i"] += 1
    _, ev = timer.run(step, rounds * len(fns), warm_rounds * len(fns), WARM_S)
    return ev / (rounds * len(fns))


def measured_ceilings(L):
    """Issue ceilings of this chip from register-only micro-benchmarks (no memory traffic): what a
    perfect kernel could reach at the clocks the device sustains, T(FL)OP/s; and what HBM delivers to
    kernels that only stream (read, write, copy of 256 MiB per launch over six rotating buffers = 1.5 GiB
    per direction, so every byte comes from HBM; 16-byte non-temporal accesses, four in flight per lane;
    the best of a few grid sizes), TB/s."""
    out = {}
    for kind, name, iters in [(0, "mfma_f32", 20000), (1, "mfma_f64", 20000), (2, "valu_int32_mac", 20000), (3, "valu_int64_mac", 5000),
                              (4, "mfma_i8", 20000)]:
        v = ctypes.c_double()
        if L.am_hip_diag_peak(kind, iters, 2, ctypes.byref(v)) == 0:
            out[name] = round(v.value / 1e12, 2)
    for kind, name in [(0, "hbm_read"), (1, "hbm_write"), (2, "hbm_copy")]:
        best = 0.0
        for blocks_per_cu in (2, 8, 32):
            for flags in ((1,) if kind == 0 else (2, 0) if kind == 1 else (3,)):
                v = ctypes.c_double()
                if L.am_hip_diag_hbm(kind, 256 << 20, 6, blocks_per_cu, 4, flags, 24, ctypes.byref(v)) == 0:
                    best = max(best, v.value)
        if best:
            out[name + "_tbs"] = round(best / 1e12, 3)
    return out


def load_traffic(key):
    """(bytes per launch from the committed rocprofv3 --pmc passes, where those were taken) - the figure is not
    re-measured by this run: counters need the profiler."""
    try:
        with open(TRAFFIC_FILE) as f:
            d = json.load(f)
        return d.get(key), d.get("_source")
    except (OSError, ValueError):
        return None, None


def at_clock(roof, peak, sclk_mhz, nominal_mhz=2400.0):
    """Adds the sustained shader clock and the fraction of the peak scaled to that clock (the published
    matrix peaks are CUs x ops per clock x 2.4 GHz)."""
    if sclk_mhz:
        roof["sclk_mhz"] = sclk_mhz
        roof["frac_of_peak_at_sclk"] = round(roof["achieved"] / (peak * sclk_mhz / nominal_mhz), 4)
    return roof


def spin_up(L, seconds=0.08):
    """Keeps the matrix cores busy for `seconds` with the register-only MFMA chain (no memory traffic, not
    the workload): the shader clock climbs from the 2.1 GHz of an idle device to the 2.39 GHz it holds under
    sustained load."""
    t_end = time.perf_counter() + seconds
    v = ctypes.c_double()
    while time.perf_counter() < t_end:
        L.am_hip_diag_peak(0, 20000, 2, ctypes.byref(v))


def bench_gemm_f32(am, timer, steps, warmup, n=4096, host=None, device_warm_s=0.0):
    A, B = host or (np.random.default_rng(1001).uniform(-1, 1, (n, n)).astype(np.float32),
                    np.random.default_rng(1002).uniform(-1, 1, (n, n)).astype(np.float32))
    dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), np.float32)
    if device_warm_s > 0:
        spin_up(timer.L, device_warm_s)
    wall, ev = timer.run(lambda: am.gemm(1.0, dA, dB, 0.0, dC), steps, warmup)
    flops = 2.0 * n ** 3
    return dict(wall=wall, ev=ev, flops=flops, host=(A, B), sclk_mhz=timer.sclk_mhz)


def cpu_baseline_gemm_f32(A, B, budget_s=12.0):
    """Times the oracle's blocked gemm_strided (the port of the reference's CPU algorithm) on the
    full 4096^3 workload: one untimed run, then as many timed runs as fit the budget (>= 1)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import am_oracle
    n = A.shape[0]
    C = np.empty((n, n), dtype=np.float32)
    am_oracle.gemm_strided(1.0, A, B, 0.0, C)
    times = []
    t_end = time.perf_counter() + budget_s
    while not times or (time.perf_counter() < t_end and len(times) < 20):
        t0 = time.perf_counter()
        am_oracle.gemm_strided(1.0, A, B, 0.0, C)
        times.append(time.perf_counter() - t0)
    best = min(times)
    return dict(value=round(2.0 * n ** 3 / best / 1e12, 4), unit="TFLOP/s", cores=am_oracle.num_threads(),
                kind="port",
                sample=f"full workload (f32 GEMM {n}^3), best of {len(times)} runs after 1 warm-up, "
                       f"oracle/laser_gemm.c (laser blocking, 6x16 AVX2+FMA register tile, OpenMP)")


def digit_pairs(A, B):
    """How many of the digit-pair products (i + j < number of bytes: ten for int32, 36 for int64) the
    digit-sliced integer GEMM runs for these operands: a balanced base-256 digit plane that is zero
    everywhere is skipped."""
    nd = A.dtype.itemsize
    mask = np.uint64(0x8080808080808080 >> (8 * (8 - nd)))
    def planes(X):   # digit d of x is byte d of (x + 0x80..80) ^ 0x80..80, modulo 2^(8 nd)
        y = X.astype(np.int64).view(np.uint64)
        y = (y + mask) ^ mask
        return [bool(((y >> np.uint64(8 * d)) & np.uint64(0xFF)).any()) for d in range(nd)]
    fa, fb = planes(A), planes(B)
    return sum(1 for i in range(nd) for j in range(nd - i) if fa[i] and fb[j])


def bench_gemm_f64_views(am, timer, steps, warmup):
    """float64 gemm(1.5, A^T view, B[:, ::2] view, 0.5, C), M=2048 N=3072 K=1024. Measured before the
    register-only int8 matrix-core chains of `measured_ceilings`: those leave the chip at a lowered
    clock for longer than a warm-up lasts."""
    pa = np.random.default_rng(3001).standard_normal((1024, 2048))
    pb = np.random.default_rng(3002).standard_normal((1024, 6144))
    C = np.random.default_rng(3003).standard_normal((2048, 3072))
    dA, dB, dC = am.toHip(pa).transpose(), am.toHip(pb)[:, ::2], am.toHip(C)
    # (0.3 s of warm-up: after the idle gap of the uploads the clock takes longer to climb under float64 matrix
    # instructions than under float32 ones - 60 ms in, the same kernel still reads 2.2 GHz and 8 % more time)
    wall, ev = timer.run(lambda: am.gemm(1.5, dA, dB, 0.5, dC), steps, warmup, 0.3)
    fl = 2.0 * 2048 * 3072 * 1024
    return dict(workload="f64 gemm(1.5, A^T view, B[:, ::2] view, 0.5, C) 2048x3072x1024", unit="TFLOP/s",
                dtype="f64", value=round(fl * steps / wall / 1e12, 3), ms_per_step=round(ev / steps * 1e3, 4),
                roofline=at_clock(dict(bound="mfma", achieved=round(fl / (ev / steps) / 1e12, 3), peak=MFMA_F64_PEAK_TFLOPS,
                                       unit="TFLOP/s", frac=round(fl / (ev / steps) / 1e12 / MFMA_F64_PEAK_TFLOPS, 4)),
                                  MFMA_F64_PEAK_TFLOPS, timer.sclk_mhz))


def other_workloads(am, timer, steps, warmup, ceilings, first=()):
    out = list(first)
    # --- int32 GEMM 4096^3, wraparound accumulate: digit-sliced on the int8 matrix cores (the
    # library's choice at this size) with the VALU kernel beside it. Entries in [-100, 100] fit one
    # base-256 digit, so one of the ten digit-pair products runs; entries over the whole int32 range
    # need all ten.
    n = 4096
    k = max(3, steps // 4)       # launches of the VALU kernels (2.5 - 8 ms each)
    kd = max(20, steps)          # launches of the digit-sliced products (0.1 - 0.7 ms each)
    peak = ceilings.get("valu_int32_mac")
    for label, lo, hi in (("entries in [-100, 100]", -100, 100), ("entries over the whole int32 range", -2 ** 31, 2 ** 31 - 1)):
        A = np.random.default_rng(2001).integers(lo, hi, (n, n), endpoint=True).astype(np.int32)
        B = np.random.default_rng(2002).integers(lo, hi, (n, n), endpoint=True).astype(np.int32)
        pairs = digit_pairs(A, B)
        dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), np.int32)
        wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), kd, 2, WARM_S)
        sclk = timer.sclk_mhz
        tops = 2.0 * n ** 3 / (ev / kd) / 1e12
        entry = dict(workload=f"i32 GEMM 4096^3, {label} (wraparound; {pairs} of 10 int8 digit-pair products on the matrix cores, "
                              "timed with the two digit-splitting passes)",
                     unit="Top/s", dtype="i32", value=round(2.0 * n ** 3 * kd / wall / 1e12, 3), ms_per_step=round(ev / kd * 1e3, 4),
                     roofline=at_clock(dict(bound="mfma", achieved=round(pairs * tops, 1), peak=MFMA_I8_PEAK_TOPS,
                                            unit=f"int8 TOP/s executed ({pairs} digit pairs x 2*M*N*K) over the whole call, two digit-splitting passes included",
                                            frac=round(pairs * tops / MFMA_I8_PEAK_TOPS, 4)), MFMA_I8_PEAK_TOPS, sclk),
                     speedup_over_valu_ceiling=round(tops / peak, 2) if peak else None)
        if lo == -100:
            os.environ["AM_HIP_GEMM_I32_PATH"] = "valu"
            try:
                _, ev_valu = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), k, 2, WARM_S)
            finally:
                del os.environ["AM_HIP_GEMM_I32_PATH"]
            valu_tops = 2.0 * n ** 3 / (ev_valu / k) / 1e12
            entry["valu_kernel"] = dict(value=round(valu_tops, 3), unit="Top/s", ms_per_step=round(ev_valu / k * 1e3, 4),
                                        roofline=dict(bound="valu (measured int32 multiply-add ceiling; no matrix instruction for int32)",
                                                      achieved=round(valu_tops, 3), peak=peak, unit="Top/s",
                                                      frac=round(valu_tops / peak, 4) if peak else None))
        out.append(entry)
        del dA, dB, dC
    # --- int64 GEMM 4096^3, entries in [-100, 100]: eight digits, 36 pairs at most, one of them here
    A = np.random.default_rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(np.int64)
    B = np.random.default_rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(np.int64)
    dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), np.int64)
    wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), kd, 2, WARM_S)
    sclk = timer.sclk_mhz
    os.environ["AM_HIP_GEMM_I64_PATH"] = "valu"
    try:
        _, ev_valu = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), 3, 1, WARM_S)
    finally:
        del os.environ["AM_HIP_GEMM_I64_PATH"]
    peak64 = ceilings.get("valu_int64_mac")
    valu_tops = 2.0 * n ** 3 / (ev_valu / 3) / 1e12
    out.append(dict(workload="i64 GEMM 4096^3, entries in [-100, 100] (wraparound; 1 of 36 int8 digit-pair products on the matrix cores, "
                             "timed with the two digit-splitting passes)",
                    unit="Top/s", dtype="i64", value=round(2.0 * n ** 3 * kd / wall / 1e12, 3), ms_per_step=round(ev / kd * 1e3, 4),
                    roofline=at_clock(dict(bound="mfma", achieved=round(2.0 * n ** 3 / (ev / kd) / 1e12, 1), peak=MFMA_I8_PEAK_TOPS,
                                           unit="int8 TOP/s executed (1 digit pair x 2*M*N*K) over the whole call, two digit-splitting passes included",
                                           frac=round(2.0 * n ** 3 / (ev / kd) / 1e12 / MFMA_I8_PEAK_TOPS, 4)), MFMA_I8_PEAK_TOPS, sclk),
                    valu_kernel=dict(value=round(valu_tops, 3), unit="Top/s", ms_per_step=round(ev_valu / 3 * 1e3, 4),
                                     roofline=dict(bound="valu (measured int64 multiply-add ceiling)", achieved=round(valu_tops, 3),
                                                   peak=peak64, unit="Top/s", frac=round(valu_tops / peak64, 4) if peak64 else None))))
    del dA, dB, dC
    # --- the one figure the reference publishes for this path: `a * b` of two 1500 x 1500 int64 tensors with
    # entries in [0, 99] (benchmarks/integer_matmul.nim:8-33: 0.14 s on an 18-core i9-9980XE, a whole process
    # with the random fill, so the ratio is an upper bound on the kernel-to-kernel one)
    n5 = 1500
    A = np.random.default_rng(2003).integers(0, 99, (n5, n5), endpoint=True).astype(np.int64)
    B = np.random.default_rng(2004).integers(0, 99, (n5, n5), endpoint=True).astype(np.int64)
    dA, dB = am.toHip(A), am.toHip(B)
    dC = dA * dB
    wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), max(steps, 50), warmup, WARM_S)
    k5 = max(steps, 50)
    want = A[n5 // 2] @ B          # one row of the product (the benchmark prints one element of it)
    out.append(dict(workload="i64 matmul 1500x1500, entries in [0, 99] (the reference's published integer benchmark: 1 of 36 int8 digit-pair "
                             "products on the matrix cores, timed with the two digit-splitting passes)",
                    unit="Top/s", dtype="i64", value=round(2.0 * n5 ** 3 * k5 / wall / 1e12, 3), ms_per_step=round(ev / k5 * 1e3, 4),
                    row_750_matches_numpy=bool(np.array_equal(dC.toCpu()[n5 // 2], want)),
                    published=dict(seconds=0.14, gops=round(2.0 * n5 ** 3 / 0.14 / 1e9, 1), hardware="i9-9980XE, 18 cores, -d:danger -d:openmp",
                                   source="benchmarks/integer_matmul.nim:8-33 (wall time of the whole process: random fill, product, one element printed)",
                                   ratio_to_this_kernel_time=round(0.14 / (ev / k5), 0))))
    del dA, dB, dC
    # --- broadcast ops on X[8192, 8192] f32 (HBM bound): 536 903 680 algorithmic bytes per op
    X = np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
    b = np.random.default_rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32)
    s = np.random.default_rng(4003).uniform(-1, 1, (8192, 1)).astype(np.float32)
    db, ds = am.toHip(b), am.toHip(s)
    dXs = [am.toHip(X) for _ in range(ROTATE)]
    dYs = [am.empty((8192, 8192), np.float32) for _ in range(ROTATE)]
    dX, dY = dXs[0], dYs[0]
    from arraymancer_amd import tensor_hip as th
    bb = db.broadcast((8192, 8192))
    sb = ds.broadcast((8192, 8192))
    nbytes = 2 * 8192 * 8192 * 4 + 8192 * 4
    # Five buffer sets round robin (2.5 GiB), so that every byte of every launch comes from HBM: both `value`
    # and `roofline` are that figure. The same-buffer time is listed beside it (part of a 256 MiB input that is
    # read again at once can still be in the 256 MB memory-side cache).
    copy_ceiling = ceilings.get("hbm_copy_tbs")
    for name, op, rhs in [("X +. b[1,8192]", "add", bb), ("Y *. s[8192,1]", "mul", sb),
                          ("map2(X, b, max(0, x+y)) (fused bias+ReLU)", "add_relu", bb)]:
        _, ev = timer.run(lambda: th._binary_into(op, dY, dX, rhs), steps, warmup, WARM_S)
        rounds = max(steps // ROTATE, 4)
        t0 = time.perf_counter()
        cold = run_rotating(timer, [(lambda i=i: th._binary_into(op, dYs[i], dXs[i], rhs)) for i in range(ROTATE)], rounds)
        gbs = nbytes / cold / 1e9
        roof = dict(bound="hbm", achieved=round(gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(gbs / HBM_PEAK_GBS, 4),
                    ms_per_launch=round(cold * 1e3, 4), protocol=f"{ROTATE} buffer sets round robin (2.5 GiB): every byte from HBM")
        if copy_ceiling:
            roof["measured_copy_ceiling_gbs"] = round(copy_ceiling * 1e3, 1)
            roof["frac_of_measured_copy_ceiling"] = round(gbs / (copy_ceiling * 1e3), 4)
        out.append(dict(workload=f"f32 8192x8192 {name}", unit="GB/s", dtype="f32", value=round(gbs, 1), ms_per_step=round(cold * 1e3, 4),
                        same_buffers_every_step_ms=round(ev / steps * 1e3, 4), roofline=roof))
    # --- the same kinds of pass on operands that are not square row-major matrices: a transposed operand, and the
    # [batch x features] shapes of a dense layer (bias add, bias gradient, row sums, weight gradient). Three buffer
    # sets round robin for the HBM-bound ones (0.4 - 0.8 GiB per set).
    def hbm_entry(workload, launches, nbytes):
        cold = run_rotating(timer, launches, max(steps // len(launches), 4))
        gbs = nbytes / cold / 1e9
        out.append(dict(workload=workload, unit="GB/s", dtype="f32", value=round(gbs, 1), ms_per_step=round(cold * 1e3, 4),
                        roofline=dict(bound="hbm", achieved=round(gbs, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(gbs / HBM_PEAK_GBS, 4),
                                      protocol=f"{len(launches)} buffer sets round robin: every byte from HBM")))
    hbm_entry("f32 8192x8192 X + Z^T (Z a transposed view)",
              [(lambda i=i: th._binary_into("add", dYs[i], dXs[i], dXs[(i + 1) % 3].transpose())) for i in range(3)], 3 * 8192 * 8192 * 4)
    del dXs, dYs
    T = np.random.default_rng(4004).uniform(-1, 1, (65536, 512)).astype(np.float32)
    dTs = [am.toHip(T) for _ in range(3)]
    dOs = [am.empty((65536, 512), np.float32) for _ in range(3)]
    bias = am.toHip(np.random.default_rng(4005).uniform(-1, 1, (1, 512)).astype(np.float32)).broadcast((65536, 512))
    hbm_entry("f32 65536x512 X +. b[1,512] (bias of a dense layer)", [(lambda i=i: th._binary_into("add", dOs[i], dTs[i], bias)) for i in range(3)],
              2 * T.nbytes + 2048)
    col_sums, row_sums = am.empty((1, 512), np.float32), am.empty((65536, 1), np.float32)
    hbm_entry("f32 sum(X[65536,512], axis=0) (bias gradient)", [(lambda i=i: th.reduce_axis_into("sum", col_sums, dTs[i], 0)) for i in range(3)], T.nbytes)
    hbm_entry("f32 sum(X[65536,512], axis=1)", [(lambda i=i: th.reduce_axis_into("sum", row_sums, dTs[i], 1)) for i in range(3)], T.nbytes)
    del dTs, dOs
    dA = am.toHip(np.random.default_rng(1003).standard_normal((500, 65536)).astype(np.float32))
    dB = am.toHip(np.random.default_rng(1004).standard_normal((65536, 800)).astype(np.float32))
    dC = am.empty((500, 800), np.float32)
    wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), max(steps, 20), warmup, WARM_S)
    fl = 2.0 * 500 * 800 * 65536
    k = max(steps, 20)
    out.append(dict(workload="f32 GEMM [500x65536].[65536x800] (weight gradient of a dense layer over a large batch: few tiles, long k)",
                    unit="TFLOP/s", dtype="f32", value=round(fl * k / wall / 1e12, 3), ms_per_step=round(ev / k * 1e3, 4),
                    roofline=at_clock(dict(bound="mfma", achieved=round(fl / (ev / k) / 1e12, 3), peak=MFMA_F32_PEAK_TFLOPS, unit="TFLOP/s",
                                           frac=round(fl / (ev / k) / 1e12 / MFMA_F32_PEAK_TFLOPS, 4)), MFMA_F32_PEAK_TFLOPS, timer.sclk_mhz)))
    del dA, dB, dC
    out.append(bench_chain(am, timer, max(steps, 50), warmup))
    out.append(bench_ex02(am, timer, max(steps, 50), warmup))
    out.extend(bench_conv_backward(am, timer, steps, warmup))
    out.append(bench_ex02_train(am, timer, max(steps, 20), warmup))
    return out


def chain_setup(am):
    """The MNIST-shaped inference chain (batch 64): conv1 and conv2 as im2col
    GEMMs, dense + bias + ReLU (fused epilogue), classifier. All outputs are allocated up front so
    that the four launches can be recorded into a HIP graph. Returns (issue, flops, bytes)."""
    rng = np.random.default_rng(5001)
    g = lambda *sh: am.toHip(rng.normal(0, 0.1, sh).astype(np.float32))
    k1, x1, o1 = g(20, 25), g(25, 36864), am.empty((20, 36864), np.float32)
    k2, x2, o2 = g(50, 500), g(500, 4096), am.empty((50, 4096), np.float32)
    x3, w3, b3, h = g(64, 800), g(500, 800), g(1, 500), am.empty((64, 500), np.float32)
    w4, o4 = g(10, 500), am.empty((64, 10), np.float32)
    w3t, w4t = w3.transpose(), w4.transpose()

    def issue():
        am.gemm(1.0, k1, x1, 0.0, o1)
        am.gemm(1.0, k2, x2, 0.0, o2)
        am.gemm(1.0, x3, w3t, 0.0, h, epilogue="bias_relu", bias=b3)
        am.gemm(1.0, h, w4t, 0.0, o4)

    flops = 2.0 * (20 * 25 * 36864 + 50 * 500 * 4096 + 64 * 800 * 500 + 64 * 500 * 10)
    return issue, flops, 17834080, (k1, x1, o1, k2, x2, o2, x3, w3, b3, h, w4, o4)


def bench_chain(am, timer, steps, warmup):
    issue, flops, nbytes, keep = chain_setup(am)
    wall_e, ev_e = timer.run(issue, steps, warmup, WARM_S)    # eager: 4 launches per chain from the host
    with am.Graph() as graph:
        issue()
    wall_g, ev_g = timer.run(graph.launch, steps, warmup, WARM_S)     # one graph launch per chain
    return dict(workload="f32 inference chain: [20x25].[25x36864], [50x500].[500x4096], "
                         "[64x800].[800x500]+bias+ReLU (fused), [64x500].[500x10]",
                unit="us per chain", dtype="f32", higher_is_better=False,
                value=round(min(ev_g, ev_e) / steps * 1e6, 2), value_is="eager" if ev_e <= ev_g else "hipgraph",
                hipgraph_us=round(ev_g / steps * 1e6, 2),
                eager_us=round(ev_e / steps * 1e6, 2), eager_wall_us=round(wall_e / steps * 1e6, 2),
                gflops=round(flops / (min(ev_g, ev_e) / steps) / 1e9, 1),
                note="kernel-time bound: 2.9e8 FLOP and 17.8 MB per chain in four kernels of 5-10 us whose durations sum to the eager "
                     "figure; a graph replay adds about 3 us per launch of the graph on this runtime and removes about 1 us of "
                     "host gap per kernel, so it pays from about six kernels per graph (the eight-launch forward pass below), "
                     "not on these four")


def bench_ex02(am, timer, steps, warmup, batch=64):
    """The whole forward pass of the reference's example 2 (conv - ReLU - maxpool twice, two dense layers) at batch 64:
    six launches per pass issued from the host (each convolution is one launch: the column matrix is gathered by the
    GEMM's loader), and the same six replayed from one HIP graph."""
    from arraymancer_amd import ex02
    rng = np.random.default_rng(5002)
    net = ex02.DemoNet(batch, ex02.random_params(rng), np.float32)
    dx = am.toHip(rng.uniform(0, 1, (batch, 1, 28, 28)).astype(np.float32))
    wall_e, ev_e = timer.run(lambda: net.forward(dx), steps, warmup, WARM_S)
    graph = net.capture(dx)
    wall_g, ev_g = timer.run(graph.launch, steps, warmup, WARM_S)
    flops = 2.0 * batch * (20 * 25 * 576 + 50 * 500 * 64 + 800 * 500 + 500 * 10)
    best = min(ev_e, ev_g)
    return dict(workload=f"f32 example-2 forward pass, batch {batch}: conv(1->20,5x5)+ReLU, maxpool 2x2, conv(20->50,5x5)+ReLU, "
                         "maxpool 2x2, flatten, linear(800->500)+ReLU, linear(500->10); 6 launches",
                unit="us per pass", dtype="f32", higher_is_better=False, value=round(best / steps * 1e6, 2),
                value_is="eager" if ev_e <= ev_g else "hipgraph", eager_us=round(ev_e / steps * 1e6, 2),
                eager_wall_us=round(wall_e / steps * 1e6, 2), hipgraph_us=round(ev_g / steps * 1e6, 2),
                images_per_s=round(batch / (best / steps), 0), gflops=round(flops / (best / steps) / 1e9, 1),
                note="3.0e8 FLOP per pass over six kernels of 3-15 us each: the graph replay runs them back to back (its time is "
                     "the sum of their durations), the eager pass adds the host's launch gap after each")


def bench_ex02_train(am, timer, steps, warmup, batch=64):
    """One step of example 2's learning loop at batch 64: forward, sparse softmax cross-entropy (read back to the
    host), the backward primitives, the SGD update of the eight parameters."""
    from arraymancer_amd import ex02
    rng = np.random.default_rng(5003)
    net = ex02.DemoNet(batch, ex02.random_params(rng), np.float32)
    dx = am.toHip(rng.uniform(0, 1, (batch, 1, 28, 28)).astype(np.float32))
    dl = am.toHip(rng.integers(0, 10, batch).astype(np.int64))
    wall, ev = timer.run(lambda: net.train_step(dx, dl, 0.01), steps, warmup, WARM_S)
    graph = net.capture_train_step(dx, dl, 0.01)
    wall_g, ev_g = timer.run(graph.launch, steps, warmup, WARM_S)
    flops = 3 * 2.0 * batch * (20 * 25 * 576 + 50 * 500 * 64 + 800 * 500 + 500 * 10)
    best = min(ev, ev_g)
    return dict(workload=f"f32 example-2 training step, batch {batch}: forward, sparse softmax cross-entropy, backward through "
                         "linear / ReLU / maxpool / conv2d, SGD update of 8 parameters",
                unit="us per step", dtype="f32", higher_is_better=False, value=round(best / steps * 1e6, 2),
                value_is="eager" if ev <= ev_g else "hipgraph", eager_us=round(ev / steps * 1e6, 2),
                eager_wall_us=round(wall / steps * 1e6, 2), hipgraph_us=round(ev_g / steps * 1e6, 2),
                images_per_s=round(batch / (best / steps), 0), gflops=round(flops / (best / steps) / 1e9, 1),
                note="eager: about forty short launches issued one by one from the host, the loss read back every step: bound "
                     "by the host's launch rate. hipgraph: the same step without the read-back recorded once with its "
                     "temporaries (a rehearsal leaves the allocator one cached block per allocation, the capture is served "
                     "from that cache) and replayed with one launch per step")


def bench_conv_backward(am, timer, steps, warmup, first_only=False):
    """conv2d_backward (grad_input, grad_weight, grad_bias) on a ResNet-like layer and on the second convolution of
    the reference's example 2. FLOP counted: twice the forward pass (one product for each of the two gradients)."""
    out = []
    for name, (N, C, H, W, co, k, pad) in (("[64,64,56,56], 64 kernels 3x3, pad 1", (64, 64, 56, 56, 64, 3, 1)),
                                           ("[64,20,12,12], 50 kernels 5x5 (example 2, conv2)", (64, 20, 12, 12, 50, 5, 0)))[:1 if first_only else 2]:
        rng = np.random.default_rng(6001)
        ho = H + 2 * pad - k + 1
        x = am.toHip(rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32))
        w = am.toHip(rng.uniform(-1, 1, (co, C, k, k)).astype(np.float32))
        b = am.toHip(rng.uniform(-1, 1, (co, 1, 1)).astype(np.float32))
        g = am.toHip(rng.uniform(-1, 1, (N, co, ho, ho)).astype(np.float32))
        _, ev_f = timer.run(lambda: am.conv2d(x, w, b, (pad, pad), (1, 1)), steps, warmup, WARM_S)
        _, ev_b = timer.run(lambda: am.conv2d_backward(x, w, b, (pad, pad), (1, 1), g), steps, warmup, WARM_S)
        fl = 2.0 * N * co * ho * ho * C * k * k
        out.append(dict(workload=f"f32 conv2d_backward {name}", unit="TFLOP/s", dtype="f32", value=round(2 * fl / (ev_b / steps) / 1e12, 2),
                        ms_per_step=round(ev_b / steps * 1e3, 4), forward_ms=round(ev_f / steps * 1e3, 4),
                        forward_tflops=round(fl / (ev_f / steps) / 1e12, 2),
                        roofline=dict(bound="mfma", achieved=round(2 * fl / (ev_b / steps) / 1e12, 2), peak=MFMA_F32_PEAK_TFLOPS, unit="TFLOP/s",
                                      frac=round(2 * fl / (ev_b / steps) / 1e12 / MFMA_F32_PEAK_TFLOPS, 4)),
                        note="five launches and a small copy: grad_output with its first two axes swapped, its row sums (grad_bias), "
                             "the column matrices of the batch side by side, grad_weight as one product over k = N*H_out*W_out, "
                             "grad_input as one convolution of grad_output with the turned kernel"))
    return out


def config_report(am, timer, L):
    """One JSON line per configuration of the path: GPU time / rate / fraction of its bound, the CPU
    port (oracle, all host cores) timed beside it on the same inputs, and the parity result of the
    GPU output against the CPU output at full size. Not the default mode (the default prints one
    line); run as `python bench.py --report`."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import am_oracle
    from arraymancer_amd import tensor_hip as th
    ceil = measured_ceilings(L)
    threads = am_oracle.num_threads()

    def cpu_time(fn, budget=4.0, max_runs=5):
        fn()
        ts = []
        end = time.perf_counter() + budget
        while not ts or (time.perf_counter() < end and len(ts) < max_runs):
            t0 = time.perf_counter(); fn(); ts.append(time.perf_counter() - t0)
        return min(ts)

    def emit(**kw):
        print(json.dumps(kw), flush=True)

    def gemm_case(config, sfx, M, N, K, A, B, dA, dB, alpha=1, beta=0, C0=None, peak=None, peak_used="", unit="TFLOP/s", steps=20):
        dt = A.dtype
        C_host = C0.copy() if C0 is not None else np.zeros((M, N), dt)
        dC = am.toHip(C_host)
        am.gemm(alpha, dA, dB, beta, dC)
        got = dC.toCpu().copy()
        # (with beta != 0 the timed calls go on accumulating into C: only their time is used)
        _, ev = timer.run(lambda: am.gemm(alpha, dA, dB, beta, dC), steps, 3, WARM_S)
        gpu_s = ev / steps
        want = am_oracle.gemm_strided(alpha, A, B, beta, C_host.copy())
        cpu_s = cpu_time(lambda: am_oracle.gemm_strided(alpha, A, B, beta, C_host.copy() if beta != 0 else C_host))
        ops = 2.0 * M * N * K
        row = dict(config=config, dtype=sfx, shape=[M, N, K], gpu_ms=round(gpu_s * 1e3, 4),
                   gpu_rate=round(ops / gpu_s / 1e12, 3), rate_unit=unit,
                   pct_peak=round(100 * ops / gpu_s / 1e12 / peak, 1) if peak else None, peak_used=peak_used,
                   cpu_impl="oracle/laser_gemm.c (port of laser gemm_strided, OpenMP)", cpu_threads=threads,
                   cpu_ms=round(cpu_s * 1e3, 2), speedup_vs_cpu=round(cpu_s / gpu_s, 1), sclk_mhz=timer.sclk_mhz)
        if dt.kind == "f":
            row["rel_frobenius_vs_cpu"] = am_oracle.rel_frobenius(got, want)
            # the reference's float `*` goes through CBLAS: NumPy's bundled BLAS as the stand-in for it
            # (a copy of each view first, as the reference makes: p_operator_blas_l2l3.nim:151-152)
            blas_s = cpu_time(lambda: alpha * (np.ascontiguousarray(A) @ np.ascontiguousarray(B)) + beta * C_host)
            row["cpu_blas_impl"] = "NumPy bundled BLAS, alpha * (A @ B) + beta * C on contiguous copies (stand-in for the reference's CBLAS path)"
            row["cpu_blas_ms"] = round(blas_s * 1e3, 2)
        else:
            row["bit_exact"] = bool(np.array_equal(got, want))
        emit(**row)

    rng = np.random.default_rng
    for n in (1024, 2048, 4096):
        A = rng(1001).uniform(-1, 1, (n, n)).astype(np.float32); B = rng(1002).uniform(-1, 1, (n, n)).astype(np.float32)
        gemm_case(f"f32 GEMM {n}^3", "f32", n, n, n, A, B, am.toHip(A), am.toHip(B), peak=MFMA_F32_PEAK_TFLOPS,
                  peak_used="MFMA fp32 157.3 TFLOP/s", steps=200 if n <= 2048 else 20)
    # extents that are not a multiple of the 16-byte vector, beside their aligned neighbour (4096): unit-stride
    # operands are moved in 16-byte pieces whatever their pitch; 4097 runs as the 4096^3 block plus two skinny strips
    for n in (4095, 4097):
        A = rng(1001).uniform(-1, 1, (n, n)).astype(np.float32); B = rng(1002).uniform(-1, 1, (n, n)).astype(np.float32)
        gemm_case(f"f32 GEMM {n}^3 (ragged extents)", "f32", n, n, n, A, B, am.toHip(A), am.toHip(B), peak=MFMA_F32_PEAK_TFLOPS,
                  peak_used="MFMA fp32 157.3 TFLOP/s", steps=20)
    for sfx, dt, key in (("i32", np.int32, "valu_int32_mac"), ("i64", np.int64, "valu_int64_mac")):
        for n in (1500, 1501, 4096) if sfx == "i32" else (1500, 4096):
            A = rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(dt)
            B = rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(dt)
            env = f"AM_HIP_GEMM_{sfx.upper()}_PATH"
            # the library's own choice (digit slicing on the int8 matrix cores at these sizes), then the VALU kernel
            pairs = digit_pairs(A, B)
            gemm_case(f"{sfx} GEMM {n}^3, entries in [-100, 100] (library's choice: digit-sliced int8 MFMA, {pairs} digit pair)", sfx, n, n, n,
                      A, B, am.toHip(A), am.toHip(B), peak=MFMA_I8_PEAK_TOPS / pairs,
                      peak_used=f"int8 MFMA 5000 TOP/s / {pairs} digit-pair product(s) executed; whole call incl. the two digit-splitting passes",
                      unit="Top/s", steps=20)
            os.environ[env] = "valu"
            try:
                gemm_case(f"{sfx} GEMM {n}^3, entries in [-100, 100] (VALU kernel)", sfx, n, n, n, A, B,
                          am.toHip(A), am.toHip(B), peak=ceil.get(key),
                          peak_used=f"measured VALU {sfx} multiply-add ceiling {ceil.get(key)} Top/s", unit="Top/s", steps=10)
            finally:
                os.environ.pop(env, None)
    n = 4096
    for sfx, dt, key in (("i32", np.int32, "valu_int32_mac"), ("i64", np.int64, "valu_int64_mac")):
        info = np.iinfo(dt)
        A = rng(2001).integers(info.min, info.max, (n, n), endpoint=True).astype(dt)
        B = rng(2002).integers(info.min, info.max, (n, n), endpoint=True).astype(dt)
        pairs = digit_pairs(A, B)
        gemm_case(f"{sfx} GEMM {n}^3, entries over the whole {sfx} range (library's choice: digit-sliced int8 MFMA, all {pairs} digit pairs)",
                  sfx, n, n, n, A, B, am.toHip(A), am.toHip(B), peak=MFMA_I8_PEAK_TOPS / pairs,
                  peak_used=f"int8 MFMA 5000 TOP/s / {pairs} digit-pair products executed; whole call incl. the two digit-splitting passes",
                  unit="Top/s", steps=10)
    pa = rng(3001).standard_normal((1024, 2048)); pb = rng(3002).standard_normal((1024, 6144))
    C0 = rng(3003).standard_normal((2048, 3072))
    gemm_case("f64 gemm(1.5, A^T view, B[:, ::2] view, 0.5, C)", "f64", 2048, 3072, 1024, pa.T, pb[:, ::2],
              am.toHip(pa).transpose(), am.toHip(pb)[:, ::2], alpha=1.5, beta=0.5, C0=C0, peak=MFMA_F64_PEAK_TFLOPS,
              peak_used="MFMA fp64 78.6 TFLOP/s", steps=1)
    # broadcast ops
    X = rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
    b = rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32); sc = rng(4003).uniform(-1, 1, (8192, 1)).astype(np.float32)
    db, ds = am.toHip(b), am.toHip(sc)
    dXs = [am.toHip(X) for _ in range(ROTATE)]
    dYs = [am.empty((8192, 8192), np.float32) for _ in range(ROTATE)]
    dX, dY = dXs[0], dYs[0]
    nbytes = 2 * 8192 * 8192 * 4 + 8192 * 4

    def warm_note(ev_s, nb):
        return (f"with the same buffers every launch the input is re-read from the 256 MB memory-side cache: "
                f"{ev_s * 1e3:.4f} ms = {nb / ev_s / 1e9:.0f} GB/s")
    # HBM-bound rows: timed over five buffer sets round robin, so that every byte comes from HBM
    for name, op, dv, hv in (("X +. b[1,8192]", "add", db, b), ("X *. s[8192,1]", "mul", ds, sc), ("map2(X, b, max(0, x+y))", "add_relu", db, b)):
        bv = dv.broadcast((8192, 8192))
        _, ev = timer.run(lambda: th._binary_into(op, dY, dX, bv), 50, 5, WARM_S)
        gpu_s = run_rotating(timer, [(lambda i=i: th._binary_into(op, dYs[i], dXs[i], bv)) for i in range(ROTATE)], 10)
        got = dYs[ROTATE - 1].toCpu().copy()
        hb = am_oracle.broadcast(hv, X.shape)
        out = np.empty_like(X)
        cpu_s = cpu_time(lambda: am_oracle.map2(op, X, hb, out=out))
        emit(config=f"f32 8192x8192 {name}", dtype="f32", shape=[8192, 8192], gpu_ms=round(gpu_s * 1e3, 4),
             gpu_rate=round(nbytes / gpu_s / 1e9, 1), rate_unit="GB/s", pct_peak=round(100 * nbytes / gpu_s / 1e9 / HBM_PEAK_GBS, 1),
             peak_used="HBM 8000 GB/s", cpu_impl="oracle/strided_map.c (port of map2_inline + strided iteration, OpenMP blocks)",
             cpu_threads=threads, cpu_ms=round(cpu_s * 1e3, 2), speedup_vs_cpu=round(cpu_s / gpu_s, 1),
             bit_exact=bool(np.array_equal(got, out)), note=warm_note(ev / 50, nbytes))
    # (X +. b) *. s fused into one pass (same bytes moved once instead of twice)
    bb, sb = db.broadcast((8192, 8192)), ds.broadcast((8192, 8192))
    _, ev = timer.run(lambda: th._ternary_into("addmul", dY, dX, bb, sb), 50, 5, WARM_S)
    gpu_s = run_rotating(timer, [(lambda i=i: th._ternary_into("addmul", dYs[i], dXs[i], bb, sb)) for i in range(ROTATE)], 10)
    two_pass = ((X + b) * sc)
    emit(config="f32 8192x8192 (X +. b) *. s fused (one pass)", dtype="f32", shape=[8192, 8192], gpu_ms=round(gpu_s * 1e3, 4),
         gpu_rate=round((nbytes + 8192 * 4) / gpu_s / 1e9, 1), rate_unit="GB/s",
         pct_peak=round(100 * (nbytes + 8192 * 4) / gpu_s / 1e9 / HBM_PEAK_GBS, 1), peak_used="HBM 8000 GB/s",
         bit_exact=bool(np.array_equal(dYs[ROTATE - 1].toCpu(), two_pass)),
         note="equals the two separate broadcast passes bit for bit; " + warm_note(ev / 50, nbytes + 8192 * 4))
    # operands whose unit stride lies on the other axis than the result's (strided iteration, p_accessors.nim:181-208)
    Xt = np.ascontiguousarray(X.T)
    for name, launch, nb, want, cpu_fn in (
            ("clone of a transposed view", lambda i: th._unary_into("copy", dYs[i], dXs[i].transpose()), 2 * X.nbytes, Xt,
             lambda: np.copyto(out, X.T)),
            ("X + X^T (transposed operand)", lambda i: th._binary_into("add", dYs[i], dXs[i], dXs[(i + 1) % ROTATE].transpose()), 3 * X.nbytes,
             X + Xt, lambda: am_oracle.map2("add", X, X.T, out=out))):
        gpu_s = run_rotating(timer, [(lambda i=i: launch(i)) for i in range(ROTATE)], 10)
        cpu_s = cpu_time(cpu_fn, budget=2.0)
        emit(config=f"f32 8192x8192 {name}", dtype="f32", shape=[8192, 8192], gpu_ms=round(gpu_s * 1e3, 4),
             gpu_rate=round(nb / gpu_s / 1e9, 1), rate_unit="GB/s", pct_peak=round(100 * nb / gpu_s / 1e9 / HBM_PEAK_GBS, 1),
             peak_used="HBM 8000 GB/s", cpu_impl="NumPy strided copy" if "clone" in name else "oracle/strided_map.c (strided iteration, OpenMP blocks)",
             cpu_threads=1 if "clone" in name else threads, cpu_ms=round(cpu_s * 1e3, 2), speedup_vs_cpu=round(cpu_s / gpu_s, 1),
             bit_exact=bool(np.array_equal(dYs[ROTATE - 1].toCpu(), want)),
             note="16-byte-vector tiled kernel: both operands read and the result written along their own unit-stride axis")
    del dYs
    # reductions, softmax, pooling (rows beyond the headline configurations)
    def hbm_case(config, fn_gpu, fn_cpu, nbytes, check, inputs):
        """fn_gpu(x) on each of the rotating inputs (every byte from HBM); the warm figure goes into the note."""
        got = fn_gpu(inputs[0])
        want = fn_cpu()
        _, ev = timer.run(lambda: fn_gpu(inputs[0]), 50, 5, WARM_S)
        gpu_s = run_rotating(timer, [(lambda x=x: fn_gpu(x)) for x in inputs], 10)
        cpu_s = cpu_time(fn_cpu, budget=2.0)
        emit(config=config, dtype="f32", gpu_ms=round(gpu_s * 1e3, 4), gpu_rate=round(nbytes / gpu_s / 1e9, 1), rate_unit="GB/s",
             pct_peak=round(100 * nbytes / gpu_s / 1e9 / HBM_PEAK_GBS, 1), peak_used="HBM 8000 GB/s",
             cpu_impl="oracle/reduce_pool.c (serial port of the reference's fold / softmax / maxpool2d)", cpu_threads=1,
             cpu_ms=round(cpu_s * 1e3, 2), speedup_vs_cpu=round(cpu_s / gpu_s, 1), note=warm_note(ev / 50, nbytes), **check(got, want))
    n2 = 8192 * 8192 * 4
    absX = np.abs(X)
    hbm_case("f32 8192x8192 sum(axis=1)", lambda x: am.sum(x, 1), lambda: am_oracle.reduce_axis("sum", X, 1), n2,
             lambda g, w: dict(max_err_rel_to_sum_abs=float(np.max(np.abs(g.toCpu().astype(np.float64) - w) / am_oracle.reduce_axis("sum", absX, 1)))), dXs)
    hbm_case("f32 8192x8192 sum(axis=0)", lambda x: am.sum(x, 0), lambda: am_oracle.reduce_axis("sum", X, 0), n2,
             lambda g, w: dict(max_err_rel_to_sum_abs=float(np.max(np.abs(g.toCpu().astype(np.float64) - w) / am_oracle.reduce_axis("sum", absX, 0)))), dXs)
    hbm_case("f32 8192x8192 softmax (rows)", lambda x: am.softmax(x), lambda: am_oracle.softmax(X), 2 * n2,
             lambda g, w: dict(max_rel_err=float(np.max(np.abs(g.toCpu() - w) / w))), dXs)
    del dXs
    P = rng(4005).uniform(-1, 1, (64, 64, 112, 112)).astype(np.float32)
    dPs = [am.toHip(P) for _ in range(ROTATE + 2)]   # 205 MB each
    hbm_case("f32 maxpool2d 64x64x112x112, 2x2 stride 2", lambda x: am.maxpool2d(x, (2, 2), (0, 0), (2, 2)),
             lambda: am_oracle.maxpool2d(P, (2, 2), (0, 0), (2, 2)), P.nbytes + P.nbytes // 4 + P.size // 4 * 8,
             lambda g, w: dict(bit_exact=bool(np.array_equal(g[1].toCpu(), w[1]) and np.array_equal(g[0].toCpu(), w[0]))), dPs)
    del dPs
    r = bench_chain(am, timer, 200, 20)
    emit(config="f32 inference chain (4 GEMMs, fused bias+ReLU)", dtype="f32", hipgraph_us=r["hipgraph_us"], eager_us=r["eager_us"],
         note=r["note"])
    r = bench_ex02(am, timer, 200, 20)
    emit(config="f32 example-2 forward pass, batch 64 (6 kernels)", dtype="f32", hipgraph_us=r["hipgraph_us"], eager_us=r["eager_us"],
         note=r["note"])


def run_only(am, timer, which, steps, warmup):
    """One workload, nothing else on the stream: what the rocprofv3 summaries under profiles/ time."""
    from arraymancer_amd import tensor_hip as th
    if which == "gemm_f32":
        r = bench_gemm_f32(am, timer, steps, warmup)
        return dict(only=which, ms_per_launch=round(r["ev"] / steps * 1e3, 4), launches=steps + warmup)
    if which == "chain":
        r = bench_chain(am, timer, steps, warmup)
        return dict(only=which, hipgraph_us=r["hipgraph_us"], eager_us=r["eager_us"])
    if which == "ex02":
        r = bench_ex02(am, timer, steps, warmup)
        return dict(only=which, hipgraph_us=r["hipgraph_us"], eager_us=r["eager_us"])
    if which == "conv_backward":
        r = bench_conv_backward(am, timer, steps, warmup, first_only=True)[0]
        return dict(only=which, ms_per_step=r["ms_per_step"], tflops=r["value"], forward_ms=r["forward_ms"])
    if which in ("gemm_i32", "gemm_i32_valu"):
        if which == "gemm_i32_valu":
            os.environ["AM_HIP_GEMM_I32_PATH"] = "valu"   # the vector-ALU kernel instead of the digit-sliced matrix-core path
        n = 4096
        A = np.random.default_rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(np.int32)
        B = np.random.default_rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(np.int32)
        dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), np.int32)
        fn = lambda: am.gemm(1, dA, dB, 0, dC)
    elif which in ("gemm_f32_1024", "gemm_f32_2048"):
        n = int(which.rsplit("_", 1)[1])
        dA = am.toHip(np.random.default_rng(1001).standard_normal((n, n)).astype(np.float32))
        dB = am.toHip(np.random.default_rng(1002).standard_normal((n, n)).astype(np.float32))
        dC = am.empty((n, n), np.float32)
        fn = lambda: am.gemm(1, dA, dB, 0, dC)
    elif which == "gemm_i32_1500":
        n = 1500
        dA = am.toHip(np.random.default_rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(np.int32))
        dB = am.toHip(np.random.default_rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(np.int32))
        dC = am.empty((n, n), np.int32)
        fn = lambda: am.gemm(1, dA, dB, 0, dC)
    elif which == "bcast_add_rotating":      # five buffer sets round robin: every byte of every launch comes from HBM
        X = np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
        b = am.toHip(np.random.default_rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32))
        bb = b.broadcast((8192, 8192))
        dXs = [am.toHip(X) for _ in range(ROTATE)]
        dYs = [am.empty((8192, 8192), np.float32) for _ in range(ROTATE)]
        rounds = max(steps // ROTATE, 4)
        per = run_rotating(timer, [(lambda i=i: th._binary_into("add", dYs[i], dXs[i], bb)) for i in range(ROTATE)], rounds)
        return dict(only=which, ms_per_launch=round(per * 1e3, 4), launches=(rounds + 1) * ROTATE)
    elif which == "gemm_f64":
        pa = np.random.default_rng(3001).standard_normal((1024, 2048))
        pb = np.random.default_rng(3002).standard_normal((1024, 6144))
        dA, dB = am.toHip(pa).transpose(), am.toHip(pb)[:, ::2]
        dC = am.toHip(np.random.default_rng(3003).standard_normal((2048, 3072)))
        fn = lambda: am.gemm(1.5, dA, dB, 0.5, dC)
    elif which in ("sum_rows", "sum_cols", "softmax"):
        dX = am.toHip(np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32))
        fn = {"sum_rows": lambda: am.sum(dX, 1), "sum_cols": lambda: am.sum(dX, 0), "softmax": lambda: am.softmax(dX)}[which]
    elif which == "maxpool":
        dX = am.toHip(np.random.default_rng(4005).uniform(-1, 1, (256, 64, 112, 112)).astype(np.float32))
        fn = lambda: am.maxpool2d(dX, (2, 2), (0, 0), (2, 2))
    elif which == "transposed_add":   # X + Z^T: operands with unit strides on different axes, three buffer sets round robin
        X = np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
        dXs = [am.toHip(X) for _ in range(3)]
        dYs = [am.empty((8192, 8192), np.float32) for _ in range(3)]
        rounds = max(steps // 3, 4)
        per = run_rotating(timer, [(lambda i=i: th._binary_into("add", dYs[i], dXs[i], dXs[(i + 1) % 3].transpose())) for i in range(3)], rounds)
        return dict(only=which, ms_per_launch=round(per * 1e3, 4), launches=(rounds + 1) * 3)
    elif which in ("bias_short_rows", "sum_cols_narrow", "sum_rows_short", "softmax_short_rows"):
        # tall and skinny: a [batch x features] activation with its bias, the bias gradient, row sums and softmax of short rows
        rows, cols = (65536, 512) if which in ("bias_short_rows", "sum_cols_narrow") else (1048576, 64)
        dX = am.toHip(np.random.default_rng(4001).uniform(-1, 1, (rows, cols)).astype(np.float32))
        if which == "bias_short_rows":
            dY = am.empty((rows, cols), np.float32)
            bb = am.toHip(np.random.default_rng(4002).uniform(-1, 1, (1, cols)).astype(np.float32)).broadcast((rows, cols))
            fn = lambda: th._binary_into("add", dY, dX, bb)
        else:
            fn = {"sum_cols_narrow": lambda: am.sum(dX, 0), "sum_rows_short": lambda: am.sum(dX, 1), "softmax_short_rows": lambda: am.softmax(dX)}[which]
    elif which in ("sce_forward", "sce_backward"):   # sparse softmax cross-entropy of [65536 x 1000] scores (262 MB)
        rows, cols = 65536, 1000
        dX = am.toHip(np.random.default_rng(4006).standard_normal((rows, cols)).astype(np.float32))
        lab = am.toHip(np.random.default_rng(4007).integers(0, cols, rows).astype(np.int64))
        fn = (lambda: am.sparse_softmax_cross_entropy(dX, lab)) if which == "sce_forward" else (lambda: am.sparse_softmax_cross_entropy_backward(1.0, dX, lab))
    elif which == "gemm_f32_long_k":   # the weight gradient of a dense layer over a large batch: few tiles, very long k
        dA = am.toHip(np.random.default_rng(1001).standard_normal((500, 65536)).astype(np.float32))
        dB = am.toHip(np.random.default_rng(1002).standard_normal((65536, 800)).astype(np.float32))
        dC = am.empty((500, 800), np.float32)
        fn = lambda: am.gemm(1, dA, dB, 0, dC)
    else:
        X = np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
        dX, dY = am.toHip(X), am.empty((8192, 8192), np.float32)
        if which == "copy":      # plain copy of known size: 268 435 456 B read + 268 435 456 B written
            fn = lambda: th._unary_into("copy", dY, dX)
        else:
            b = am.toHip(np.random.default_rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32))
            bb = b.broadcast((8192, 8192))
            fn = lambda: th._binary_into("add", dY, dX, bb)
    wall, ev = timer.run(fn, steps, warmup, WARM_S)
    return dict(only=which, ms_per_launch=round(ev / steps * 1e3, 4), launches=steps + warmup)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-others", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--report", action="store_true",
                    help="print one JSON line per configuration (GPU vs CPU port, parity at full size) instead of the single benchmark line")
    ap.add_argument("--only", choices=["gemm_f32", "gemm_i32", "gemm_i32_valu", "gemm_f64", "bcast_add", "copy", "chain", "ex02", "sum_rows", "sum_cols", "softmax", "maxpool", "transposed_add", "bias_short_rows", "sum_cols_narrow", "sum_rows_short", "softmax_short_rows", "gemm_f32_long_k", "conv_backward", "sce_forward", "sce_backward",
                                      "gemm_f32_1024", "gemm_f32_2048", "gemm_i32_1500", "bcast_add_rotating"],
                    help="profiling aid: run just this workload's launches and print a short JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one MI355X; --gpus above 1 is not supported "
              "(no collective or multi-GPU code is part of this path)", file=sys.stderr)
        sys.exit(2)

    import arraymancer_amd as am
    L = am.load_library()
    am.sync()
    info = device_info(L)
    timer = Timer(am, L)

    if args.only:
        print(json.dumps(run_only(am, timer, args.only, args.steps, args.warmup)))
        return
    if args.report:
        config_report(am, timer, L)
        return

    # The same W warm-up steps + K timed steps twice: straight from the idle device (`from_idle`: the shader
    # clock is still climbing then), and again right after 80 ms of register-only matrix-core work that is not
    # the workload (`value`: the clock the device holds under sustained load, printed beside it).
    idle = bench_gemm_f32(am, timer, args.steps, args.warmup)
    r = bench_gemm_f32(am, timer, args.steps, args.warmup, host=idle["host"], device_warm_s=0.08)
    f64_views = [] if args.no_others else [bench_gemm_f64_views(am, timer, args.steps, args.warmup)]
    ceilings = measured_ceilings(L)
    tflops = r["flops"] * args.steps / r["wall"] / 1e12
    kern_tflops = r["flops"] / (r["ev"] / args.steps) / 1e12
    traffic, traffic_src = load_traffic("gemm_f32_4096")
    line = {
        "metric": "GEMM TFLOP/s (%MFMA peak) fp32/int32 4096^3; broadcast op HBM GB/s (%peak)",
        "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["wall"] / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "f32 GEMM C=A*B, M=N=K=4096, row-major contiguous, uniform[-1,1) seeds 1001/1002 "
                               "(the 4096^3 size the metric is quoted on)"},
        "roofline": at_clock({"bound": "mfma", "achieved": round(kern_tflops, 3), "peak": MFMA_F32_PEAK_TFLOPS,
                              "unit": "TFLOP/s", "frac": round(kern_tflops / MFMA_F32_PEAK_TFLOPS, 4),
                              "traffic": traffic, "traffic_source": traffic_src}, MFMA_F32_PEAK_TFLOPS, r["sclk_mhz"]),
        "from_idle": {"value": round(idle["flops"] * args.steps / idle["wall"] / 1e12, 3), "unit": "TFLOP/s",
                      "ms_per_step": round(idle["wall"] / args.steps * 1e3, 4), "sclk_mhz": idle["sclk_mhz"],
                      "what": "the same warm-up and timed steps started on the idle device, before anything else ran: the shader "
                              "clock needs 20-50 ms under load to reach the frequency it then holds. `value` is taken right "
                              "after 80 ms of register-only matrix-core work (am_hip_diag_peak, not the workload)"},
        "device": info,
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_gemm_f32(*r["host"])
    if not args.no_others:
        line["measured_ceilings"] = dict(ceilings, unit="T(FL)OP/s (hbm_*: TB/s)",
                                         how="am_hip_diag_peak: register-only MFMA / VALU chains; am_hip_diag_hbm: streaming kernels over rotating buffers")
        line["others"] = other_workloads(am, timer, args.steps, args.warmup, ceilings, first=f64_views)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
