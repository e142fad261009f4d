#!/usr/bin/env python3
"""Benchmark of the GEMM + broadcast hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-others] [--no-cpu] [--no-graphs]
    python bench.py --only <workload> [--steps K] [--warmup W]     one entry of `others`, alone (what profiles/ traces)
    python bench.py --report                                        one line per configuration with the CPU port beside it

Prints ONE JSON line. The headline workload is the float32 GEMM C = A*B at M = N = K = 4096
(row-major, A and B iid uniform[-1, 1) from fixed seeds, resident in HBM before the timed
region). A step is one launch of the GEMM. `value` is TFLOP/s over the K timed steps, wall clock
bracketed by stream synchronisation; `roofline` prices the same kernel against the MFMA fp32
peak using HIP events recorded on the library's stream; `cpu_baseline` times the CPU restatement
of the reference's laser gemm_strided (oracle/, OpenMP, all host cores) on the same workload and
`cpu_blas_standin` NumPy's bundled BLAS on it (the reference's float `*` goes through CBLAS).
`others` carries the remaining configurations of the path, each with its own bound, in the order
of the configurations they belong to (C1 .. C5, then the rows beyond them).

Protocol of every entry: a register-only chain of the workload's arithmetic type (am_hip_diag_peak:
no memory traffic, not the workload) keeps the device busy until its shader clock has settled, then
W warm-up launches, then K launches timed between two HIP events on the library's stream. `--only X`
runs exactly the code that produces entry X of the default line, so a kernel trace of it averages
launches taken under the same protocol.
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
VALU_FULL_RATE_TOPS = 78.6     # 256 CU x 64 lanes x 2 ops x 2.4 GHz: one 32-bit multiply-add per lane and cycle
# Measured separately with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE), see profiles/; None = not measured.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")

SPIN_F32, SPIN_F64, SPIN_VALU32, SPIN_VALU64, SPIN_I8 = 0, 1, 2, 3, 4   # kinds of am_hip_diag_peak
MATRIX_WARM_S = 1.0   # seconds of its own launches before a matrix-bound entry is timed (see Timer.run)
ROTATE = 5   # buffer sets of the rotating protocol: together far beyond the 256 MB memory-side cache


def device_info(L):
    name = ctypes.create_string_buffer(128)
    cus, khz, lds = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    hbm = ctypes.c_size_t()
    L.am_hip_device_info(name, 128, ctypes.byref(cus), ctypes.byref(khz), ctypes.byref(hbm), ctypes.byref(lds))
    return dict(name=name.value.decode(), compute_units=cus.value, clock_mhz=khz.value / 1000.0,
                hbm_gib=round(hbm.value / 2**30, 1))


def spin_up(L, seconds=0.08, kind=SPIN_F32):
    """Keeps the device busy for `seconds` with a register-only chain (no memory traffic, not the workload):
    the shader clock climbs from the 2.1 GHz of an idle device to what it holds under sustained load of that kind
    (2.39 GHz under float32 matrix instructions; float64 ones need 0.2-0.3 s; int8 ones settle lower)."""
    t_end = time.perf_counter() + seconds
    v = ctypes.c_double()
    iters = 5000 if kind == SPIN_VALU64 else 20000
    while time.perf_counter() < t_end:
        L.am_hip_diag_peak(kind, iters, 2, ctypes.byref(v))


class Timer:
    """HIP events on the library stream + host wall clock around a synchronised region."""

    def __init__(self, am, L):
        self.am, self.L = am, L
        self.e0, self.e1 = ctypes.c_void_p(), ctypes.c_void_p()
        L.am_hip_event_create(ctypes.byref(self.e0))
        L.am_hip_event_create(ctypes.byref(self.e1))
        self.sclk_mhz = None
        self.launches = 0
        self.history = []

    def run(self, fn, steps, warmup, spin=(SPIN_F32, 0.08), min_warm_s=0.05):
        """`spin` = (kind, seconds) of register-only work first (None: start from whatever state the device is in, and
        no time-based warm-up either), then `warmup` untimed calls of fn - continued until they have kept the device
        busy for min_warm_s: what a kernel is timed at is the clock its own launches sustain, and the governor settles
        slowly after the kind of work changes (f32 1024^3 launches: 2.03 GHz after 30 ms of them, 2.20 after 0.3 s,
        2.32 after 1 s; the matrix-bound entries therefore warm up for MATRIX_WARM_S) - then `steps` timed ones. While the timed steps run, the GEMM kernels count shader cycles against the constant-rate counter
        (am_hip_diag_clock_*): self.sclk_mhz is the shader clock they sustained (None when no such kernel ran).
        Returns (wall seconds, event seconds) for all timed steps."""
        if spin:
            spin_up(self.L, spin[1], spin[0])
        if "BENCH_WARM_S" in os.environ:      # experiments
            min_warm_s = float(os.environ["BENCH_WARM_S"])
        extra = 0
        self.L.am_hip_event_record(self.e0)
        for _ in range(warmup):
            fn()
        self.L.am_hip_event_record(self.e1)
        self.am.sync()
        if spin and min_warm_s > 0 and warmup > 0:
            ms = ctypes.c_float()
            self.L.am_hip_event_elapsed_ms(self.e0, self.e1, ctypes.byref(ms))
            if ms.value / 1e3 < min_warm_s:
                per_call = max(ms.value / 1e3 / warmup, 1e-6)
                extra = min(int((min_warm_s - ms.value / 1e3) / per_call) + 1, 20000)
                for _ in range(extra):
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
        self.launches = steps + warmup + extra
        self.history.append(steps)            # timed steps of every run, in order (what a trace of --only is cut by)
        return wall, ms.value / 1e3


def run_rotating(timer, fns, rounds, warm_rounds=1):
    """The same operation on len(fns) disjoint buffer sets, issued round robin, so that no byte of an
    input is still in the memory-side cache when it is read again: every byte comes from HBM.
    Returns seconds per launch (HIP events)."""
    state = {"i": 0}

    def step():
        fns[state["i"] % len(fns)]()
        state["i"] += 1
    _, ev = timer.run(step, rounds * len(fns), warm_rounds * len(fns), (SPIN_F32, 0.05))
    return ev / (rounds * len(fns))


def measured_ceilings(L):
    """Issue ceilings of this chip from register-only micro-benchmarks (no memory traffic): what a
    perfect kernel could reach at the clocks the device sustains, T(FL)OP/s; and what HBM delivers to
    kernels that only stream (read, write, copy of 256 MiB per launch over six rotating buffers = 1.5 GiB
    per direction, so every byte comes from HBM; 16-byte non-temporal accesses, four in flight per lane;
    the best of a few grid sizes), TB/s. runtime_d2d_copy_tbs: the same rotating copy made by the runtime's own
    hipMemcpyAsync (device to device) instead of a kernel of this library."""
    out = {}
    for kind, name, iters in [(0, "mfma_f32", 20000), (1, "mfma_f64", 20000), (2, "valu_int32_mac", 20000), (3, "valu_int64_mac", 5000),
                              (4, "mfma_i8", 20000)]:
        v = ctypes.c_double()
        if L.am_hip_diag_peak(kind, iters, 2, ctypes.byref(v)) == 0:
            out[name] = round(v.value / 1e12, 2)
    # the int32 GEMM's instruction alone, with the shader clock it ran at: cycles per instruction and SIMD
    v, mhz = ctypes.c_double(), ctypes.c_double()
    L.am_hip_diag_peak(6, 20000, 2, ctypes.byref(v))
    if L.am_hip_diag_clock_begin() == 0 and L.am_hip_diag_peak(6, 20000, 2, ctypes.byref(v)) == 0 and \
            L.am_hip_diag_clock_end(ctypes.byref(mhz)) == 0 and mhz.value > 0:
        info = device_info(L)
        per_simd_per_s = v.value / 2.0 / 64.0 / (info["compute_units"] * 4)      # wavefront instructions per SIMD and second
        out["v_mad_u64_u32"] = dict(tops=round(v.value / 1e12, 2), sclk_mhz=round(mhz.value, 0),
                                    cycles_per_wavefront_instruction=round(mhz.value * 1e6 / per_simd_per_s, 2))
    for kind, name in [(0, "hbm_read"), (1, "hbm_write"), (2, "hbm_copy")]:
        best = 0.0
        for blocks_per_cu in (2, 8, 32):
            for flags in ((1,) if kind == 0 else (2, 0) if kind == 1 else (3,)):
                v = ctypes.c_double()
                if L.am_hip_diag_hbm(kind, 256 << 20, 6, blocks_per_cu, 4, flags, 24, ctypes.byref(v)) == 0:
                    best = max(best, v.value)
        if best:
            out[name + "_tbs"] = round(best / 1e12, 3)
    v = ctypes.c_double()
    if L.am_hip_diag_hbm(3, 256 << 20, 6, 1, 4, 0, 24, ctypes.byref(v)) == 0:
        out["runtime_d2d_copy_tbs"] = round(v.value / 1e12, 3)
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
        roof["frac_at_sclk"] = round(roof["achieved"] / (peak * sclk_mhz / nominal_mhz), 4)
    return roof


def mfma_roof(tflops, peak, sclk, unit=None):
    """(the unit is the entry's own unless given)"""
    r = dict(bound="mfma", achieved=round(tflops, 3), peak=peak, frac=round(tflops / peak, 4))
    if unit:
        r["unit"] = unit
    return at_clock(r, peak, sclk)


def hbm_roof(gbs, **extra):
    return dict(bound="hbm", achieved=round(gbs, 1), peak=HBM_PEAK_GBS, frac=round(gbs / HBM_PEAK_GBS, 4), **extra)


class Ctx:
    def __init__(self, am, L, timer, steps, warmup, graphs=True):
        self.am, self.L, self.timer, self.steps, self.warmup, self.graphs = am, L, timer, steps, warmup, graphs
        self._ceilings = None

    @property
    def ceilings(self):
        if self._ceilings is None:
            self._ceilings = measured_ceilings(self.L)
        return self._ceilings


WORKLOADS = {}   # name -> (function(ctx) -> entry or list of entries, part of the default line?)


def workload(name, default=True):
    def deco(fn):
        WORKLOADS[name] = (fn, default)
        return fn
    return deco


# ------------------------------------------------------------------------------------------ headline and C1
def bench_gemm_f32(ctx, steps, warmup, n=4096, host=None, spin=(SPIN_F32, 0.08), min_warm_s=0.0):
    am, timer = ctx.am, ctx.timer
    A, B = host or (np.random.default_rng(1001).uniform(-1, 1, (n, n)).astype(np.float32),
                    np.random.default_rng(1002).uniform(-1, 1, (n, n)).astype(np.float32))
    dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), np.float32)
    wall, ev = timer.run(lambda: am.gemm(1.0, dA, dB, 0.0, dC), steps, warmup, spin, min_warm_s)
    return dict(wall=wall, ev=ev, flops=2.0 * n ** 3, host=(A, B), sclk_mhz=timer.sclk_mhz)


def gemm_f32_entry(ctx, n, config, steps, min_warm_s=MATRIX_WARM_S):
    r = bench_gemm_f32(ctx, steps, ctx.warmup, n=n, min_warm_s=min_warm_s)
    t = r["flops"] / (r["ev"] / steps) / 1e12
    return dict(workload=f"f32 GEMM {n}^3", config=config, unit="TFLOP/s", value=round(r["flops"] * steps / r["wall"] / 1e12, 3),
                ms_per_step=round(r["ev"] / steps * 1e3, 5), roofline=mfma_roof(t, MFMA_F32_PEAK_TFLOPS, r["sclk_mhz"]))


@workload("gemm_f32", default=False)     # the headline itself, for traces (the default line times it as `value`)
def wl_gemm_f32(ctx):
    return gemm_f32_entry(ctx, 4096, "headline", ctx.steps, min_warm_s=0.0)   # the headline's own protocol: spin, W steps, K timed


@workload("gemm_f32_1024")
def wl_gemm_f32_1024(ctx):
    return gemm_f32_entry(ctx, 1024, "C1", max(ctx.steps, 200))


@workload("gemm_f32_2048")
def wl_gemm_f32_2048(ctx):
    return gemm_f32_entry(ctx, 2048, "C1", max(ctx.steps, 100))


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
                sample=f"full f32 GEMM {n}^3, best of {len(times)}, oracle/laser_gemm.c (OpenMP)")


def cpu_blas_standin_gemm_f32(A, B, budget_s=6.0):
    """The reference's float `*` goes through CBLAS (p_operator_blas_l2l3.nim:175-187); that library is whatever the
    host links and is not part of the reference's sources. NumPy's bundled BLAS (A @ B) stands in for it on the same
    full workload: one untimed run, then as many timed runs as fit the budget."""
    threads = None
    try:
        from threadpoolctl import threadpool_info
        pools = [p for p in threadpool_info() if p.get("user_api") == "blas"]
        if pools:
            threads = pools[0].get("num_threads")
            lib = f"{pools[0].get('internal_api')} {pools[0].get('version')}"
    except Exception:
        pools = []
    n = A.shape[0]
    A @ B
    times = []
    t_end = time.perf_counter() + budget_s
    while not times or (time.perf_counter() < t_end and len(times) < 20):
        t0 = time.perf_counter()
        A @ B
        times.append(time.perf_counter() - t0)
    best = min(times)
    return dict(value=round(2.0 * n ** 3 / best / 1e12, 4), unit="TFLOP/s", cores=threads or os.cpu_count(), kind="stand-in",
                sample=f"full f32 GEMM {n}^3, best of {len(times)}, NumPy A @ B" + (f" ({lib})" if pools else "") + " for the CBLAS behind `*`")


# ------------------------------------------------------------------------------------------ C2: integer GEMM
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


def int_gemm_entries(ctx, dt, n, lo, hi, config, label, valu=True, seeds=(2001, 2002)):
    """One integer product through the library's own choice of path (digit-sliced on the int8 matrix cores at these
    sizes: whole call, the two digit-splitting passes included) and, beside it, through the VALU kernel the path
    falls back to (priced against the measured multiply-add ceiling and against the full-rate bound of one 32-bit
    multiply-add per lane and cycle)."""
    am, timer = ctx.am, ctx.timer
    sfx = "i32" if dt == np.int32 else "i64"
    A = np.random.default_rng(seeds[0]).integers(lo, hi, (n, n), endpoint=True).astype(dt)
    B = np.random.default_rng(seeds[1]).integers(lo, hi, (n, n), endpoint=True).astype(dt)
    pairs, npairs = digit_pairs(A, B), (10 if dt == np.int32 else 36)
    dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), dt)
    kd = max(20, ctx.steps)
    wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), kd, ctx.warmup, (SPIN_I8, 0.08), min_warm_s=0.3)
    tops = 2.0 * n ** 3 / (ev / kd) / 1e12
    entry = dict(workload=f"{sfx} GEMM {n}^3, {label}", config=config, unit="Top/s", value=round(2.0 * n ** 3 * kd / wall / 1e12, 3),
                 ms_per_step=round(ev / kd * 1e3, 5), digit_pairs=f"{pairs}/{npairs}",
                 roofline=mfma_roof(pairs * tops, MFMA_I8_PEAK_TOPS, timer.sclk_mhz, unit="int8 TOP/s"))
    out = [entry]
    if valu:
        env = f"AM_HIP_GEMM_{sfx.upper()}_PATH"
        k = max(3, ctx.steps // 4) if n >= 4096 else max(20, ctx.steps)
        os.environ[env] = "valu"
        try:
            _, ev_valu = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), k, 2, (SPIN_VALU32 if dt == np.int32 else SPIN_VALU64, 0.08), min_warm_s=0.3)
        finally:
            del os.environ[env]
        vt = 2.0 * n ** 3 / (ev_valu / k) / 1e12
        peak = ctx.ceilings.get("valu_int32_mac" if dt == np.int32 else "valu_int64_mac")
        roof = dict(bound="valu", achieved=round(vt, 3), peak=peak, unit="Top/s, measured",
                    frac=round(vt / peak, 4) if peak else None)
        if dt == np.int32:
            roof["frac_of_78.6"] = round(vt / VALU_FULL_RATE_TOPS, 4)
        if timer.sclk_mhz:
            roof["sclk_mhz"] = timer.sclk_mhz
            if dt == np.int32:
                roof["frac_of_78.6_at_sclk"] = round(vt / (VALU_FULL_RATE_TOPS * timer.sclk_mhz / 2400.0), 4)
        out.append(dict(workload=f"{sfx} GEMM {n}^3, {label}, VALU", config=config, unit="Top/s", value=round(vt, 3),
                        ms_per_step=round(ev_valu / k * 1e3, 5), roofline=roof))
    return out


@workload("gemm_i32_1500")
def wl_gemm_i32_1500(ctx):
    return int_gemm_entries(ctx, np.int32, 1500, -100, 100, "C2", "in [-100,100]")


@workload("gemm_i32")
def wl_gemm_i32(ctx):
    return int_gemm_entries(ctx, np.int32, 4096, -100, 100, "C2", "in [-100,100]")


@workload("gemm_i32_prepared")
def wl_gemm_i32_prepared(ctx):
    """int32 4096^3 with the digit planes of B, then of both operands, split once ahead of the timed calls
    (am_hip_digits_prepare_i32): what a weight matrix that enters many products costs per product."""
    am, timer, n = ctx.am, ctx.timer, 4096
    A = np.random.default_rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(np.int32)
    B = np.random.default_rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(np.int32)
    dA, dB, dC = am.toHip(A), am.toHip(B), am.empty((n, n), np.int32)
    pa, pb = am.digits_prepare(dA, "left"), am.digits_prepare(dB, "right")
    kd = max(20, ctx.steps)
    out = []
    for label, kw in (("B's digits prepared", dict(b_digits=pb)), ("A's and B's digits prepared", dict(a_digits=pa, b_digits=pb))):
        wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC, **kw), kd, ctx.warmup, (SPIN_I8, 0.08), min_warm_s=0.3)
        tops = 2.0 * n ** 3 / (ev / kd) / 1e12
        out.append(dict(workload=f"i32 GEMM 4096^3, in [-100,100], {label}", config="C2", unit="Top/s",
                        value=round(2.0 * n ** 3 * kd / wall / 1e12, 3), ms_per_step=round(ev / kd * 1e3, 5),
                        roofline=mfma_roof(tops, MFMA_I8_PEAK_TOPS, timer.sclk_mhz, unit="int8 TOP/s")))
    return out


@workload("gemm_i32_whole_range")
def wl_gemm_i32_whole(ctx):
    return int_gemm_entries(ctx, np.int32, 4096, -2 ** 31, 2 ** 31 - 1, "C2", "whole int32 range", valu=False)


@workload("gemm_i64")
def wl_gemm_i64(ctx):
    return int_gemm_entries(ctx, np.int64, 4096, -100, 100, "C2", "in [-100,100]")


@workload("gemm_i32_valu", default=False)   # the VALU kernel alone at 4096^3 (traces, counters)
def wl_gemm_i32_valu(ctx):
    os.environ["AM_HIP_GEMM_I32_PATH"] = "valu"
    am, timer, n = ctx.am, ctx.timer, 4096
    dA = am.toHip(np.random.default_rng(2001).integers(-100, 100, (n, n), endpoint=True).astype(np.int32))
    dB = am.toHip(np.random.default_rng(2002).integers(-100, 100, (n, n), endpoint=True).astype(np.int32))
    dC = am.empty((n, n), np.int32)
    k = max(3, ctx.steps // 4)
    _, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), k, 2, (SPIN_VALU32, 0.08))
    vt = 2.0 * n ** 3 / (ev / k) / 1e12
    return dict(workload="i32 GEMM 4096^3, entries in [-100, 100], VALU kernel", config="C2", unit="Top/s", value=round(vt, 3),
                ms_per_step=round(ev / k * 1e3, 5), roofline={"bound": "valu", "achieved": round(vt, 3), "peak": VALU_FULL_RATE_TOPS,
                                                               "unit": "Top/s (full-rate bound)", "frac": round(vt / VALU_FULL_RATE_TOPS, 4),
                                                               "sclk_mhz": timer.sclk_mhz})


@workload("matmul_i64_1500_published")
def wl_i64_1500(ctx):
    """The one figure the reference publishes for this path: `a * b` of two 1500 x 1500 int64 tensors with entries in
    [0, 99] (benchmarks/integer_matmul.nim:8-33: 0.14 s on an 18-core i9-9980XE, the wall time of a whole process with
    the random fill, so the ratio is an upper bound on the kernel-to-kernel one)."""
    am, timer, n5 = ctx.am, ctx.timer, 1500
    A = np.random.default_rng(2003).integers(0, 99, (n5, n5), endpoint=True).astype(np.int64)
    B = np.random.default_rng(2004).integers(0, 99, (n5, n5), endpoint=True).astype(np.int64)
    dA, dB = am.toHip(A), am.toHip(B)
    dC = dA * dB
    k5 = max(ctx.steps, 50)
    wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), k5, ctx.warmup, (SPIN_I8, 0.08))
    want = A[n5 // 2] @ B          # one row of the product (the benchmark prints one element of it)
    tops = 2.0 * n5 ** 3 / (ev / k5) / 1e12
    return dict(workload="i64 matmul 1500^2, entries in [0, 99]", config="published",
                unit="Top/s", value=round(2.0 * n5 ** 3 * k5 / wall / 1e12, 3), ms_per_step=round(ev / k5 * 1e3, 5),
                row_750_matches_numpy=bool(np.array_equal(dC.toCpu()[n5 // 2], want)),
                roofline=mfma_roof(tops, MFMA_I8_PEAK_TOPS, timer.sclk_mhz, unit="int8 TOP/s"),
                published_s=0.14, published_on="i9-9980XE, integer_matmul.nim:8-33")


# ------------------------------------------------------------------------------------------ C3: float64 views
@workload("gemm_f64")
def wl_gemm_f64_views(ctx):
    """float64 gemm(1.5, A^T view, B[:, ::2] view, 0.5, C), M=2048 N=3072 K=1024 (0.3 s of float64 matrix work first:
    the clock takes longer to settle under float64 matrix instructions than under float32 ones)."""
    am, timer = ctx.am, ctx.timer
    pa = np.random.default_rng(3001).standard_normal((1024, 2048))
    pb = np.random.default_rng(3002).standard_normal((1024, 6144))
    C = np.random.default_rng(3003).standard_normal((2048, 3072))
    dA, dB, dC = am.toHip(pa).transpose(), am.toHip(pb)[:, ::2], am.toHip(C)
    steps = max(ctx.steps, 50)
    wall, ev = timer.run(lambda: am.gemm(1.5, dA, dB, 0.5, dC), steps, ctx.warmup, (SPIN_F64, 0.1), min_warm_s=MATRIX_WARM_S)
    fl = 2.0 * 2048 * 3072 * 1024
    return dict(workload="f64 gemm(1.5, A^T, B[:, ::2], 0.5, C) 2048x3072x1024", config="C3", unit="TFLOP/s",
                value=round(fl * steps / wall / 1e12, 3), ms_per_step=round(ev / steps * 1e3, 5),
                roofline=mfma_roof(fl / (ev / steps) / 1e12, MFMA_F64_PEAK_TFLOPS, timer.sclk_mhz))


# ------------------------------------------------------------------------------------------ C4: broadcast ops
_C4 = {}


def c4_buffers(ctx):
    """X[8192, 8192] f32 five times over (rotating inputs), as many outputs, b[1, 8192] and s[8192, 1]; built once."""
    if not _C4:
        am = ctx.am
        X = np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32)
        b = np.random.default_rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32)
        s = np.random.default_rng(4003).uniform(-1, 1, (8192, 1)).astype(np.float32)
        _C4.update(dXs=[am.toHip(X) for _ in range(ROTATE)], dYs=[am.empty((8192, 8192), np.float32) for _ in range(ROTATE)],
                   bb=am.toHip(b).broadcast((8192, 8192)), sb=am.toHip(s).broadcast((8192, 8192)))
    return _C4


def c4_entry(ctx, name, launch_of, nbytes, same_buffers=None):
    """One HBM-bound pass over five buffer sets round robin (2.5 GiB), so that every byte of every launch comes from
    HBM: both `value` and `roofline` are that figure. The same-buffer time is listed beside it (part of a 256 MiB
    input that is read again at once can still be in the 256 MB memory-side cache)."""
    timer = ctx.timer
    rounds = max(ctx.steps // ROTATE, 4)
    cold = run_rotating(timer, [launch_of(i) for i in range(ROTATE)], rounds)
    launches = timer.launches
    gbs = nbytes / cold / 1e9
    roof = hbm_roof(gbs)
    if not getattr(ctx, "solo", False):      # (a traced run of one workload does not launch the ceiling kernels)
        copy_ceiling = ctx.ceilings.get("hbm_copy_tbs")
        d2d = ctx.ceilings.get("runtime_d2d_copy_tbs")
        if copy_ceiling:
            roof["vs_copy_ceiling"] = round(gbs / (copy_ceiling * 1e3), 4)
        if d2d:
            roof["vs_runtime_d2d"] = round(gbs / (d2d * 1e3), 4)
    e = dict(workload=f"f32 8192x8192 {name}", config="C4", unit="GB/s", value=round(gbs, 1), ms_per_step=round(cold * 1e3, 5), roofline=roof)
    if same_buffers is not None:
        _, ev = timer.run(same_buffers, ctx.steps, ctx.warmup, None)
        e["same_buffers_ms"] = round(ev / ctx.steps * 1e3, 5)
    timer.launches = launches
    return e


C4_BYTES = 2 * 8192 * 8192 * 4 + 8192 * 4


def _c4_binary(ctx, name, op, rhs_key):
    from arraymancer_amd import tensor_hip as th
    c = c4_buffers(ctx)
    rhs = c[rhs_key]
    return c4_entry(ctx, name, lambda i: (lambda: th._binary_into(op, c["dYs"][i], c["dXs"][i], rhs)), C4_BYTES,
                    None if getattr(ctx, "solo", False) else (lambda: th._binary_into(op, c["dYs"][0], c["dXs"][0], rhs)))


@workload("bcast_add_rotating")
def wl_bcast_add(ctx):
    return _c4_binary(ctx, "X +. b[1,8192]", "add", "bb")


@workload("bcast_mul_rotating")
def wl_bcast_mul(ctx):
    return _c4_binary(ctx, "Y *. s[8192,1]", "mul", "sb")


@workload("bias_relu_rotating")
def wl_bias_relu(ctx):
    return _c4_binary(ctx, "map2(X, b, max(0, x+y)) bias+ReLU", "add_relu", "bb")


@workload("bcast_addmul_fused_rotating")
def wl_addmul(ctx):
    from arraymancer_amd import tensor_hip as th
    c = c4_buffers(ctx)
    e = c4_entry(ctx, "(X +. b) *. s fused, one pass",
                 lambda i: (lambda: th._ternary_into("addmul", c["dYs"][i], c["dXs"][i], c["bb"], c["sb"])), C4_BYTES + 8192 * 4)
    return e


@workload("transposed_add")
def wl_transposed_add(ctx):
    from arraymancer_amd import tensor_hip as th
    c = c4_buffers(ctx)
    dXs, dYs = c["dXs"], c["dYs"]
    cold = run_rotating(ctx.timer, [(lambda i=i: th._binary_into("add", dYs[i], dXs[i], dXs[(i + 1) % 3].transpose())) for i in range(3)],
                        max(ctx.steps // 3, 4))
    gbs = 3 * 8192 * 8192 * 4 / cold / 1e9
    return dict(workload="f32 8192x8192 X + Z^T (Z a transposed view)", config="a18", unit="GB/s", value=round(gbs, 1),
                ms_per_step=round(cold * 1e3, 5), roofline=hbm_roof(gbs))


# ------------------------------------------------------------------------------------------ C5 and the rows beyond
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

    stages = [lambda: am.gemm(1.0, k1, x1, 0.0, o1), lambda: am.gemm(1.0, k2, x2, 0.0, o2),
              lambda: am.gemm(1.0, x3, w3t, 0.0, h, epilogue="bias_relu", bias=b3), lambda: am.gemm(1.0, h, w4t, 0.0, o4)]

    def issue():
        for f in stages:
            f()

    # the same four calls with their arguments converted to C types once: what a compiled host pays per launch (the
    # Python wrapper's shape checks and conversions take about as long as the smallest of these kernels runs)
    L, vp, f32 = am.load_library(), ctypes.c_void_p, ctypes.c_float

    def bound(A, B, C, epi=0, bias=None):
        (M, K), N = A.shape, B.shape[1]
        a = (M, N, K, f32(1.0), vp(A.data_ptr()), A.strides[0], A.strides[1], vp(B.data_ptr()), B.strides[0], B.strides[1],
             f32(0.0), vp(C.data_ptr()), C.strides[0], C.strides[1])
        if not epi:
            return L.am_hip_gemm_f32, a
        bb = bias.broadcast((M, N))
        return L.am_hip_gemm_ex_f32, a + (epi, vp(bb.data_ptr()), bb.strides[0], bb.strides[1])
    calls = [bound(k1, x1, o1), bound(k2, x2, o2), bound(x3, w3t, h, 3, b3), bound(h, w4t, o4)]

    def issue_bound():
        rc = 0
        for fn, a in calls:
            rc |= fn(*a)
        if rc:
            raise RuntimeError("a product of the chain failed")

    issue.stages = stages
    issue.bound = issue_bound
    flops = 2.0 * (20 * 25 * 36864 + 50 * 500 * 4096 + 64 * 800 * 500 + 64 * 500 * 10)
    return issue, flops, 17834080, (k1, x1, o1, k2, x2, o2, x3, w3, b3, h, w4, o4)


def eager_and_graph(ctx, issue, capture, steps):
    """issue() from the host `steps` times, then (unless --no-graphs) the same sequence replayed from one HIP graph."""
    timer = ctx.timer
    wall_e, ev_e = timer.run(issue, steps, ctx.warmup, (SPIN_F32, 0.05))
    out = dict(eager_us=round(ev_e / steps * 1e6, 2))
    if getattr(ctx, "solo", False):
        out["eager_wall_us"] = round(wall_e / steps * 1e6, 2)
    best = ev_e
    out["value_is"] = "eager"
    if getattr(issue, "bound", None):
        _, ev_b = timer.run(issue.bound, steps, ctx.warmup, (SPIN_F32, 0.05))
        out["eager_c_abi_us"] = round(ev_b / steps * 1e6, 2)
        if ev_b < best:
            best, out["value_is"] = ev_b, "eager_c_abi"
    if ctx.graphs:
        graph = capture()
        _, ev_g = timer.run(graph.launch, steps, ctx.warmup, (SPIN_F32, 0.05))
        out["hipgraph_us"] = round(ev_g / steps * 1e6, 2)
        if ev_g < best:
            best, out["value_is"] = ev_g, "hipgraph"
    out["value"] = round(best / steps * 1e6, 2)
    return out, best / steps


@workload("chain")
def wl_chain(ctx):
    am = ctx.am
    issue, flops, nbytes, keep = chain_setup(am)

    def capture():
        with am.Graph() as graph:
            issue()
        return graph
    steps = max(ctx.steps, 50)
    # the pre-converted calls do the same work as the wrapper's: all four results, bit for bit
    outs = [keep[2], keep[5], keep[9], keep[11]]
    issue()
    want = [o.toCpu().copy() for o in outs]
    from arraymancer_amd import tensor_hip as th
    for o in outs:
        th._scalar_into("mul", o, o, 0.0, False)      # (the second run must write them again)
    issue.bound()
    if not all(np.array_equal(o.toCpu(), w) for o, w in zip(outs, want)):
        raise RuntimeError("chain: the pre-converted C-ABI calls and the wrapper calls disagree")
    r, best = eager_and_graph(ctx, issue, capture, steps)
    return dict(workload="f32 chain of 4 GEMMs [20x25x36864], [50x500x4096], [64x800x500]+bias+ReLU, [64x500x10]",
                config="C5", unit="us per chain", higher_is_better=False, **r, gflops=round(flops / best / 1e9, 1),
                roofline=dict(hbm_roof(nbytes / best / 1e9), unit="GB/s"))


@workload("chain_phases", default=False)
def wl_chain_phases(ctx):
    """Where the time of each of the chain's four products goes, read inside the kernels (am_hip_diag_phases): one
    launch per clock window, `steps` windows per product, means in microseconds; beside them the time between two
    HIP events around that one launch."""
    am, L, timer = ctx.am, ctx.L, ctx.timer
    issue, _, _, keep = chain_setup(am)
    names = ["[20x25].[25x36864]", "[50x500].[500x4096]", "[64x800].[800x500]+bias+ReLU", "[64x500].[500x10]"]
    spin_up(L, 0.05)
    for _ in range(200):
        issue()
    am.sync()
    out = []
    buf = (ctypes.c_double * 6)()
    ms, mhz = ctypes.c_float(), ctypes.c_double()
    for name, f in zip(names, issue.stages):
        acc, ev_us = np.zeros(6), 0.0
        for _ in range(ctx.steps):
            for _ in range(3):
                issue()                      # the launch that is measured follows others, as in the chain
            L.am_hip_diag_phases_begin()
            L.am_hip_event_record(timer.e0)
            f()
            L.am_hip_event_record(timer.e1)
            L.am_hip_diag_phases(buf)
            L.am_hip_event_elapsed_ms(timer.e0, timer.e1, ctypes.byref(ms))
            acc += np.array(list(buf))
            ev_us += ms.value * 1e3
        acc /= ctx.steps
        out.append(dict(workload=f"f32 {name}", workgroups=int(round(acc[0])), us_to_loads_issued=round(acc[1], 2),
                        us_until_arrived=round(acc[2], 2), us_multiply_and_fold=round(acc[3], 2), us_stores=round(acc[4], 2),
                        us_first_start_to_last_store=round(acc[5], 2), us_between_events=round(ev_us / ctx.steps, 2)))
    return out


@workload("ex02")
def wl_ex02(ctx, batch=64):
    """The whole forward pass of the reference's example 2 (conv - ReLU - maxpool twice, two dense layers) at batch 64:
    six launches per pass issued from the host (each convolution is one launch: the column matrix is gathered by the
    GEMM's loader), and the same six replayed from one HIP graph."""
    from arraymancer_amd import ex02
    am = ctx.am
    rng = np.random.default_rng(5002)
    net = ex02.DemoNet(batch, ex02.random_params(rng), np.float32)
    dx = am.toHip(rng.uniform(0, 1, (batch, 1, 28, 28)).astype(np.float32))
    steps = max(ctx.steps, 50)
    r, best = eager_and_graph(ctx, lambda: net.forward(dx), lambda: net.capture(dx), steps)
    flops = 2.0 * batch * (20 * 25 * 576 + 50 * 500 * 64 + 800 * 500 + 500 * 10)
    return dict(workload=f"f32 example-2 forward pass, batch {batch}, 6 launches",
                config="f2", unit="us per pass", higher_is_better=False, **r, images_per_s=round(batch / best, 0),
                gflops=round(flops / best / 1e9, 1))


_TALL = {}


def tall_buffers(ctx):
    if not _TALL:
        am = ctx.am
        T = np.random.default_rng(4004).uniform(-1, 1, (65536, 512)).astype(np.float32)
        _TALL.update(nbytes=T.nbytes, dTs=[am.toHip(T) for _ in range(3)])
    return _TALL


def hbm_entry(ctx, workload_name, config, launches, nbytes):
    cold = run_rotating(ctx.timer, launches, max(ctx.steps // len(launches), 4))
    gbs = nbytes / cold / 1e9
    return dict(workload=workload_name, config=config, unit="GB/s", value=round(gbs, 1), ms_per_step=round(cold * 1e3, 5),
                roofline=hbm_roof(gbs))


@workload("bias_short_rows")
def wl_bias_short_rows(ctx):
    from arraymancer_amd import tensor_hip as th
    am, t = ctx.am, tall_buffers(ctx)
    dOs = [am.empty((65536, 512), np.float32) for _ in range(3)]
    bias = am.toHip(np.random.default_rng(4005).uniform(-1, 1, (1, 512)).astype(np.float32)).broadcast((65536, 512))
    return hbm_entry(ctx, "f32 65536x512 X +. b[1,512]", "a19",
                     [(lambda i=i: th._binary_into("add", dOs[i], t["dTs"][i], bias)) for i in range(3)], 2 * t["nbytes"] + 2048)


@workload("sum_cols_narrow")
def wl_sum_cols_narrow(ctx):
    from arraymancer_amd import tensor_hip as th
    am, t = ctx.am, tall_buffers(ctx)
    col_sums = am.empty((1, 512), np.float32)
    return hbm_entry(ctx, "f32 sum(X[65536,512], axis=0)", "f3",
                     [(lambda i=i: th.reduce_axis_into("sum", col_sums, t["dTs"][i], 0)) for i in range(3)], t["nbytes"])


@workload("sum_rows_512")
def wl_sum_rows_512(ctx):
    from arraymancer_amd import tensor_hip as th
    am, t = ctx.am, tall_buffers(ctx)
    row_sums = am.empty((65536, 1), np.float32)
    return hbm_entry(ctx, "f32 sum(X[65536,512], axis=1)", "f3",
                     [(lambda i=i: th.reduce_axis_into("sum", row_sums, t["dTs"][i], 1)) for i in range(3)], t["nbytes"])


@workload("gemm_f32_long_k")
def wl_gemm_long_k(ctx):
    am, timer = ctx.am, ctx.timer
    dA = am.toHip(np.random.default_rng(1003).standard_normal((500, 65536)).astype(np.float32))
    dB = am.toHip(np.random.default_rng(1004).standard_normal((65536, 800)).astype(np.float32))
    dC = am.empty((500, 800), np.float32)
    k = max(ctx.steps, 20)
    wall, ev = timer.run(lambda: am.gemm(1, dA, dB, 0, dC), k, ctx.warmup, min_warm_s=MATRIX_WARM_S)
    fl = 2.0 * 500 * 800 * 65536
    return dict(workload="f32 GEMM [500x65536].[65536x800]", config="a19",
                unit="TFLOP/s", value=round(fl * k / wall / 1e12, 3), ms_per_step=round(ev / k * 1e3, 5),
                roofline=mfma_roof(fl / (ev / k) / 1e12, MFMA_F32_PEAK_TFLOPS, timer.sclk_mhz))


# ------------------------------------------------------------------------------------------ not in the default line
def simple(ctx, name, fn, spin=(SPIN_F32, 0.05), steps=None):
    steps = steps or ctx.steps
    _, ev = ctx.timer.run(fn, steps, ctx.warmup, spin)
    return dict(workload=name, ms_per_step=round(ev / steps * 1e3, 5))


def _x8192(ctx):
    return ctx.am.toHip(np.random.default_rng(4001).uniform(-1, 1, (8192, 8192)).astype(np.float32))


@workload("copy", default=False)     # plain copy of known size: 268 435 456 B read + 268 435 456 B written (scales the traffic counters)
def wl_copy(ctx):
    from arraymancer_amd import tensor_hip as th
    dX, dY = _x8192(ctx), ctx.am.empty((8192, 8192), np.float32)
    return simple(ctx, "f32 8192x8192 copy", lambda: th._unary_into("copy", dY, dX))


@workload("bcast_add", default=False)   # the same buffers every launch
def wl_bcast_add_same(ctx):
    from arraymancer_amd import tensor_hip as th
    dX, dY = _x8192(ctx), ctx.am.empty((8192, 8192), np.float32)
    bb = ctx.am.toHip(np.random.default_rng(4002).uniform(-1, 1, (1, 8192)).astype(np.float32)).broadcast((8192, 8192))
    return simple(ctx, "f32 8192x8192 X +. b[1,8192], same buffers every launch", lambda: th._binary_into("add", dY, dX, bb))


@workload("sum_rows", default=False)
def wl_sum_rows(ctx):
    dX = _x8192(ctx)
    return simple(ctx, "f32 8192x8192 sum(axis=1)", lambda: ctx.am.sum(dX, 1))


@workload("sum_cols", default=False)
def wl_sum_cols(ctx):
    dX = _x8192(ctx)
    return simple(ctx, "f32 8192x8192 sum(axis=0)", lambda: ctx.am.sum(dX, 0))


@workload("softmax", default=False)
def wl_softmax(ctx):
    dX = _x8192(ctx)
    return simple(ctx, "f32 8192x8192 softmax (rows)", lambda: ctx.am.softmax(dX))


@workload("maxpool", default=False)
def wl_maxpool(ctx):
    dX = ctx.am.toHip(np.random.default_rng(4005).uniform(-1, 1, (256, 64, 112, 112)).astype(np.float32))
    return simple(ctx, "f32 maxpool2d 256x64x112x112, 2x2 stride 2", lambda: ctx.am.maxpool2d(dX, (2, 2), (0, 0), (2, 2)))


@workload("sum_rows_short", default=False)
def wl_sum_rows_short(ctx):
    dX = ctx.am.toHip(np.random.default_rng(4001).uniform(-1, 1, (1048576, 64)).astype(np.float32))
    return simple(ctx, "f32 sum(X[1048576,64], axis=1)", lambda: ctx.am.sum(dX, 1))


@workload("softmax_short_rows", default=False)
def wl_softmax_short_rows(ctx):
    dX = ctx.am.toHip(np.random.default_rng(4001).uniform(-1, 1, (1048576, 64)).astype(np.float32))
    return simple(ctx, "f32 softmax(X[1048576,64])", lambda: ctx.am.softmax(dX))


def _sce(ctx, backward):   # sparse softmax cross-entropy of [65536 x 1000] scores (262 MB)
    am = ctx.am
    dX = am.toHip(np.random.default_rng(4006).standard_normal((65536, 1000)).astype(np.float32))
    lab = am.toHip(np.random.default_rng(4007).integers(0, 1000, 65536).astype(np.int64))
    fn = (lambda: am.sparse_softmax_cross_entropy_backward(1.0, dX, lab)) if backward else (lambda: am.sparse_softmax_cross_entropy(dX, lab))
    return simple(ctx, f"f32 sparse softmax cross-entropy {'backward' if backward else 'forward'} 65536x1000", fn)


@workload("sce_forward", default=False)
def wl_sce_forward(ctx):
    return _sce(ctx, False)


@workload("sce_backward", default=False)
def wl_sce_backward(ctx):
    return _sce(ctx, True)


@workload("conv_backward", default=False)
def wl_conv_backward(ctx):
    """conv2d_backward (grad_input, grad_weight, grad_bias) on a ResNet-like layer. FLOP counted: twice the forward
    pass (one product for each of the two gradients)."""
    am, timer, steps = ctx.am, ctx.timer, ctx.steps
    N, C, H, W, co, k, pad = 64, 64, 56, 56, 64, 3, 1
    rng = np.random.default_rng(6001)
    ho = H + 2 * pad - k + 1
    x = am.toHip(rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32))
    w = am.toHip(rng.uniform(-1, 1, (co, C, k, k)).astype(np.float32))
    b = am.toHip(rng.uniform(-1, 1, (co, 1, 1)).astype(np.float32))
    g = am.toHip(rng.uniform(-1, 1, (N, co, ho, ho)).astype(np.float32))
    _, ev_f = timer.run(lambda: am.conv2d(x, w, b, (pad, pad), (1, 1)), steps, ctx.warmup)
    _, ev_b = timer.run(lambda: am.conv2d_backward(x, w, b, (pad, pad), (1, 1), g), steps, ctx.warmup)
    fl = 2.0 * N * co * ho * ho * C * k * k
    return dict(workload="f32 conv2d_backward [64,64,56,56], 64 kernels 3x3, pad 1", unit="TFLOP/s",
                value=round(2 * fl / (ev_b / steps) / 1e12, 2), ms_per_step=round(ev_b / steps * 1e3, 5), forward_ms=round(ev_f / steps * 1e3, 5),
                roofline=mfma_roof(2 * fl / (ev_b / steps) / 1e12, MFMA_F32_PEAK_TFLOPS, None))


@workload("ex02_train", default=False)
def wl_ex02_train(ctx, batch=64):
    """One step of example 2's learning loop at batch 64: forward, sparse softmax cross-entropy (read back to the
    host), the backward primitives, the SGD update of the eight parameters; eager and as one replayed graph."""
    from arraymancer_amd import ex02
    am = ctx.am
    rng = np.random.default_rng(5003)
    net = ex02.DemoNet(batch, ex02.random_params(rng), np.float32)
    dx = am.toHip(rng.uniform(0, 1, (batch, 1, 28, 28)).astype(np.float32))
    dl = am.toHip(rng.integers(0, 10, batch).astype(np.int64))
    steps = max(ctx.steps, 20)
    r, best = eager_and_graph(ctx, lambda: net.train_step(dx, dl, 0.01), lambda: net.capture_train_step(dx, dl, 0.01), steps)
    return dict(workload=f"f32 example-2 training step, batch {batch}", unit="us per step", higher_is_better=False, **r,
                images_per_s=round(batch / best, 0))


# ------------------------------------------------------------------------------------------ per-configuration report
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
    ctx = Ctx(am, L, timer, 200, 20)

    def cpu_time(fn, budget=4.0, max_runs=5):
        fn()
        ts = []
        end = time.perf_counter() + budget
        while not ts or (time.perf_counter() < end and len(ts) < max_runs):
            t0 = time.perf_counter(); fn(); ts.append(time.perf_counter() - t0)
        return min(ts)

    def emit(**kw):
        print(json.dumps(kw), flush=True)

    def gemm_case(config, sfx, M, N, K, A, B, dA, dB, alpha=1, beta=0, C0=None, peak=None, peak_used="", unit="TFLOP/s", steps=20,
                  spin=(SPIN_F32, 0.08), warm=0.05):
        dt = A.dtype
        C_host = C0.copy() if C0 is not None else np.zeros((M, N), dt)
        dC = am.toHip(C_host)
        am.gemm(alpha, dA, dB, beta, dC)
        got = dC.toCpu().copy()
        # (with beta != 0 the timed calls go on accumulating into C: only their time is used)
        _, ev = timer.run(lambda: am.gemm(alpha, dA, dB, beta, dC), steps, 3, spin, min_warm_s=warm)
        gpu_s = ev / steps
        want = am_oracle.gemm_strided(alpha, A, B, beta, C_host.copy())
        cpu_s = cpu_time(lambda: am_oracle.gemm_strided(alpha, A, B, beta, C_host.copy() if beta != 0 else C_host))
        ops = 2.0 * M * N * K
        row = dict(config=config, shape=[M, N, K], gpu_ms=round(gpu_s * 1e3, 4),
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
                  peak_used="MFMA fp32 157.3 TFLOP/s", steps=200 if n <= 2048 else 20, warm=MATRIX_WARM_S if n <= 2048 else 0.05)
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
                      unit="Top/s", steps=20, spin=(SPIN_I8, 0.08))
            os.environ[env] = "valu"
            try:
                gemm_case(f"{sfx} GEMM {n}^3, entries in [-100, 100] (VALU kernel)", sfx, n, n, n, A, B,
                          am.toHip(A), am.toHip(B), peak=ceil.get(key),
                          peak_used=f"measured VALU {sfx} multiply-add ceiling {ceil.get(key)} Top/s", unit="Top/s", steps=10,
                          spin=(SPIN_VALU32 if sfx == "i32" else SPIN_VALU64, 0.08))
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
                  unit="Top/s", steps=10, spin=(SPIN_I8, 0.08))
    pa = rng(3001).standard_normal((1024, 2048)); pb = rng(3002).standard_normal((1024, 6144))
    C0 = rng(3003).standard_normal((2048, 3072))
    gemm_case("f64 gemm(1.5, A^T view, B[:, ::2] view, 0.5, C)", "f64", 2048, 3072, 1024, pa.T, pb[:, ::2],
              am.toHip(pa).transpose(), am.toHip(pb)[:, ::2], alpha=1.5, beta=0.5, C0=C0, peak=MFMA_F64_PEAK_TFLOPS,
              peak_used="MFMA fp64 78.6 TFLOP/s", steps=20, spin=(SPIN_F64, 0.1), warm=MATRIX_WARM_S)   # the entry's protocol (wl_gemm_f64_views)
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
        _, ev = timer.run(lambda: th._binary_into(op, dY, dX, bv), 50, 5)
        gpu_s = run_rotating(timer, [(lambda i=i: th._binary_into(op, dYs[i], dXs[i], bv)) for i in range(ROTATE)], 10)
        got = dYs[ROTATE - 1].toCpu().copy()
        hb = am_oracle.broadcast(hv, X.shape)
        out = np.empty_like(X)
        cpu_s = cpu_time(lambda: am_oracle.map2(op, X, hb, out=out))
        emit(config=f"f32 8192x8192 {name}", shape=[8192, 8192], gpu_ms=round(gpu_s * 1e3, 4),
             gpu_rate=round(nbytes / gpu_s / 1e9, 1), rate_unit="GB/s", pct_peak=round(100 * nbytes / gpu_s / 1e9 / HBM_PEAK_GBS, 1),
             peak_used="HBM 8000 GB/s", cpu_impl="oracle/strided_map.c (port of map2_inline + strided iteration, OpenMP blocks)",
             cpu_threads=threads, cpu_ms=round(cpu_s * 1e3, 2), speedup_vs_cpu=round(cpu_s / gpu_s, 1),
             bit_exact=bool(np.array_equal(got, out)), note=warm_note(ev / 50, nbytes))
    # (X +. b) *. s fused into one pass (same bytes moved once instead of twice)
    bb, sb = db.broadcast((8192, 8192)), ds.broadcast((8192, 8192))
    _, ev = timer.run(lambda: th._ternary_into("addmul", dY, dX, bb, sb), 50, 5)
    gpu_s = run_rotating(timer, [(lambda i=i: th._ternary_into("addmul", dYs[i], dXs[i], bb, sb)) for i in range(ROTATE)], 10)
    two_pass = ((X + b) * sc)
    emit(config="f32 8192x8192 (X +. b) *. s fused (one pass)", shape=[8192, 8192], gpu_ms=round(gpu_s * 1e3, 4),
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
        emit(config=f"f32 8192x8192 {name}", shape=[8192, 8192], gpu_ms=round(gpu_s * 1e3, 4),
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
        _, ev = timer.run(lambda: fn_gpu(inputs[0]), 50, 5)
        gpu_s = run_rotating(timer, [(lambda x=x: fn_gpu(x)) for x in inputs], 10)
        cpu_s = cpu_time(fn_cpu, budget=2.0)
        emit(config=config, gpu_ms=round(gpu_s * 1e3, 4), gpu_rate=round(nbytes / gpu_s / 1e9, 1), rate_unit="GB/s",
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
    r = wl_chain(ctx)
    emit(config="f32 inference chain (4 GEMMs, fused bias+ReLU)", hipgraph_us=r.get("hipgraph_us"), eager_us=r["eager_us"])
    r = wl_ex02(ctx)
    emit(config="f32 example-2 forward pass, batch 64 (6 kernels)", hipgraph_us=r.get("hipgraph_us"), eager_us=r["eager_us"])


# Order of the default line: the float32 / float64 matrix workloads first (the int8 chains of the ceilings and the
# digit-sliced products leave the chip at a lowered clock for a while), then the integer ones, then the rest.
DEFAULT_ORDER = ["gemm_f32_1024", "gemm_f32_2048", "gemm_f64", "gemm_f32_long_k",
                 "gemm_i32_1500", "gemm_i32", "gemm_i32_prepared", "gemm_i32_whole_range", "gemm_i64", "matmul_i64_1500_published",
                 "bcast_add_rotating", "bcast_mul_rotating", "bias_relu_rotating", "bcast_addmul_fused_rotating", "transposed_add",
                 "bias_short_rows", "sum_cols_narrow", "sum_rows_512", "chain", "ex02"]
# ... and the order they are printed in: by configuration
PRINT_ORDER = ["gemm_f32_1024", "gemm_f32_2048", "gemm_i32_1500", "gemm_i32", "gemm_i32_prepared", "gemm_i32_whole_range", "gemm_i64", "matmul_i64_1500_published",
               "gemm_f64", "bcast_add_rotating", "bcast_mul_rotating", "bias_relu_rotating", "bcast_addmul_fused_rotating", "chain",
               "ex02", "transposed_add", "bias_short_rows", "sum_cols_narrow", "sum_rows_512", "gemm_f32_long_k"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-others", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-graphs", action="store_true", help="time the small chains eagerly only: no HIP graph is captured or launched")
    ap.add_argument("--report", action="store_true",
                    help="print one JSON line per configuration (GPU vs CPU port, parity at full size) instead of the single benchmark line")
    ap.add_argument("--only", choices=sorted(WORKLOADS), help="run just this workload's entry of the line and print it (what the profiles trace)")
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
    ctx = Ctx(am, L, timer, args.steps, args.warmup, graphs=not args.no_graphs)

    if args.only:
        ctx.solo = True
        if args.only in ("gemm_i32_1500", "gemm_i32", "gemm_i64"):     # their VALU leg is priced against a measured ceiling
            ctx._ceilings = {}
        r = WORKLOADS[args.only][0](ctx)
        print(json.dumps(dict(only=args.only, steps=args.steps, warmup=args.warmup, timed_steps_of_each_run=timer.history,
                              entries=r if isinstance(r, list) else [r])))
        return
    if args.report:
        config_report(am, timer, L)
        return

    # The same W warm-up steps + K timed steps twice: straight from the idle device (`from_idle`: the shader
    # clock is still climbing then), and again right after 80 ms of register-only matrix-core work that is not
    # the workload (`value`: the clock the device holds under sustained load, printed beside it).
    idle = bench_gemm_f32(ctx, args.steps, args.warmup, spin=None)
    r = bench_gemm_f32(ctx, args.steps, args.warmup, host=idle["host"])
    tflops = r["flops"] * args.steps / r["wall"] / 1e12
    kern_tflops = r["flops"] / (r["ev"] / args.steps) / 1e12
    traffic, traffic_src = load_traffic("gemm_f32_4096")
    roof = mfma_roof(kern_tflops, MFMA_F32_PEAK_TFLOPS, r["sclk_mhz"], unit="TFLOP/s")
    roof.update(traffic=traffic, traffic_source=traffic_src)
    protocol = "per entry: MFMA spin, own launches (1 s if matrix-bound), K timed by HIP events; HBM-bound: rotating buffers"
    line = {
        "metric": "GEMM TFLOP/s (%MFMA peak) fp32/int32 4096^3; broadcast op HBM GB/s (%peak)",
        "value": round(tflops, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["wall"] / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "f32 GEMM C=A*B, M=N=K=4096, row-major, uniform[-1,1) seeds 1001/1002"},
        "roofline": roof,
        "from_idle": {"value": round(idle["flops"] * args.steps / idle["wall"] / 1e12, 3), "unit": "TFLOP/s",
                      "ms_per_step": round(idle["wall"] / args.steps * 1e3, 4), "sclk_mhz": idle["sclk_mhz"],
                      "what": "no spin or warm-up second first"},
        "device": info, "protocol": protocol,
    }
    if not args.no_others:
        results = {}
        for name in DEFAULT_ORDER:
            if name == "gemm_i32_1500":      # the first entry that needs them; after the float matrix workloads
                line["measured_ceilings"] = dict(ctx.ceilings, unit="T(FL)OP/s; *_tbs TB/s")
            results[name] = WORKLOADS[name][0](ctx)
            _C4.clear() if name == "transposed_add" else None
            _TALL.clear() if name == "sum_rows_512" else None
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_gemm_f32(*r["host"])
        line["cpu_blas_standin"] = cpu_blas_standin_gemm_f32(*r["host"])
    if not args.no_others:
        line["others"] = [e for name in PRINT_ORDER for e in (results[name] if isinstance(results[name], list) else [results[name]])]
    text = json.dumps(line, separators=(",", ":"))
    print(text)
    print(f"bench.py: line of {len(text)} characters", file=sys.stderr)


if __name__ == "__main__":
    main()
