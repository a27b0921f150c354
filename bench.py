#!/usr/bin/env python3
"""Benchmark of the BF16 GEMM path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg1..cfg5|m64|sq2048|mid|f8|f8n|f8s|f32|f64] [--kernel NAME]

A step is one launch of maize_hip_gemm_bf16 (maize_hip_gemm_bf16_ex for the 8-bit, fp32 and fp64
configurations) on synthetic, seeded inputs that are already resident in HBM.  Prints ONE JSON line:
whole-job TFLOP/s (wall clock around exactly K steps), the roofline object of the kernel (HIP events on
the launch stream) and the CPU oracle timed on a bounded slab of the same problem on this machine's host
cores.  The timed region follows a clock ramp (launches until the batch time settles) and W warm-up steps: it
is a hot-clock figure of a few milliseconds; --config energy measures the sustained one.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA, published
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published
# HBM-side bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs per workload), each scaled by what
# the same counter reads for a 256 MiB copy (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000).  These are figures of an earlier
# profiling session, not of this run: each entry names the kernel it was measured on and is reported only when this
# run's kernel is that one, together with its source file.
TRAFFIC_SOURCE = "profiles/hbm_traffic_fetch_write_size.md"
MEASURED_TRAFFIC = {"cfg1": ("maize_gemm_bf16_mt256_nn", 235.2e6), "cfg2": ("maize_gemm_bf16_mt256_nn_ragged", 239.4e6),
                    "cfg3": ("maize_gemm_bf16_mt256_nt", 1746.3e6), "cfg4": ("maize_gemm_bf16_skinny_nn", 126.5e6),
                    "m64": ("maize_gemm_bf16_skinny_nn_m64", 153.1e6),
                    "cfg5": ("maize_gemm_bf16_mt256_nn", 1074.3e6), "sq2048": ("maize_gemm_bf16_t128_nn", 58.9e6), "mid": ("maize_gemm_bf16_t128_nt", 109.2e6), "f8": ("maize_gemm_e4m3_mt256_nt", 134.5e6),
                    "f8n": ("maize_gemm_e4m3_mt256_nn", 134.5e6),
                    "f8mid": ("maize_gemm_e4m3_t128_nt", 58.9e6),
                    "f8s": ("maize_gemm_e4m3_skinny_nt", 67.2e6), "f32": ("maize_gemm_f32_mt128_nn", 828.9e6),
                    "f64": ("maize_gemm_f64_mt128_nn", 3162.3e6)}

# name -> (M, N, K, layout, batch, A distribution, B distribution, bound)
CONFIGS = {
    "cfg1": dict(m=4096, n=4096, k=4096, nt=0, batch=1, da=("uniform",), db=("uniform",), bound="mfma",
                 label="bf16 GEMM 4096x4096x4096 NN, uniform[-1,1)"),
    "cfg2": dict(m=4000, n=4104, k=4032, nt=0, batch=1, da=("uniform",), db=("uniform",), bound="mfma",
                 label="bf16 GEMM 4000x4104x4032 NN ragged, uniform[-1,1)"),
    "cfg3": dict(m=8192, n=8192, k=8192, nt=1, batch=1, da=("normal", "inv_sqrt_k"), db=("normal", "inv_sqrt_k"),
                 bound="mfma", label="bf16 GEMM 8192x8192x8192 NT, N(0,1)/sqrt(K)"),
    "cfg4": dict(m=16, n=14336, k=4096, nt=0, batch=1, da=("normal", 1.0), db=("normal", 0.02), bound="hbm",
                 label="bf16 GEMM 16x14336x4096 NN skinny, A~N(0,1), B~N(0,0.02)"),
    # cfg4's weights against 64 rows: the four-row-group version of the streaming kernel.
    "m64": dict(m=64, n=14336, k=4096, nt=0, batch=1, da=("normal", 1.0), db=("normal", 0.02), bound="hbm",
                label="bf16 GEMM 64x14336x4096 NN few rows, A~N(0,1), B~N(0,0.02)"),
    "cfg5": dict(m=2048, n=2048, k=2048, nt=0, batch=32, da=("uniform",), db=("uniform",), bound="mfma",
                 label="bf16 strided-batched GEMM 32 x 2048^3 NN, uniform[-1,1)"),
    # One product of cfg5's batch alone: 64 tiles of 256 x 256 on 256 compute units -- the dispatcher takes 128 x 256 tiles.
    "sq2048": dict(m=2048, n=2048, k=2048, nt=0, batch=1, da=("uniform",), db=("uniform",), bound="mfma",
                   label="bf16 GEMM 2048x2048x2048 NN, uniform[-1,1)"),
    # A prefill-sized product against a 4096 x 4096 weight stored N x K: 128 tiles of 128 x 256, 64 K steps -- the
    # three-stage form of the 128-row kernel.
    "mid": dict(m=1024, n=4096, k=4096, nt=1, batch=1, da=("normal", 1.0), db=("normal", 0.02), bound="mfma",
                label="bf16 GEMM 1024x4096x4096 NT, A~N(0,1), B~N(0,0.02)"),
    # Beside the five bf16 configurations: the same product on 8-bit operands (E4M3), both K-contiguous.
    "f8": dict(m=4096, n=4096, k=4096, nt=1, batch=1, da=("uniform",), db=("uniform",), bound="mfma", in_type="e4m3",
               label="E4M3 GEMM 4096x4096x4096 NT (bf16 C), uniform[-1,1) rounded to E4M3"),
    # ... with B stored K x N (row-major), read where it lies through transposing LDS reads.
    "f8n": dict(m=4096, n=4096, k=4096, nt=0, batch=1, da=("uniform",), db=("uniform",), bound="mfma", in_type="e4m3",
                label="E4M3 GEMM 4096x4096x4096 NN (bf16 C), uniform[-1,1) rounded to E4M3"),
    # ... and the decode-style shape of cfg4 against 8-bit weights stored N x K.
    "f8s": dict(m=16, n=14336, k=4096, nt=1, batch=1, da=("uniform",), db=("uniform",), bound="hbm", in_type="e4m3",
                label="E4M3 GEMM 16x14336x4096 NT skinny (bf16 C), uniform[-1,1) rounded to E4M3"),
    # ... and the 8-bit twin of "mid": a prefill of 1024 tokens against 8-bit 4096 x 4096 weights stored N x K.
    "f8mid": dict(m=1024, n=4096, k=4096, nt=1, batch=1, da=("uniform",), db=("uniform",), bound="mfma", in_type="e4m3",
                  label="E4M3 GEMM 1024x4096x4096 NT (bf16 C), uniform[-1,1) rounded to E4M3"),
    # The catalogue's fp32 and fp64 entries (v_mfma_f32_16x16x4_f32, v_mfma_f64_16x16x4_f64), C in the operands' type.
    "f32": dict(m=4096, n=4096, k=4096, nt=0, batch=1, da=("uniform",), db=("uniform",), bound="mfma", in_type="f32",
                label="fp32 GEMM 4096x4096x4096 NN (fp32 C), uniform[-1,1)"),
    "f64": dict(m=4096, n=4096, k=4096, nt=0, batch=1, da=("uniform",), db=("uniform",), bound="mfma", in_type="f64",
                label="fp64 GEMM 4096x4096x4096 NN (fp64 C), uniform[-1,1)"),
}
WIDE = {"f32": (np.float32, 157.3), "f64": (np.float64, 78.6)}     # element type, published dense MFMA peak in TFLOP/s


def make(mz, dist, count, seed, in_type=None):
    if in_type in WIDE:
        return (np.random.default_rng(seed).random(count) * 2 - 1).astype(WIDE[in_type][0])
    if in_type is not None:
        return mz.gen.uniform_f8(count, seed, mz.IN_E4M3 if in_type == "e4m3" else mz.IN_E5M2)
    if dist[0] == "uniform":
        return mz.gen.uniform_bf16(count, seed)
    sigma = mz.gen.SIGMA_INV_SQRT_8192 if dist[1] == "inv_sqrt_k" else dist[1]
    return mz.gen.normal_bf16(count, seed, sigma)


def cpu_baseline(cfg, a, b_storage, got, seconds_target=12.0):
    """Times the CPU oracle (fp64 accumulate, one RNE) on the first R rows of batch 0 and
    uses the same rows to check the device result.  The oracle is only the checker and
    the reported baseline here; it is never on the measured GPU path."""
    from oracle import pyoracle
    m, n, k = cfg["m"], cfg["n"], cfg["k"]
    if cfg.get("in_type") in WIDE:
        return cpu_baseline_wide(cfg, a, b_storage, got, seconds_target)
    elem = {None: pyoracle.BF16, "e4m3": pyoracle.E4M3, "e5m2": pyoracle.E5M2}[cfg.get("in_type")]
    coeff = pyoracle.floor_coeff_f8(k) if cfg.get("in_type") else None
    threads = pyoracle.default_threads()
    probe_rows = min(m, 4)
    t0 = time.perf_counter()
    pyoracle.ref_gemm_rows(a[:m * k], b_storage[:k * n], m, n, k, np.arange(probe_rows, dtype=np.uint32),
                           layout=cfg["nt"], want_abs=False, nthreads=1, elem=elem)
    per_row = max((time.perf_counter() - t0) / probe_rows, 1e-6)
    rows = int(min(m, max(threads, seconds_target * threads / per_row)))
    rows = max(1, (rows // threads) * threads) if rows >= threads else rows
    sel = np.arange(rows, dtype=np.uint32)
    t0 = time.perf_counter()
    ref, f64, _ = pyoracle.ref_gemm_rows(a[:m * k], b_storage[:k * n], m, n, k, sel, layout=cfg["nt"], want_abs=False,
                                         nthreads=threads, elem=elem)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * n * k
    out = {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
           "sample": f"rows 0..{rows - 1} of batch 0 ({rows}x{n}x{k}, {flops / 1e9:.1f} GFLOP, {dt:.1f} s), "
                     f"fp64 accumulate + one RNE to bf16, {threads} POSIX threads"}
    parity = None
    if got is not None:
        _, _, ab = pyoracle.ref_gemm_rows(a[:m * k], b_storage[:k * n], m, n, k, sel[:min(rows, 64)], layout=cfg["nt"],
                                          nthreads=threads, elem=elem)
        r = min(rows, 64)
        parity = pyoracle.compare(got[:r * n], ref[:r], f64[:r], ab, k, coeff=coeff)
        tight = pyoracle.tight_violations(parity) if coeff is None else None      # (16-bit operands: the bar below the floor)
        parity = {key: parity[key] for key in ("n", "max_ulp", "n_gt1ulp", "n_fail", "max_floor_ratio", "max_err_over_abs")}
        if tight is not None:
            parity.update({"gt1ulp_rate": parity["n_gt1ulp"] / max(1, parity["n"]), "gt1ulp_rate_bar": pyoracle.TIGHT_GT1ULP_RATE,
                           "max_floor_ratio_bar": pyoracle.floor_ratio_bar(k), "sums_as_accurate_as_fp32": not tight})
    return out, parity


def cpu_baseline_wide(cfg, a, b_storage, got, seconds_target):
    """The same for fp32 / fp64 operands: the oracle's long-double sums on the first R rows."""
    from oracle import pyoracle
    m, n, k = cfg["m"], cfg["n"], cfg["k"]
    threads = pyoracle.default_threads()
    t0 = time.perf_counter()
    pyoracle.ref_gemm_wide(a, b_storage, m, n, k, layout=cfg["nt"], rows=np.arange(2, dtype=np.uint32), nthreads=1)
    per_row = max((time.perf_counter() - t0) / 2, 1e-6)
    rows = int(min(m, max(threads, seconds_target * threads / per_row)))
    rows = max(1, (rows // threads) * threads) if rows >= threads else rows
    sel = np.arange(rows, dtype=np.uint32)
    t0 = time.perf_counter()
    hi, lo, ab = pyoracle.ref_gemm_wide(a, b_storage, m, n, k, layout=cfg["nt"], rows=sel, nthreads=threads)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * n * k
    out = {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
           "sample": f"rows 0..{rows - 1} ({rows}x{n}x{k}, {flops / 1e9:.1f} GFLOP, {dt:.1f} s), long-double products and sums "
                     f"(and sum|a||b| beside them), {threads} POSIX threads"}
    parity = None
    if got is not None:
        worst = pyoracle.check_wide(got.reshape(m, n)[:rows], hi, lo, ab, k)
        parity = {"n": int(rows * n), "worst_error_over_bound": worst, "n_fail": int(worst > 1.0),
                  "bound": "(K/4 + 4) * u * sum|a||b|, u = 2^-24 (fp32) / 2^-53 (fp64)"}
    return out, parity


def copy_calibration(steps, warmup):
    """Streams 256 MiB through maize_copy_u128 (one read + one write of every byte): the
    known-size copy that the FETCH_SIZE / WRITE_SIZE hardware counters are scaled against."""
    import ctypes as C
    import maize_amd as mz

    class CopyArgs(C.Structure):
        _fields_ = [("src", C.c_void_p), ("dst", C.c_void_p), ("n_vec", C.c_uint64)]

    nbytes = 256 * 2 ** 20
    ctx = mz.Context(0)
    src, dst = ctx.malloc(nbytes), ctx.malloc(nbytes)
    src.fill(0x5A)
    kern = mz.new_hip_kernel("maize_copy_u128").with_launch_bounds_1d(256).finalize().compile(mz.Gfx.Gfx950, ctx)
    args = CopyArgs(src.ptr, dst.ptr, nbytes // 16)
    grid = (ctx.info()["compute_units"] * 8, 1, 1)
    ev0, ev1 = ctx.event(), ctx.event()
    for _ in range(warmup):
        kern.launch(grid, args)
    ctx.sync()
    ev0.record(None)
    for _ in range(steps):
        kern.launch(grid, args)
    ev1.record(None)
    ctx.sync()
    us = ev0.elapsed_ms(ev1) / steps * 1e3
    print(json.dumps({"metric": "copy calibration", "kernel": "maize_copy_u128", "bytes_read": nbytes,
                      "bytes_written": nbytes, "kernel_avg_us": us, "value": 2 * nbytes / us / 1e3, "unit": "GB/s",
                      "steps": steps, "warmup": warmup}), flush=True)
    kern.release()
    src.free(); dst.free()
    ctx.close()


class PowerSampler:
    """Board power from sysfs (hwmon power1_input or power1_average, microwatts), sampled every 20 ms on a thread
    while the GPU works.  No GPU runtime call is made here."""

    def __init__(self, period=0.02):
        import glob
        self.period = period
        cands = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")) or \
            sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"))
        self.path = cands[0] if cands else None
        self.samples = []

    def read(self):
        try:
            with open(self.path) as f:
                return float(f.read().strip()) / 1e6
        except Exception:
            return None

    def __enter__(self):
        import threading
        self._stop = False

        def loop():
            while not self._stop:
                w = self.read()
                if w is not None:
                    self.samples.append((time.time(), w))
                time.sleep(self.period)
        self._t = threading.Thread(target=loop, daemon=True)
        self._t.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        self._t.join()

    def mean_between(self, t0, t1):
        w = [x for t, x in self.samples if t0 <= t <= t1]
        return sum(w) / len(w) if w else None

    def count_between(self, t0, t1):
        return sum(1 for t, _ in self.samples if t0 <= t <= t1)


CEILING_PROBES = {None: ("maize_probe_mfma_loop_16x16x32", 512, "v_mfma_f32_16x16x32_bf16"),
                  "e4m3": ("maize_probe_mfma_loop_16x16x128_e4m3", 128, "v_mfma_f32_16x16x128_f8f6f4 on E4M3")}


def box_ceiling(mz, ctx, stream, launches=50, in_type=None):
    """What this box's matrix pipe does right now with no data movement at all: a register-only loop of
    v_mfma_f32_16x16x32_bf16 on random operands, 256 workgroups x 4 waves x 512 rounds x 131072 multiply-adds = the
    multiply-adds of 4096^3 (E4M3 operands: v_mfma_f32_16x16x128_f8f6f4, 128 rounds x 524288), timed by HIP events on
    `stream` straight after the timed region (same clocks, same temperature).  A slow or hot box shows up here as a
    slow ceiling.  Returns microseconds per launch."""
    import ctypes as C

    class LoopArgs(C.Structure):
        _fields_ = [("out", C.c_void_p), ("iters", C.c_uint32), ("zero", C.c_uint32)]

    out = ctx.malloc(4096)
    probe, rounds, _ = CEILING_PROBES[in_type]
    kern = mz.new_hip_kernel(probe).with_launch_bounds_1d(256).finalize().compile(mz.Gfx.Gfx950, ctx)
    args = LoopArgs(out.ptr, rounds, 0)
    ev0, ev1 = ctx.event(), ctx.event()
    for _ in range(10):
        kern.launch((256, 1, 1), args, stream=stream)
    ev0.record(stream)
    for _ in range(launches):
        kern.launch((256, 1, 1), args, stream=stream)
    ev1.record(stream)
    ctx.sync()
    us = ev0.elapsed_ms(ev1) / launches * 1e3
    ev0.destroy(); ev1.destroy()
    kern.release()
    out.free()
    return us


def energy_vendor_child(seconds):
    """Child process of --config energy --vendor: times torch.matmul (the vendor library) on the 4096^3 workload, NN
    and NT, and prints one JSON line per row with wall-clock stamps for the parent's power samples."""
    import torch
    n = 4096
    import maize_amd as mz
    a = mz.gen.uniform_bf16(n * n, mz.gen.SEED_A)
    b = mz.gen.uniform_bf16(n * n, mz.gen.SEED_B)
    ta = torch.from_numpy(a.view(np.int16).reshape(n, n)).cuda().view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16).reshape(n, n)).cuda().view(torch.bfloat16)
    tbt = tb.t().contiguous()
    tc = torch.empty(n, n, dtype=torch.bfloat16, device="cuda")
    for label, fn in (("vendor library NN (torch.matmul(A, B))", lambda: torch.matmul(ta, tb, out=tc)),
                      ("vendor library NT (torch.matmul(A, Bt.T))", lambda: torch.matmul(ta, tbt.t(), out=tc))):
        t0, us = time.time(), 0.0
        while time.time() - t0 < seconds:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(50):
                fn()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / 50 * 1e3
        print(json.dumps({"kernel": label, "us": us, "t0": t0, "t1": time.time()}), flush=True)
        time.sleep(0.7)


def energy_table(seconds, vendor):
    """Power x time per launch for the 4096^3 workload: this library's NN and NT kernels, register-only loops of
    the two bf16 matrix instructions doing the same multiply-adds (zeros and random operands), and -- with
    --vendor -- the vendor library's kernels through torch.matmul.  Each row runs back to back for `seconds`;
    power is averaged over the last 60 % of that time, when clocks and power have settled.  One JSON line."""
    import ctypes as C
    import maize_amd as mz

    class LoopArgs(C.Structure):
        _fields_ = [("out", C.c_void_p), ("iters", C.c_uint32), ("zero", C.c_uint32)]

    n = 4096
    rows = []
    sampler = PowerSampler()
    if sampler.path is None:
        print("bench.py --config energy: no hwmon power file under /sys/class/drm", file=sys.stderr)
    if vendor:
        # The vendor library's kernels, for comparison only: torch.matmul in a child process (its HIP runtime and this
        # library's do not share a process), run before this process touches the GPU; power is sampled here.
        import subprocess
        with sampler:
            out = subprocess.run([sys.executable, os.path.abspath(__file__), "--config", "energy-vendor-child", "--seconds", str(seconds)],
                                 capture_output=True, text=True, timeout=120)
        if out.returncode != 0:
            print("bench.py --config energy: the vendor rows failed:\n" + out.stderr[-2000:], file=sys.stderr)
        for line in out.stdout.splitlines():
            if line.startswith("{"):
                r = json.loads(line)
                watts = sampler.mean_between(r["t0"] + 0.4 * (r["t1"] - r["t0"]), r["t1"])
                rows.append({"kernel": r["kernel"], "us_per_launch": r["us"], "watts": watts,
                             "mj_per_launch": None if watts is None else watts * r["us"] / 1e3})
                print(f"energy: {r['kernel']}: {r['us']:.1f} us, {watts} W", file=sys.stderr, flush=True)
        sampler.samples = []
    ctx = mz.Context(0)
    info = ctx.info()
    a = mz.gen.uniform_bf16(n * n, mz.gen.SEED_A)
    b = mz.gen.uniform_bf16(n * n, mz.gen.SEED_B)
    da, db, dbt, dc, dz = ctx.upload(a), ctx.upload(b), ctx.upload(np.ascontiguousarray(b.reshape(n, n).T)), ctx.malloc(2 * n * n), ctx.malloc(2 * n * n)
    dz.fill(0)
    out = ctx.malloc(4096)
    time.sleep(1.0)
    idle = sampler.read()

    def run(label, launch, batch=50):
        ev0, ev1 = ctx.event(), ctx.event()
        with sampler:
            t_begin = time.time()
            launches, ev_ms = 0, 0.0
            while time.time() - t_begin < seconds:
                ev0.record(None)
                for _ in range(batch):
                    launch()
                ev1.record(None)
                ctx.sync()
                ev_ms, launches = ev0.elapsed_ms(ev1), launches + batch       # the last batch: settled clocks
            t_end = time.time()
        us = ev_ms / batch * 1e3
        watts = sampler.mean_between(t_begin + 0.4 * (t_end - t_begin), t_end)
        rows.append({"kernel": label, "us_per_launch": us, "watts": watts, "mj_per_launch": None if watts is None else watts * us / 1e3,
                     "launches": launches})
        print(f"energy: {label}: {us:.1f} us, {watts} W", file=sys.stderr, flush=True)
        ev0.destroy(); ev1.destroy()
        time.sleep(0.7)                                           # let the board cool to the same starting point

    def gemm(dA, dB, nt):
        desc = mz.gemm_desc(mz.Matrix(dA, n, n), mz.Matrix(dB, n, n), mz.Matrix(dc, n, n), layout=nt)
        return lambda: ctx.gemm_bf16(desc)

    run("maize_gemm_bf16_mt256_nn, uniform[-1,1) operands", gemm(da, db, 0))
    run("maize_gemm_bf16_mt256_nt, uniform[-1,1) operands", gemm(da, dbt, 1))
    run("maize_gemm_bf16_mt256_nn, all-zero operands", gemm(dz, dz, 0))
    for name in ("maize_probe_mfma_loop_16x16x32", "maize_probe_mfma_loop_32x32x16"):
        k = mz.new_hip_kernel(name).with_launch_bounds_1d(256).finalize().compile(mz.Gfx.Gfx950, ctx)
        for zero in (0, 1):
            args = LoopArgs(out.ptr, 512, zero)                  # 256 workgroups x 4 waves x 512 rounds x 131072 MACs = 4096^3
            run(f"{name} (registers only, same multiply-adds), {'zeros' if zero else 'random operands'}",
                lambda: k.launch((256, 1, 1), args))
        k.release()
    flop = 2.0 * n ** 3
    for r in rows:
        r["frac_of_bf16_peak"] = flop / (r["us_per_launch"] * 1e-6) / 1e12 / PEAK_BF16_TFLOPS
    print(json.dumps({"metric": "energy per 4096^3 launch", "unit": "mJ", "idle_watts": idle, "power_file": sampler.path,
                      "seconds_per_row": seconds, "device": info, "rows": rows}), flush=True)
    for x in (da, db, dbt, dc, dz, out):
        x.free()
    ctx.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--config", default=None, choices=sorted(CONFIGS) + ["copy", "energy", "energy-vendor-child"],
                    help="cfg1..cfg5: a benchmark configuration; m64: 64x14336x4096; sq2048: 2048^3 (half a round of tiles); mid: 1024x4096x4096 N x K; f8, f8n, f8s: 4096^3 (B stored N x K, K x N) and 16x14336x4096 on E4M3 operands; f32, f64: 4096^3 on fp32 / fp64 operands; copy: the 256 MiB copy "
                         "used to scale HBM counters; energy: board power x time per 4096^3 launch for this library's kernels and register-only MFMA loops")
    ap.add_argument("--kernel", default=None, help="force a kernel by name (default: the dispatcher's choice)")
    ap.add_argument("--shape", default=None, help="M,N,K[,batch]: a bf16 product of that shape instead of a named configuration "
                                                   "(uniform[-1,1) operands; --layout says how B is stored)")
    ap.add_argument("--layout", default="nn", choices=["nn", "nt"], help="--shape: B stored K x N (nn) or N x K (nt)")
    ap.add_argument("--in-type", default="bf16", choices=["bf16", "e4m3", "e5m2"], help="--shape: element type of A and B")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--others", action=argparse.BooleanOptionalAction, default=None,
                    help="also measure the other benchmark configurations (shorter runs) and report them under "
                         "\"other_configs\" (default: on when no --config is given)")
    ap.add_argument("--seconds", type=float, default=2.5, help="--config energy: how long each row runs back to back")
    ap.add_argument("--vendor", action="store_true", help="--config energy: add the vendor library's kernels (needs torch)")
    ap.add_argument("--rotate", type=int, default=0,
                    help="number of distinct operand sets cycled through (0: enough to exceed the 256 MiB "
                         "last-level cache for the HBM-bound config, 1 otherwise)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (independent output tiles need no exchange step; "
              "every box here has one GPU) -- run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.others is None:
        args.others = args.config is None and args.kernel is None
    if args.shape:
        dims = [int(x) for x in args.shape.split(",")]
        m_, n_, k_ = dims[:3]
        batch_ = dims[3] if len(dims) > 3 else 1
        CONFIGS["custom"] = dict(m=m_, n=n_, k=k_, nt=int(args.layout == "nt"), batch=batch_, da=("uniform",), db=("uniform",), bound="mfma",
                                 label=f"{args.in_type} GEMM {'%d x ' % batch_ if batch_ > 1 else ''}{m_}x{n_}x{k_} {args.layout.upper()}, uniform[-1,1)")
        if args.in_type != "bf16":
            CONFIGS["custom"]["in_type"] = args.in_type
        args.config, args.others = "custom", False
    args.config = args.config or "cfg1"
    if args.config == "copy":
        copy_calibration(args.steps, args.warmup)
        return
    if args.config == "energy-vendor-child":
        energy_vendor_child(args.seconds)
        return
    if args.config == "energy":
        energy_table(args.seconds, args.vendor)
        return
    import maize_amd as mz
    ctx = mz.Context(0)
    probed = CONFIGS[args.config]['bound'] == 'mfma' and CONFIGS[args.config].get('in_type') in CEILING_PROBES
    line = measure(mz, ctx, args.config, args.steps, args.warmup, args.kernel, args.rotate, not args.no_cpu, ceiling=probed)
    if args.others:
        # The other benchmark configurations, shorter runs, same process: reported beside the headline.
        others = {}
        for name in sorted(CONFIGS):
            if name == args.config:
                continue
            o = measure(mz, ctx, name, max(20, args.steps // 4), max(10, args.warmup // 2), None, 0, False)
            others[name] = {"workload": o["config"]["workload"], "us_per_step": o["ms_per_step"] * 1e3, "value": o["value"],
                            "unit": o["unit"], "kernel": o["roofline"]["kernel"], "roofline_bound": o["roofline"]["bound"],
                            "roofline_frac": o["roofline"]["frac"], "steps": o["steps"], "kernel_avg_us": o["roofline"]["kernel_avg_us"],
                            "traffic": o["roofline"]["traffic"], "traffic_source": o["roofline"].get("traffic_source")}
        line["other_configs"] = others
    print(json.dumps(line), flush=True)
    ctx.close()


def measure(mz, ctx, config, steps, warmup, force_kernel, rotate, with_cpu, ceiling=False):
    """One configuration: untimed clock ramp and warm-up, then exactly `steps` launches timed by the wall
    clock (sync on both sides) and by HIP events on the launch stream.  Returns the JSON line as a dict."""
    class A:  # the names the body below was written against
        pass
    args = A()
    args.config, args.steps, args.warmup, args.kernel, args.rotate, args.no_cpu = config, steps, warmup, force_kernel, rotate, not with_cpu
    cfg = CONFIGS[args.config]
    m, n, k, batch, nt = cfg["m"], cfg["n"], cfg["k"], cfg["batch"], cfg["nt"]
    f8 = cfg.get("in_type")
    wide = f8 if f8 in WIDE else None                      # fp32 / fp64 operands: C has their type
    esz = np.dtype(WIDE[wide][0]).itemsize if wide else 1 if f8 else 2     # bytes per element of A and B
    csz = esz if wide else 2                               # ... and of C
    flops = 2.0 * batch * m * n * k
    alg_bytes = float(batch) * (esz * (m * k + k * n) + csz * m * n)

    a = make(mz, cfg["da"], batch * m * k, mz.gen.SEED_A, f8)
    b = make(mz, cfg["db"], batch * k * n, mz.gen.SEED_B, f8)
    if nt:  # same logical B, stored N x K
        b = np.concatenate([b[i * k * n:(i + 1) * k * n].reshape(k, n).T.ravel() for i in range(batch)])

    info = ctx.info()
    nsets = args.rotate or (max(2, int(np.ceil(3 * 256 * 2 ** 20 / alg_bytes))) if cfg["bound"] == "hbm" else 1)
    sets = []
    for _ in range(nsets):
        da, db, dc = ctx.upload(a), ctx.upload(b), ctx.malloc(csz * batch * m * n)
        A = mz.Matrix(da, m, k, elem_bytes=esz)
        B = mz.Matrix(db, n, k, elem_bytes=esz) if nt else mz.Matrix(db, k, n, elem_bytes=esz)
        if f8:
            desc = mz.gemm_ex_desc(A, B, mz.Matrix(dc, m, n, elem_bytes=csz), layout=nt, batch=batch, stride_a=m * k, stride_b=k * n,
                                   stride_c=m * n, in_type={"e4m3": mz.IN_E4M3, "e5m2": mz.IN_E5M2, "f32": mz.IN_F32, "f64": mz.IN_F64}[f8])
        else:
            desc = mz.gemm_desc(A, B, mz.Matrix(dc, m, n), layout=nt, batch=batch, stride_a=m * k, stride_b=k * n,
                                stride_c=m * n)
        sets.append((da, db, dc, desc))
    kernel = args.kernel or mz.gemm_plan(sets[0][3], compute_units=info["compute_units"])["kernel"]
    stream = ctx.stream()
    ev0, ev1 = ctx.event(), ctx.event()

    # Clock ramp (set-up, untimed): a fresh process starts at idle clocks and the first few
    # hundred launches run slower than the steady state.  Launch in batches until the batch time
    # settles (or 2 s have passed), then do the W warm-up steps proper.
    ramp_t0, prev, ramp_launches = time.perf_counter(), None, 0
    while time.perf_counter() - ramp_t0 < 2.0:
        ev0.record(stream)
        for i in range(50):
            ctx.gemm_bf16(sets[i % nsets][3], stream=stream, kernel=args.kernel)
        ev1.record(stream)
        ctx.sync()
        ramp_launches += 50
        cur = ev0.elapsed_ms(ev1)
        if prev is not None and ramp_launches >= 300 and abs(cur - prev) <= 0.01 * prev:
            break
        prev = cur
    for i in range(args.warmup):
        ctx.gemm_bf16(sets[i % nsets][3], stream=stream, kernel=args.kernel)
    ctx.sync()
    sampler = PowerSampler(period=0.001) if ceiling else None     # (sysfs reads on a host thread; no GPU call)
    if sampler is not None and sampler.path is not None:
        sampler.__enter__()
    wall_t0 = time.time()
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        ctx.gemm_bf16(sets[i % nsets][3], stream=stream, kernel=args.kernel)
    ev1.record(stream)
    ctx.sync()
    wall = time.perf_counter() - t0
    wall_t1 = time.time()
    ev_ms = ev0.elapsed_ms(ev1)
    # The box's own ceiling, straight behind the timed region: the same multiply-adds from registers only.
    ceiling_us = box_ceiling(mz, ctx, stream, in_type=cfg.get("in_type")) if ceiling else None
    if sampler is not None and sampler.path is not None:
        sampler.__exit__()

    got = sets[(args.steps - 1) % nsets][2].download(WIDE[wide][0] if wide else np.uint16, count=m * n)
    ms_per_step = wall * 1e3 / args.steps
    kern_ms = ev_ms / args.steps
    value = flops / (wall / args.steps) / 1e12
    peak_flops = WIDE[wide][1] if wide else PEAK_FP8_TFLOPS if f8 else PEAK_BF16_TFLOPS
    if cfg["bound"] == "mfma":
        ach = flops / (kern_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": ach, "peak": peak_flops, "unit": "TFLOP/s",
                "frac": ach / peak_flops, "traffic": None}
    else:
        ach = alg_bytes / (kern_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": ach, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": ach / PEAK_HBM_GBS,
                "traffic": None}
    profiled = MEASURED_TRAFFIC.get(args.config)
    if profiled and profiled[0] == kernel:
        roof["traffic"] = profiled[1]
        roof["traffic_source"] = f"{TRAFFIC_SOURCE} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE on {kernel}, an earlier session; not measured in this run)"
    roof["kernel"] = kernel
    roof["kernel_avg_us"] = kern_ms * 1e3
    if ceiling_us is not None:
        # the register-only loop does 4096^3 multiply-adds; scaled to this workload's
        scaled = ceiling_us * flops / (2.0 * 4096 ** 3)
        roof["box_ceiling_us"] = scaled
        roof["box_ceiling_frac_of_peak"] = flops / (scaled * 1e-6) / 1e12 / peak_flops
        roof["frac_of_box_ceiling"] = scaled / (kern_ms * 1e3)
        probe, _, what = CEILING_PROBES[cfg.get("in_type")]
        roof["box_ceiling_source"] = (f"{probe}: {what} from registers only, uniform random "
                                      "operands, the workload's multiply-adds, 50 launches straight after the timed region")
        watts = sampler.mean_between(wall_t0, wall_t1) if sampler.path else None
        roof["board_watts_timed_region"] = watts
        roof["board_watts_samples"] = sampler.count_between(wall_t0, wall_t1) if sampler.path else 0
    roof["algorithmic_flop"] = flops
    roof["algorithmic_bytes"] = alg_bytes

    cpu, parity = (None, None)
    if not args.no_cpu:
        cpu, parity = cpu_baseline(cfg, a, b, got)

    line = {
        "metric": "bf16 GEMM TFLOP/s at 4096^3 on 1 MI355X" if args.config == "cfg1"
                  else f"{'fp32' if wide == 'f32' else 'fp64'} GEMM TFLOP/s, {args.config}" if wide
                  else f"E4M3 GEMM TFLOP/s, {args.config}" if f8 else f"bf16 GEMM TFLOP/s, {args.config}",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": wide if wide else "fp8 (e4m3)" if f8 else "bf16", "data": "synthetic (seeded counter-based generators, inputs resident in HBM)",
        "config": {"workload": cfg["label"], "M": m, "N": n, "K": k, "batch": batch, "layout": "NT" if nt else "NN",
                   "accumulate": wide or "fp32", "output": wide or "bf16", "operand_sets_cycled": nsets,
                   "clock_ramp_launches": ramp_launches},
        (f"pct_of_mfma_{wide}_peak" if wide else "pct_of_mfma_fp8_peak" if f8 else "pct_of_mfma_bf16_peak"): 100.0 * flops / (wall / args.steps) / 1e12 / peak_flops,
        "roofline": roof, "cpu_baseline": cpu, "parity_vs_oracle": parity,
        "device": {"name": info["name"], "compute_units": info["compute_units"], "clock_khz": info["clock_khz"]},
    }
    for da, db, dc, _ in sets:
        da.free(); db.free(); dc.free()
    ev0.destroy(); ev1.destroy()
    ctx.stream_destroy(stream)
    return line




if __name__ == "__main__":
    main()
