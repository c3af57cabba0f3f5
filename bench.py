#!/usr/bin/env python3
"""Benchmark of the matmul hot path on one MI355X.

A "step" is one pass of the path over one synthetic batch: the forward GEMM
C = A·B and both backward GEMMs dA = dC·Bᵀ and dB = Aᵀ·dC at M = N = K = 8192 in
bf16 (fp32 accumulate, bf16 output), operands resident in HBM, transposes passed
as stride views.  Prints ONE JSON line: whole-step TFLOP/s as `value`, the
forward kernel's roofline fraction, a one-core CPU baseline on a bounded slab of
the same workload, and secondary figures (skinny GEMM GB/s, fp32 / fp64 GEMMs,
the config-2 MLP step) under `secondary`.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3, "f64": 78.6}     # MI355X dense MFMA
PEAK_HBM_GBS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "pmc_traffic_gemm_bf16_8192.md")


def forward_traffic(kernel):
    """HBM-side bytes per launch of the forward GEMM as the committed counter summary records them (its line
    `roofline.traffic: <bytes> (<kernel>)`), or None when the summary is absent or was taken from another kernel than
    the one this run dispatched: the figure is a counter reading, never a constant of this script."""
    try:
        import re
        m = re.search(r"roofline\.traffic:\s*([0-9.eE+]+)\s*\(([^)]+)\)", open(TRAFFIC_PROFILE).read())
    except OSError:
        return None
    if not m or m.group(2).strip() != kernel:
        return None
    return float(m.group(1))


def _bf16_bits(x32):
    """fp32 -> bf16 bit patterns, the reference's rounding (truncate + first dropped bit)."""
    w = np.ascontiguousarray(x32, dtype=np.float32).view(np.uint32)
    return ((w >> 16) + ((w >> 15) & 1)).astype(np.uint16)


def _normal_bf16(rng, shape):
    out = np.empty(shape, dtype=np.uint16)
    rows = shape[0]
    step = max(1, (1 << 22) // max(1, int(np.prod(shape[1:]))))
    for r0 in range(0, rows, step):
        out[r0:r0 + step] = _bf16_bits(rng.standard_normal((min(step, rows - r0),) + tuple(shape[1:]), dtype=np.float32))
    return out


def _time_launches(capi, fn, reps, warmup):
    """Average milliseconds per call of fn(), HIP events on the launch stream (host launch cost included)."""
    for _ in range(warmup):
        fn()
    e0, e1 = capi.Event(), capi.Event()
    capi.synchronize()
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_ms(e1) / reps


def _time_graph(capi, fn, reps, warmup, replays=5):
    """Average milliseconds per call of fn() with `reps` calls recorded into one HIP graph and replayed, so
    that short kernels are timed back to back on the device instead of at the pace Python can launch them."""
    fn()                                   # eager once: fills the allocation pool, sets kernel attributes
    capi.synchronize()
    stream = capi.Stream()
    with stream:
        with capi.Graph.capture() as graph:
            for _ in range(reps):
                fn()
        for _ in range(warmup):
            graph.launch()
        e0, e1 = capi.Event(), capi.Event()
        e0.record()
        for _ in range(replays):
            graph.launch()
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_ms(e1) / (reps * replays)
    return ms


def headline(capi, steps, warmup, n=8192, data="normal"):
    rng = np.random.default_rng(2)
    dt = capi.BF16
    if data == "normal":
        a, b, dc = (_normal_bf16(rng, (n, n)) for _ in range(3))
    elif data == "ints":
        a, b, dc = (_bf16_bits(rng.integers(-3, 4, (n, n)).astype(np.float32)) for _ in range(3))
    else:
        a, b, dc = (np.full((n, n), 0x3f80 if data == "ones" else 0, dtype=np.uint16) for _ in range(3))
    d_a, d_b, d_dc = (capi.DeviceBuffer.from_numpy(t) for t in (a, b, dc))
    d_c, d_da, d_db = (capi.DeviceBuffer(n * n * 2) for _ in range(3))
    rm, tr = (0, n, 1), (0, 1, n)            # row-major and transposed-view strides (batch, row, col)

    def fwd():
        capi.gemm(d_c.ptr, d_a.ptr, d_b.ptr, None, 1, n, n, n, rm, rm, rm, False, dt)

    def bwd_a():                              # dA = dC · Bᵀ
        capi.gemm(d_da.ptr, d_dc.ptr, d_b.ptr, None, 1, n, n, n, rm, tr, rm, False, dt)

    def bwd_b():                              # dB = Aᵀ · dC
        capi.gemm(d_db.ptr, d_a.ptr, d_dc.ptr, None, 1, n, n, n, tr, rm, rm, False, dt)

    kernels = (("fwd_nn", fwd), ("dA_nt", bwd_a), ("dB_tn", bwd_b))
    for _ in range(warmup):
        for _, fn in kernels:
            fn()
    capi.synchronize()
    # timed region: exactly `steps` steps; an event after every launch gives per-kernel durations
    marks = [capi.Event() for _ in range(steps * 3 + 1)]
    capi.synchronize()
    t0 = time.perf_counter()
    marks[0].record()
    for s in range(steps):
        for j, (_, fn) in enumerate(kernels):
            fn()
            marks[s * 3 + j + 1].record()
    marks[-1].synchronize()
    capi.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    total_ms = marks[0].elapsed_ms(marks[-1])
    per = {name: 0.0 for name, _ in kernels}
    for s in range(steps):
        for j, (name, _) in enumerate(kernels):
            per[name] += marks[s * 3 + j].elapsed_ms(marks[s * 3 + j + 1])
    per = {k: v / steps for k, v in per.items()}
    flops = 2.0 * n * n * n

    # spot parity inside the bench: sampled entries against float64 dot products
    c = d_c.to_numpy(np.uint16, (n, n))
    rows = np.array([0, 257, 4095, 8191]); cols = np.array([1, 300, 5000, 8190])
    a64 = (a[rows].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    b64 = (b[:, cols].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    ref = a64 @ b64
    got = (c[np.ix_(rows, cols)].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    err = float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30))
    if not err <= 2e-2:
        raise RuntimeError(f"bf16 8192^3 forward GEMM fails parity: sampled normwise error {err}")
    return {
        "ms_per_step": total_ms / steps, "wall_ms_per_step": wall_ms / steps,
        "tflops": 3 * flops / (total_ms / steps * 1e-3) / 1e12,
        "kernel_ms": per, "fwd_tflops": flops / (per["fwd_nn"] * 1e-3) / 1e12,
        "sampled_rel_err": err, "operands": (a, b),
        "kernel": capi.gemm_kernel_name(1, n, n, n, (n, 1), (n, 1), (n, 1), dt),
    }


def sustained(capi, seconds, data="normal", n=8192, period=0.2, dtype="bf16"):
    """The forward 8192^3 bf16 GEMM launched back to back for `seconds` while a second thread polls the machine's SMI
    tool (amd-smi, a separate process that opens no compute context) for the shader clock and the socket power: the figures that say whether
    the part runs against its power limit on these operand values.  Returns TFLOP/s over the whole interval with the
    mean / min / max of every quantity sampled."""
    import subprocess
    import threading
    rng = np.random.default_rng(2)
    dt = capi.BF16 if dtype == "bf16" else capi.F16
    to_bits = _bf16_bits if dtype == "bf16" else (lambda x: x.astype(np.float16).view(np.uint16))
    if data == "normal":
        a, b = (to_bits(rng.standard_normal((n, n)).astype(np.float32)) for _ in range(2))
    elif data == "ints":
        a, b = (to_bits(rng.integers(-3, 4, (n, n)).astype(np.float32)) for _ in range(2))
    else:
        a, b = (to_bits(np.full((n, n), 1.0 if data == "ones" else 0.0, dtype=np.float32)) for _ in range(2))
    d_a, d_b = (capi.DeviceBuffer.from_numpy(t) for t in (a, b))
    d_c = capi.DeviceBuffer(n * n * 2)
    rm = (0, n, 1)
    fwd = lambda: capi.gemm(d_c.ptr, d_a.ptr, d_b.ptr, None, 1, n, n, n, rm, rm, rm, False, dt)
    samples, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            try:
                txt = subprocess.run(["amd-smi", "metric", "-g", "0", "--power", "--clock", "--json"], capture_output=True, text=True, timeout=10).stdout
                doc = json.loads(txt)
                gpu = (doc.get("gpu_data") if isinstance(doc, dict) else doc)[0]
                row = {}
                power = gpu.get("power", {}).get("socket_power", {})
                if isinstance(power, dict) and isinstance(power.get("value"), (int, float)):
                    row["power_w"] = float(power["value"])
                clocks = [c["clk"]["value"] for name, c in gpu.get("clock", {}).items()
                          if name.startswith("gfx_") and isinstance(c, dict) and isinstance(c.get("clk", {}).get("value"), (int, float))]
                if clocks:
                    row["sclk_mhz"] = sum(clocks) / len(clocks)          # mean over the XCDs
                if row:
                    samples.append(row)
            except Exception:
                pass
            stop.wait(period)

    fwd(); capi.synchronize()
    stream = capi.Stream()
    reps = 25
    with stream:
        with capi.Graph.capture() as graph:
            for _ in range(reps):
                fwd()
        graph.launch(); capi.check(capi.lib().rp_hip_stream_synchronize(), "sync")
        th = threading.Thread(target=poll, daemon=True)
        th.start()
        time.sleep(0.3)
        e0, e1 = capi.Event(), capi.Event()
        launched, t0 = 0, time.perf_counter()
        e0.record()
        while time.perf_counter() - t0 < seconds:
            for _ in range(4):
                graph.launch()
            launched += 4 * reps
            capi.check(capi.lib().rp_hip_stream_synchronize(), "sync")      # keeps the queue a few graphs deep, not unbounded
        e1.record(); e1.synchronize()
        ms = e0.elapsed_ms(e1)
        stop.set(); th.join(timeout=6)
    out = {"dtype": dtype, "data": data, "seconds": round(ms * 1e-3, 2), "gemms": launched, "ms_per_gemm": ms / launched,
           "TFLOP/s": 2.0 * n ** 3 * launched / ms / 1e9, "smi_samples": len(samples)}
    busy = samples[2:] if len(samples) > 4 else samples               # the first polls may predate the clock ramp
    for key in ("sclk_mhz", "power_w"):
        vals = [r[key] for r in busy if key in r]
        if vals:
            out[key] = {"mean": round(sum(vals) / len(vals), 1), "min": min(vals), "max": max(vals)}
    return out


def cpu_baseline(a, b, target_s=15.0):
    """The reference's CPU path for the bf16 GEMM (functional/functional.c:986-1000: widen A and B to float32, the
    i-j-l loop of matmul_kernel_host_f32, narrow C) on a row slab of the 8192^3 GEMM, one core.  When the reference's
    own host kernel was compiled into oracle/_ref the loop is that code ("reference"); otherwise the oracle's
    restatement of it ("port").  Two rows are timed first and the slab is sized from them for about `target_s`
    seconds of CPU work (4 to 256 rows)."""
    import oracle
    n = b.shape[0]
    ref = oracle.load_reference()

    def run(slab):
        if ref is None:
            return oracle.matmul(slab, b, oracle.BF16)              # widens B to fp32 once per call, as the reference does
        c32 = oracle.reference_matmul(ref, oracle.widen(slab, oracle.BF16), oracle.widen(b, oracle.BF16), oracle.F32)
        return oracle.narrow(c32, oracle.BF16)

    t0 = time.perf_counter()
    run(np.ascontiguousarray(a[:2]))
    probe = time.perf_counter() - t0
    rows = int(min(256, max(4, round(target_s / (probe / 2)))))
    slab = np.ascontiguousarray(a[:rows])
    t0 = time.perf_counter()
    run(slab)
    dt = time.perf_counter() - t0
    flops = 2.0 * rows * n * n
    what = "the reference's matmul_kernel_host_f32 compiled from its own source" if ref is not None else "the oracle's restatement of the reference loop"
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "reference" if ref is not None else "port",
            "sample": f"{rows} of {n} rows of the bf16 {n}^3 forward GEMM ({what}; fp32 pivot, i-j-l loop), {dt:.1f} s; "
                      f"host has {os.cpu_count()} logical cores"}


def cpu_baseline_configs():
    """The same CPU path on the other configurations, one core, each bounded to a second or two: configuration 1
    (fp32 Linear forward), configuration 2 (the nine fp32 GEMMs of the MLP step), configuration 3 at N = 1024 (bf16,
    a 256-row slab) and at N = 4096 (bf16 and fp32, an 8-row slab, the whole GEMM extrapolated), configuration 4 as a
    loop of per-head 2-D products (2 of the 192 heads, extrapolated), 5a (bf16, m = 1 against the 8192 x 8192 matrix)
    and 5b (fp64 2048^2, a 32-row slab).
    fp32 / fp64 products run in the reference's own matmul_kernel_host_* when oracle/_ref holds it, 16-bit ones
    and everything else in the oracle's restatement."""
    import oracle
    ref = oracle.load_reference()
    rng = np.random.default_rng(6)

    def mm(a, b, dt):
        if ref is not None and dt in (oracle.F32, oracle.F64):
            return oracle.reference_matmul(ref, a, b, dt)
        return oracle.matmul(a, b, dt)

    def timed(shapes, dt, npdt, whole=1.0):
        """`whole`: how many times the timed slab fits into the configuration; above 1 the full time is an extrapolation
        (the loop's cost is linear in the rows of A and in the number of per-head products)."""
        if dt == oracle.BF16:
            ops = [(_normal_bf16(rng, (m, k)), _normal_bf16(rng, (k, n))) for m, k, n in shapes]
        else:
            ops = [(rng.standard_normal((m, k)).astype(npdt), rng.standard_normal((k, n)).astype(npdt)) for m, k, n in shapes]
        t0 = time.perf_counter()
        for x, y in ops:
            mm(x, y, dt)
        sec = time.perf_counter() - t0
        out = {"ms": round(sec * 1e3, 2), "GFLOP/s": round(sum(2.0 * m * k * n for m, k, n in shapes) / sec / 1e9, 3)}
        if whole != 1.0:
            out["extrapolated_whole_config_ms"] = round(sec * 1e3 * whole, 1)
        return out

    mlp = []
    for rows, fan_in, fan_out in ((256, 784, 256), (256, 256, 128), (256, 128, 10)):
        mlp += [(rows, fan_in, fan_out), (rows, fan_out, fan_in), (fan_in, rows, fan_out)]          # forward, dX, dW
    out = {
        "config1_linear_fwd_f32": timed([(128, 784, 256)], oracle.F32, np.float32),
        "config2_mlp_9_gemms_f32": timed(mlp, oracle.F32, np.float32),
        "config3_bf16_1024_rows_0_255": timed([(256, 1024, 1024)], oracle.BF16, np.float32),
        # N = 4096: 8 of the 4096 rows of one GEMM (forward; dA and dB cost the same)
        "config3_bf16_4096_rows_0_7": timed([(8, 4096, 4096)], oracle.BF16, np.float32, whole=512.0),
        "config3_f32_4096_rows_0_7": timed([(8, 4096, 4096)], oracle.F32, np.float32, whole=512.0),
        # configuration 4 as the reference would run it: op_matmul is 2-D only (ops/ops.c:6818), so a loop of per-head
        # products; 2 of the 192 heads, S = Q.K^T on a densified K^T and O = P.V (the four backward GEMMs cost twice that again)
        "config4_bf16_2_heads_fwd": timed([(512, 64, 512), (512, 512, 64)] * 2, oracle.BF16, np.float32, whole=96.0),
        "config4_f32_2_heads_fwd": timed([(512, 64, 512), (512, 512, 64)] * 2, oracle.F32, np.float32, whole=96.0),
        "config5a_bf16_m1": timed([(1, 8192, 8192)], oracle.BF16, np.float32),           # the loop is linear in m: m = 8 and 32 take 8 and 32 times as long
        "config5b_f64_2048_rows_0_31": timed([(32, 2048, 2048)], oracle.F64, np.float64),
    }
    out["kind"] = "reference for fp32/fp64, port for bf16" if ref is not None else "port"
    out["cores"] = 1
    return out


def skinny_times(capi, quick_reps=20, rows=(1, 8, 16, 32), weights=8):
    """Config 5a: bf16 A[m, 8192] x W[8192, 8192], replayed from a HIP graph; bytes are A, W and the output once.

    `us` replays the product with one W, the first one the process streams.  How fast a W streams depends on more than
    the kernel: the same launch takes 21.4 - 22.0 us (m = 1, 8) on the first W a process streams and 23.1 - 23.2 us on
    every W used after it, a fixed 1.2 us at the start of each launch whatever the size of W and whichever allocation
    it is; the first W loses the advantage when other large transfers or GEMMs run in between.  Re-reading the same
    134 MB every launch also saves about 0.5 us against reading a different W each time.  `us_weights_in_turn` is the
    launch with `weights` different W's in turn (1 GB in all, more than any cache holds): what a caller that walks
    through many weight matrices sees."""
    out = {}
    rng = np.random.default_rng(4)
    k = n = 8192
    w = _normal_bf16(rng, (k, n))
    d_ws = [capi.DeviceBuffer.from_numpy(w) for _ in range(max(1, weights))]
    d_w = d_ws[0]
    for m in rows:
        a = _normal_bf16(rng, (m, k))
        d_a = capi.DeviceBuffer.from_numpy(a); d_y = capi.DeviceBuffer(m * n * 2)
        product = lambda d_b: capi.gemm(d_y.ptr, d_a.ptr, d_b.ptr, None, 1, m, k, n, (0, k, 1), (0, n, 1), (0, n, 1), False, capi.BF16)
        ms = _time_graph(capi, lambda: product(d_w), quick_reps, 2)
        nbytes = (m * k + k * n + m * n) * 2
        row = {"us": ms * 1e3, "GB/s": nbytes / (ms * 1e-3) / 1e9, "frac_hbm": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
               "kernel": capi.gemm_kernel_name(1, m, k, n, (k, 1), (n, 1), (n, 1), capi.BF16)}
        if len(d_ws) > 1:
            turn = [0]
            def next_weight():
                product(d_ws[turn[0] % len(d_ws)]); turn[0] += 1
            reps = (quick_reps + len(d_ws) - 1) // len(d_ws) * len(d_ws)          # every W equally often
            ms_turn = _time_graph(capi, next_weight, reps, 2)
            row["us_weights_in_turn"] = ms_turn * 1e3
            row["frac_hbm_weights_in_turn"] = nbytes / (ms_turn * 1e-3) / 1e9 / PEAK_HBM_GBS
        out[f"skinny_bf16_m{m}"] = row
    return out


def wide_times(capi, cases=(("gemm_f32_4096", "f32", 4096), ("gemm_f64_2048", "f64", 2048))):
    """Config 3's fp32 GEMM at 4096 and config 5b's fp64 GEMM at 2048 (square, row-major, N(0,1))."""
    out = {}
    rng = np.random.default_rng(5)
    for name, which, size in cases:
        dt, npdt, peak = (capi.F32, np.float32, PEAK_TFLOPS["f32"]) if which == "f32" else (capi.F64, np.float64, PEAK_TFLOPS["f64"])
        draw = (lambda: rng.standard_normal((size, size))) if which == "f32" else (lambda: rng.uniform(-1.0, 1.0, (size, size)))     # as the configurations say
        a = draw().astype(npdt); b = draw().astype(npdt)
        d_a, d_b = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
        d_c = capi.DeviceBuffer(a.nbytes)
        s = (0, size, 1)
        fn = lambda: capi.gemm(d_c.ptr, d_a.ptr, d_b.ptr, None, 1, size, size, size, s, s, s, False, dt)
        ms = _time_launches(capi, fn, 10, 3)
        tf = 2.0 * size ** 3 / (ms * 1e-3) / 1e12
        out[name] = {"ms": ms, "TFLOP/s": tf, "frac_mfma": tf / peak}
    return out


def f16_time(capi, n=8192):
    """Config 3 in fp16 at N = 8192: the forward GEMM (fp32 accumulate, fp16 output), N(0,1) operands."""
    rng = np.random.default_rng(2)
    a = rng.standard_normal((n, n)).astype(np.float16).view(np.uint16); b = rng.standard_normal((n, n)).astype(np.float16).view(np.uint16)
    d_a, d_b = capi.DeviceBuffer.from_numpy(a), capi.DeviceBuffer.from_numpy(b)
    d_c = capi.DeviceBuffer(a.nbytes)
    s = (0, n, 1)
    ms = _time_launches(capi, lambda: capi.gemm(d_c.ptr, d_a.ptr, d_b.ptr, None, 1, n, n, n, s, s, s, False, capi.F16), 60, 15)       # as many launches as the headline times
    tf = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
    for d in (d_a, d_b, d_c):
        d.free()
    return {"ms": ms, "TFLOP/s": tf, "frac_mfma": tf / PEAK_TFLOPS["f16"]}


def square_sweep(capi, sizes=(1024, 4096)):
    """Config 3 below the headline size: C = A.B, dA = dC.Bt, dB = At.dC (transposes as stride views) in bf16 and
    fp16 at N = 1024 and 4096, each replayed from a HIP graph; microseconds, TFLOP/s and the fraction of the MFMA peak."""
    out = {}
    rng = np.random.default_rng(2)
    for n in sizes:
        for name, dt in (("bf16", capi.BF16), ("f16", capi.F16)):
            mk = (lambda: _normal_bf16(rng, (n, n))) if dt == capi.BF16 else (lambda: rng.standard_normal((n, n)).astype(np.float16).view(np.uint16))
            d_a, d_b, d_dc = (capi.DeviceBuffer.from_numpy(mk()) for _ in range(3))
            d_c = capi.DeviceBuffer(n * n * 2)
            s, st = (0, n, 1), (0, 1, n)
            ops = {"fwd": lambda: capi.gemm(d_c.ptr, d_a.ptr, d_b.ptr, None, 1, n, n, n, s, s, s, False, dt),
                   "dA": lambda: capi.gemm(d_c.ptr, d_dc.ptr, d_b.ptr, None, 1, n, n, n, s, st, s, False, dt),
                   "dB": lambda: capi.gemm(d_c.ptr, d_a.ptr, d_dc.ptr, None, 1, n, n, n, st, s, s, False, dt)}
            _time_graph(capi, ops["fwd"], 10, 2)            # clocks up before the first figure
            row = {}
            for op, fn in ops.items():
                ms = _time_graph(capi, fn, 10, 2)
                tf = 2.0 * n ** 3 / ms / 1e9
                row[op] = {"us": round(ms * 1e3, 1), "TFLOP/s": round(tf, 1), "frac_mfma": round(tf / PEAK_TFLOPS[name], 3)}
            out[f"{name}_{n}"] = row
            for d in (d_a, d_b, d_dc, d_c):
                d.free()
    return out


def secondary(capi, quick_reps=20):
    out = skinny_times(capi, quick_reps)
    out["square_sweep"] = square_sweep(capi)
    out["gemm_f16_8192"] = f16_time(capi)
    out.update(wide_times(capi))
    # config 4: attention-shaped batched GEMMs on stride views
    out["attention_bf16"] = attention_times(capi, "bf16")
    out["attention_f32"] = attention_times(capi, "f32")
    # conv2d (the next caller of the GEMM): ResNet-style 3x3 layer, every launch of forward + backward
    out["conv2d_bf16"] = conv2d_times(capi, "bf16")
    out["conv2d_f32"] = conv2d_times(capi, "f32")
    # an LSTM step (the last caller of the GEMM on the list): small GEMMs bound by the weights' bytes and by launches
    out["lstm_step_bf16"] = lstm_step_times(capi, "bf16")
    out["lstm_step_f32"] = lstm_step_times(capi, "f32")
    # config 2: fp32 MLP 784-256-128-10, batch 256, forward + backward through the C ABI (9 GEMMs + neighbours)
    out["mlp_f32_step"] = mlp_step_time(capi)
    out["mlp_f32_step"]["ms_separate_launches"] = mlp_step_time(capi, fused_backward=False)["ms"]
    out["mlp_f32_step"]["ms_through_python_api"] = mlp_step_time_dropin()
    return out


def memory_ceilings(capi, sizes_mb=(64, 128, 200, 256, 384, 512, 1024, 2048)):
    """What the memory system gives plain streaming kernels of this library at a given footprint: rp_hip_fill (stores
    only), rp_hip_channel_sums over 1024 contiguous runs (loads only) and rp_hip_convert fp32 -> fp32 (one load per store).
    Up to the 256 MB of the memory-side cache repeated passes over the same buffer never reach HBM; beyond it they do."""
    L = capi.lib()
    out = {}
    for mb in sizes_mb:
        n = mb * (1 << 20) // 4
        a, b, red = capi.DeviceBuffer(n * 4), capi.DeviceBuffer(n * 4), capi.DeviceBuffer(1024 * 4)
        capi.check(L.rp_hip_fill(a.ptr, 1.0, n, capi.F32), "fill")
        reps = max(3, min(20, 4096 // mb))
        t_fill = _time_launches(capi, lambda: capi.check(L.rp_hip_fill(b.ptr, 2.0, n, capi.F32), "fill"), reps, 2)
        t_read = _time_launches(capi, lambda: capi.check(L.rp_hip_channel_sums(red.ptr, a.ptr, 1, 1024, n // 1024, 0, capi.F32), "channel_sums"), reps, 2)
        t_copy = _time_launches(capi, lambda: capi.check(L.rp_hip_convert(b.ptr, capi.F32, a.ptr, capi.F32, n), "convert"), reps, 2)
        out[f"{mb}MB"] = {"store_us": round(t_fill * 1e3, 1), "store_GB/s": round(n * 4 / t_fill / 1e6), "load_us": round(t_read * 1e3, 1),
                          "load_GB/s": round(n * 4 / t_read / 1e6), "copy_us": round(t_copy * 1e3, 1), "copy_GB/s_load_plus_store": round(2 * n * 4 / t_copy / 1e6)}
        for d in (a, b, red):
            d.free()
    return out


def attention_times(capi, dt_name="bf16"):
    """Config 4: Q, K, V [16*12, 512, 64]; S = Q·Kᵀ (Kᵀ a stride view), P = softmax(S/8), O = P·V, and the four
    backward GEMMs, each timed on its own from a HIP graph.  GEMM bytes are A, B and C once."""
    rng = np.random.default_rng(3)
    Z, S, D = 16 * 12, 512, 64
    dt = {"bf16": capi.BF16, "f32": capi.F32}[dt_name]
    esz = 2 if dt == capi.BF16 else 4
    mk = (lambda shape: _normal_bf16(rng, shape)) if dt == capi.BF16 else (lambda shape: rng.standard_normal(shape).astype(np.float32))
    D_ = capi.DeviceBuffer
    d_q, d_k, d_v, d_do = (D_.from_numpy(mk((Z, S, D))) for _ in range(4))
    d_s, d_ss, d_p, d_dp, d_dss = (D_(Z * S * S * esz) for _ in range(5))
    d_o, d_dq, d_dk, d_dv = (D_(Z * S * D * esz) for _ in range(4))
    sd, ss = S * D, S * S
    L = capi.lib()
    import ctypes
    scale = (ctypes.c_float * 1)(0.125)              # scalars travel as float for every dtype but float64
    ops = {
        "S=Q.Kt": (lambda: capi.gemm(d_s.ptr, d_q.ptr, d_k.ptr, None, Z, S, D, S, (sd, D, 1), (sd, 1, D), (ss, S, 1), False, dt), 2.0 * Z * S * S * D, (2 * sd + ss) * Z * esz),
        "scale": (lambda: capi.check(L.mul_scalar_kernel_device(d_ss.ptr, d_s.ptr, scale, Z * ss, dt), "mul_scalar"), 0.0, 2 * ss * Z * esz),
        "softmax": (lambda: capi.check(L.softmax_kernel_device(d_p.ptr, d_ss.ptr, Z * S, S, 1, dt), "softmax"), 0.0, 2 * ss * Z * esz),
        "O=P.V": (lambda: capi.gemm(d_o.ptr, d_p.ptr, d_v.ptr, None, Z, S, S, D, (ss, S, 1), (sd, D, 1), (sd, D, 1), False, dt), 2.0 * Z * S * S * D, (2 * sd + ss) * Z * esz),
        "dP=dO.Vt": (lambda: capi.gemm(d_dp.ptr, d_do.ptr, d_v.ptr, None, Z, S, D, S, (sd, D, 1), (sd, 1, D), (ss, S, 1), False, dt), 2.0 * Z * S * S * D, (2 * sd + ss) * Z * esz),
        "dV=Pt.dO": (lambda: capi.gemm(d_dv.ptr, d_p.ptr, d_do.ptr, None, Z, S, S, D, (ss, 1, S), (sd, D, 1), (sd, D, 1), False, dt), 2.0 * Z * S * S * D, (2 * sd + ss) * Z * esz),
        "softmax_bwd": (lambda: capi.check(L.backwards_softmax_device(d_dp.ptr, d_p.ptr, d_dss.ptr, Z * S, S, 1, dt), "backwards_softmax"), 0.0, 3 * ss * Z * esz),
        "dQ=dS.K": (lambda: capi.gemm(d_dq.ptr, d_dss.ptr, d_k.ptr, None, Z, S, S, D, (ss, S, 1), (sd, D, 1), (sd, D, 1), False, dt), 2.0 * Z * S * S * D, (2 * sd + ss) * Z * esz),
        "dK=dSt.Q": (lambda: capi.gemm(d_dk.ptr, d_dss.ptr, d_q.ptr, None, Z, S, S, D, (ss, 1, S), (sd, D, 1), (sd, D, 1), False, dt), 2.0 * Z * S * S * D, (2 * sd + ss) * Z * esz),
    }
    for fn, _, _ in ops.values():        # eager once, in dependency order, so every buffer holds finite values
        fn()
    kn = lambda m, k, n, a_rc, b_rc: capi.gemm_kernel_name(Z, m, k, n, a_rc, b_rc, (n, 1), dt)
    gemm_names = {"S=Q.Kt": kn(S, D, S, (D, 1), (1, D)), "dP=dO.Vt": kn(S, D, S, (D, 1), (1, D)), "O=P.V": kn(S, S, D, (S, 1), (D, 1)),
                  "dQ=dS.K": kn(S, S, D, (S, 1), (D, 1)), "dV=Pt.dO": kn(S, S, D, (1, S), (D, 1)), "dK=dSt.Q": kn(S, S, D, (1, S), (D, 1))}
    out, total = {}, 0.0
    for _ in range(300):                 # the clock the power management grants settles within some tens of milliseconds of load
        ops["S=Q.Kt"][0]()
    for name, (fn, flops, nbytes) in ops.items():
        ms = _time_graph(capi, fn, 10, 2)
        total += ms
        out[name] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 3)}
        if flops:
            out[name]["TFLOP/s"] = round(flops / ms / 1e9, 1)
            out[name]["frac_mfma"] = round(flops / ms / 1e9 / PEAK_TFLOPS[dt_name], 3)       # these GEMMs sit near the ridge: both fractions are given
            out[name]["kernel"] = gemm_names[name]
    # The scalar multiply and the softmax next to it as one pass each way (rp_hip_scaled_softmax and its gradient: the bits
    # of the two ops, the scaled tensor neither written nor re-read), which is how the drop-in runs `s.op_mul_scalar(c).op_softmax()`
    fused_ops = {
        "scale+softmax": (lambda: capi.check(L.rp_hip_scaled_softmax(d_p.ptr, d_s.ptr, scale, Z * S, S, 1, dt), "scaled_softmax"), 2 * ss * Z * esz),
        "softmax_bwd+scale": (lambda: capi.check(L.rp_hip_backwards_scaled_softmax(d_dp.ptr, d_p.ptr, d_dss.ptr, scale, Z * S, S, 1, dt), "backwards_scaled_softmax"), 3 * ss * Z * esz),
    }
    for name, (fn, nbytes) in fused_ops.items():
        ms = _time_graph(capi, fn, 10, 2)
        out[name] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 3)}
    out["fwd_bwd_ms_separate_scale"] = round(total + out["scale"]["us"] * 1e-3, 4)     # every reference op its own launch; the scale runs twice (S/8 and dS/8)
    gemms = sum(out[k]["us"] for k in ("S=Q.Kt", "O=P.V", "dP=dO.Vt", "dV=Pt.dO", "dQ=dS.K", "dK=dSt.Q"))
    out["fwd_bwd_ms"] = round((gemms + out["scale+softmax"]["us"] + out["softmax_bwd+scale"]["us"]) * 1e-3, 4)
    # the same forward (S, scale, softmax, O) as one fused kernel that never writes S or P
    fused = lambda: capi.check(L.rp_hip_attention_forward(d_o.ptr, d_q.ptr, d_k.ptr, d_v.ptr, None, Z, S, S, D,
                                                          sd, D, sd, D, sd, D, sd, D, 0.125, dt), "rp_hip_attention_forward")
    ms = _time_graph(capi, fused, 10, 2)
    chain = sum(out[k]["us"] for k in ("S=Q.Kt", "scale+softmax", "O=P.V"))
    nbytes = 4 * sd * Z * esz
    out["fused_forward"] = {"us": round(ms * 1e3, 1), "unfused_chain_us": round(chain, 1), "TFLOP/s": round(4.0 * Z * S * S * D / ms / 1e9, 1),
                            "GB/s": round(nbytes / ms / 1e6, 1)}
    # and the backward (dQ, dK, dV from Q, K, V, O, dO and the saved row statistics) as two launches
    d_lse = D_(Z * S * 4)
    capi.check(L.rp_hip_attention_forward(d_o.ptr, d_q.ptr, d_k.ptr, d_v.ptr, d_lse.ptr, Z, S, S, D, sd, D, sd, D, sd, D, sd, D, 0.125, dt), "rp_hip_attention_forward")
    fused_b = lambda: capi.check(L.rp_hip_attention_backward(d_dq.ptr, d_dk.ptr, d_dv.ptr, d_q.ptr, d_k.ptr, d_v.ptr, d_o.ptr, d_do.ptr, d_lse.ptr,
                                                             Z, S, S, D, sd, D, sd, D, sd, D, sd, D, sd, D, 0.125, dt), "rp_hip_attention_backward")
    fused_b()
    msb = _time_graph(capi, fused_b, 10, 2)
    chain_b = out["fwd_bwd_ms"] * 1e3 - chain
    out["fused_backward"] = {"us": round(msb * 1e3, 1), "unfused_chain_us": round(chain_b, 1), "TFLOP/s": round(10.0 * Z * S * S * D / msb / 1e9, 1)}
    out["fused_fwd_bwd_ms"] = round(ms + msb, 4)
    return out


def conv2d_times(capi, dt_name="bf16"):
    """A ResNet-style 3x3 layer (N 64, 64 -> 64 channels, 56 x 56, padding 1) lowered onto the batched GEMM: every
    launch of the forward and backward timed on its own from a HIP graph.  Lowering bytes are read + written once."""
    rng = np.random.default_rng(4)
    N, C, H, W, Co, k, pad = 64, 64, 56, 56, 64, 3, 1
    dt = {"bf16": capi.BF16, "f32": capi.F32}[dt_name]
    esz = 2 if dt == capi.BF16 else 4
    mk = (lambda shape: _normal_bf16(rng, shape)) if dt == capi.BF16 else (lambda shape: rng.standard_normal(shape).astype(np.float32))
    D_ = capi.DeviceBuffer
    rows, cols = C * k * k, H * W
    x_n, y_n, col_n = C * H * W, Co * cols, rows * cols
    d_x, d_w, d_b, d_dy = D_.from_numpy(mk((N, C, H, W))), D_.from_numpy(mk((Co, rows))), D_.from_numpy(mk((Co,))), D_.from_numpy(mk((N, Co, cols)))
    d_col, d_y, d_dx = D_(N * col_n * esz), D_(N * y_n * esz), D_(N * x_n * esz)
    d_dws, d_dw, d_db = D_(N * Co * rows * esz), D_(Co * rows * esz), D_(Co * esz)
    L = capi.lib()
    geom = (C, H, W, k, k, 1, 1, pad, pad, 1, 1, H, W)
    gemm_flops = 2.0 * N * Co * rows * cols
    ops = {
        "im2col": (lambda: capi.check(L.rp_hip_im2col_batched(d_col.ptr, d_x.ptr, N, *geom, dt), "im2col"), 0.0, N * (x_n + col_n) * esz),
        "y=W.col": (lambda: capi.gemm(d_y.ptr, d_w.ptr, d_col.ptr, None, N, Co, rows, cols, (0, rows, 1), (col_n, cols, 1), (y_n, cols, 1), False, dt),
                    gemm_flops, (Co * rows + N * (col_n + y_n)) * esz),
        "bias_add": (lambda: capi.check(L.rp_hip_channel_bias_add(d_y.ptr, d_b.ptr, N, Co, cols, dt), "bias"), 0.0, 2 * N * y_n * esz),
        "dcol=Wt.dy": (lambda: capi.gemm(d_col.ptr, d_w.ptr, d_dy.ptr, None, N, rows, Co, cols, (0, 1, rows), (y_n, cols, 1), (col_n, cols, 1), False, dt),
                       gemm_flops, (Co * rows + N * (col_n + y_n)) * esz),
        "col2im": (lambda: capi.check(L.rp_hip_col2im_batched(d_dx.ptr, d_col.ptr, N, *geom, 0, dt), "col2im"), 0.0, N * (x_n + col_n) * esz),
        "dW_n=dy.colt": (lambda: capi.gemm(d_dws.ptr, d_dy.ptr, d_col.ptr, None, N, Co, cols, rows, (y_n, cols, 1), (col_n, 1, cols), (Co * rows, rows, 1), False, dt),
                         gemm_flops, N * (col_n + y_n + Co * rows) * esz),
        "dW=sum_n": (lambda: capi.check(L.rp_hip_reduce_rows(d_dw.ptr, d_dws.ptr, N, Co * rows, 0, dt), "reduce_rows"), 0.0, (N + 1) * Co * rows * esz),
        "db": (lambda: capi.check(L.rp_hip_channel_sums(d_db.ptr, d_dy.ptr, N, Co, cols, 0, dt), "channel_sums"), 0.0, N * y_n * esz),
    }
    for fn, _, _ in ops.values():
        fn()
    capi.check(L.rp_hip_im2col_batched(d_col.ptr, d_x.ptr, N, *geom, dt), "im2col")       # dW reads the lowered activations, not dcol
    out, total = {}, 0.0
    for name, (fn, flops, nbytes) in ops.items():
        ms = _time_graph(capi, fn, 10, 2)
        total += ms
        out[name] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
        if flops:
            out[name]["TFLOP/s"] = round(flops / ms / 1e9, 1)
    total += out["im2col"]["us"] * 1e-3                 # the backward lowers the activations again for dW
    out["fwd_bwd_ms"] = round(total, 4)
    out["fwd_bwd_TFLOP/s"] = round(3 * gemm_flops / total / 1e9, 1)
    if L.rp_hip_conv2d_same_supported(C, H, W, k, k, dt) == 1:
        # forward and both gradients straight from zero-bordered planes (no lowered matrix)
        direct = {
            "y=conv(x,W)+b": (lambda: capi.check(L.rp_hip_conv2d_same_forward(d_y.ptr, d_x.ptr, d_w.ptr, d_b.ptr, N, C, H, W, Co, k, k, dt), "same forward"),
                              gemm_flops, N * (x_n + y_n) * esz),
            "dx,dW=conv_bwd(dy,x,W)": (lambda: capi.check(L.rp_hip_conv2d_same_backward(d_dx.ptr, d_dw.ptr, d_dy.ptr, d_x.ptr, d_w.ptr, N, C, H, W, Co, k, k, dt), "same backward"),
                                       2 * gemm_flops, N * (2 * x_n + y_n) * esz),
        }
        out["lowered_fwd_bwd_ms"] = out["fwd_bwd_ms"]
        total = out["db"]["us"] * 1e-3
        for name, (fn, flops, nbytes) in direct.items():
            ms = _time_graph(capi, fn, 10, 2)
            total += ms
            out[name] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1), "TFLOP/s": round(flops / ms / 1e9, 1)}
        out["fwd_bwd_ms"] = round(total, 4)
        out["fwd_bwd_TFLOP/s"] = round(3 * gemm_flops / total / 1e9, 1)
    for d in (d_x, d_w, d_b, d_dy, d_col, d_y, d_dx, d_dws, d_dw, d_db):
        d.free()
    return out


def lstm_step_times(capi, dt_name="bf16"):
    """One LSTM step (batch 64, input 1024, hidden 1024) forward + backward through the C ABI: the two gate products,
    the four gradient products (as two launches of two matrices each, the way the host layer issues them, and one by
    one), the two fused element-wise kernels and the bias reduction; each launch on its own and the whole step from one
    HIP graph."""
    rng = np.random.default_rng(5)
    B, I, H = 64, 1024, 1024
    G = 4 * H
    dt = {"bf16": capi.BF16, "f32": capi.F32}[dt_name]
    esz = 2 if dt == capi.BF16 else 4
    if dt == capi.BF16:
        mk = lambda shape, s=1.0: _bf16_bits((rng.standard_normal(shape) * s).astype(np.float32))
    else:
        mk = lambda shape, s=1.0: (rng.standard_normal(shape) * s).astype(np.float32)
    D_ = capi.DeviceBuffer
    d_x, d_h, d_c = D_.from_numpy(mk((B, I))), D_.from_numpy(mk((B, H), 0.5)), D_.from_numpy(mk((B, H), 0.5))
    d_wi, d_wh = D_.from_numpy(mk((I, G), 1 / 32)), D_.from_numpy(mk((H, G), 1 / 32))
    d_bi, d_bh, d_dhc = D_.from_numpy(mk((G,), 0.1)), D_.from_numpy(mk((G,), 0.1)), D_.from_numpy(mk((B, 2 * H)))
    d_g, d_act, d_hc, d_dg = D_(B * G * esz), D_(B * G * esz), D_(B * 2 * H * esz), D_(B * G * esz)
    d_dc, d_dx, d_dh = D_(B * H * esz), D_(B * I * esz), D_(B * H * esz)
    d_dwi, d_dwh, d_db = D_(I * G * esz), D_(H * G * esz), D_(G * esz)
    L = capi.lib()
    ops = {
        "gates=x.Wih": (lambda: capi.gemm(d_g.ptr, d_x.ptr, d_wi.ptr, None, 1, B, I, G, (0, I, 1), (0, G, 1), (0, G, 1), False, dt), 2.0 * B * I * G, (B * I + I * G + B * G) * esz),
        "gates+=h.Whh": (lambda: capi.gemm(d_g.ptr, d_h.ptr, d_wh.ptr, None, 1, B, H, G, (0, H, 1), (0, G, 1), (0, G, 1), True, dt), 2.0 * B * H * G, (B * H + H * G + 2 * B * G) * esz),
        "cell_fwd": (lambda: capi.check(L.rp_hip_lstm_cell_forward(d_hc.ptr, d_act.ptr, d_g.ptr, d_bi.ptr, d_bh.ptr, d_c.ptr, H, B, H, dt), "lstm fwd"), 0.0, (2 * B * G + 3 * B * H) * esz),
        "cell_bwd": (lambda: capi.check(L.rp_hip_lstm_cell_backward(d_dg.ptr, d_dc.ptr, d_dhc.ptr, d_act.ptr, d_hc.ptr, d_c.ptr, H, B, H, dt), "lstm bwd"), 0.0, (2 * B * G + 6 * B * H) * esz),
        "dx=dg.Wiht": (lambda: capi.gemm(d_dx.ptr, d_dg.ptr, d_wi.ptr, None, 1, B, G, I, (0, G, 1), (0, 1, G), (0, I, 1), False, dt), 2.0 * B * I * G, (B * G + I * G + B * I) * esz),
        "dh=dg.Whht": (lambda: capi.gemm(d_dh.ptr, d_dg.ptr, d_wh.ptr, None, 1, B, G, H, (0, G, 1), (0, 1, G), (0, H, 1), False, dt), 2.0 * B * H * G, (B * G + H * G + B * H) * esz),
        "dWih=xt.dg": (lambda: capi.gemm(d_dwi.ptr, d_x.ptr, d_dg.ptr, None, 1, I, B, G, (0, 1, I), (0, G, 1), (0, G, 1), False, dt), 2.0 * B * I * G, (B * I + B * G + I * G) * esz),
        "dWhh=ht.dg": (lambda: capi.gemm(d_dwh.ptr, d_h.ptr, d_dg.ptr, None, 1, H, B, G, (0, 1, H), (0, G, 1), (0, G, 1), False, dt), 2.0 * B * H * G, (B * H + B * G + H * G) * esz),
        "db": (lambda: capi.check(L.rp_hip_reduce_rows(d_db.ptr, d_dg.ptr, B, G, 0, dt), "reduce_rows"), 0.0, (B * G + G) * esz),
    }
    # With input size = hidden size the host layer issues the two input gradients, and the two weight gradients, as one
    # launch each over a batch of two: the second matrix of every operand is addressed by its distance from the first.
    def dist(p, q):
        return (q.ptr - p.ptr) // esz
    pairs = {
        "dx,dh=dg.W^t (pair)": (lambda: capi.gemm(d_dx.ptr, d_dg.ptr, d_wi.ptr, None, 2, B, G, I, (0, G, 1), (dist(d_wi, d_wh), 1, G), (dist(d_dx, d_dh), I, 1), False, dt),
                                4.0 * B * I * G, 2 * (B * G + I * G + B * I) * esz),
        "dW=x^t.dg,h^t.dg (pair)": (lambda: capi.gemm(d_dwi.ptr, d_x.ptr, d_dg.ptr, None, 2, I, B, G, (dist(d_x, d_h), 1, I), (0, G, 1), (dist(d_dwi, d_dwh), G, 1), False, dt),
                                    4.0 * B * I * G, 2 * (B * I + B * G + I * G) * esz),
    }
    paired = {k: v for k, v in ops.items() if k in ("gates=x.Wih", "gates+=h.Whh", "cell_fwd", "cell_bwd")}
    paired.update(pairs)
    paired["db"] = ops["db"]
    for fn, _, _ in list(ops.values()) + list(pairs.values()):
        fn()
    out = {}
    for name, (fn, flops, nbytes) in list(ops.items()) + list(pairs.items()):
        ms = _time_graph(capi, fn, 20, 2)
        out[name] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
    def step_of(group):
        def step():
            for fn, _, _ in group.values():
                fn()
        return step
    ms = _time_graph(capi, step_of(paired), 10, 2)
    total_bytes = sum(nb for _, _, nb in ops.values())
    out["step_ms"] = round(ms, 4)
    out["step_GB/s"] = round(total_bytes / ms / 1e6, 1)
    out["launches"] = len(paired)
    out["step_ms_separate_gradients"] = round(_time_graph(capi, step_of(ops), 10, 2), 4)
    out["launches_separate_gradients"] = len(ops)
    return out


def mlp_step_time(capi, reps=50, fused_backward=True):
    """Configuration 2 through the C ABI.  fused_backward: each layer's three gradients (dX, dW, db) come from one
    rp_hip_linear_backward call, which runs them as one launch for layers this small; False issues the two GEMMs and
    the bias reduction separately (the same bits, 18 launches instead of 12)."""
    import ctypes
    rng = np.random.default_rng(1)
    dims = [784, 256, 128, 10]; batch = 256
    F = capi.F32
    L = capi.lib()
    x = rng.uniform(0, 1, (batch, dims[0])).astype(np.float32)
    ws = [rng.normal(0, np.sqrt(2.0 / dims[i]), (dims[i], dims[i + 1])).astype(np.float32) for i in range(3)]
    bs = [np.zeros(dims[i + 1], np.float32) for i in range(3)]
    y = rng.integers(0, 10, batch).astype(np.int32)
    D = capi.DeviceBuffer
    d_x = D.from_numpy(x); d_w = [D.from_numpy(w) for w in ws]; d_b = [D.from_numpy(b) for b in bs]; d_y = D.from_numpy(y)
    d_z = [D(batch * dims[i + 1] * 4) for i in range(3)]; d_h = [D(batch * dims[i + 1] * 4) for i in range(2)]
    d_g = [D(batch * dims[i + 1] * 4) for i in range(3)]; d_gh = [D(batch * dims[i + 1] * 4) for i in range(2)]
    d_dw = [D(ws[i].nbytes) for i in range(3)]; d_db = [D(bs[i].nbytes) for i in range(3)]
    d_dx = D(x.nbytes); d_loss = D(4)

    def step():
        h = d_x
        for i in range(3):
            m, k, n = batch, dims[i], dims[i + 1]
            capi.gemm(d_z[i].ptr, h.ptr, d_w[i].ptr, d_b[i].ptr, 1, m, k, n, (0, k, 1), (0, n, 1), (0, n, 1), False, F)
            if i < 2:
                L.relu_kernel_device(d_h[i].ptr, d_z[i].ptr, m * n, F)
                h = d_h[i]
        L.rp_hip_cross_entropy_mean(d_loss.ptr, d_g[2].ptr, d_z[2].ptr, d_y.ptr, batch, 10, 1.0, F)
        for i in (2, 1, 0):
            m, k, n = batch, dims[i], dims[i + 1]
            inp = d_x if i == 0 else d_h[i - 1]
            dst = d_dx if i == 0 else d_gh[i - 1]
            if fused_backward:
                L.rp_hip_linear_backward(dst.ptr, d_dw[i].ptr, d_db[i].ptr, d_g[i].ptr, inp.ptr, d_w[i].ptr, m, k, n,
                                         k, 1, n, 1, k, 1, n, 1, 0, 0, 0, F)
            else:
                L.rp_hip_reduce_rows(d_db[i].ptr, d_g[i].ptr, m, n, 0, F)
                # dW[k,n] = inpᵀ[k,m] · g[m,n]
                capi.gemm(d_dw[i].ptr, inp.ptr, d_g[i].ptr, None, 1, k, m, n, (0, 1, k), (0, n, 1), (0, n, 1), False, F)
                # dIn[m,k] = g[m,n] · Wᵀ[n,k]
                capi.gemm(dst.ptr, d_g[i].ptr, d_w[i].ptr, None, 1, m, n, k, (0, n, 1), (0, 1, n), (0, k, 1), False, F)
            if i > 0:
                L.backwards_relu_device(d_gh[i - 1].ptr, d_z[i - 1].ptr, d_g[i - 1].ptr, m * k, F)

    ms = _time_launches(capi, step, reps, 5)
    ms_graph = _time_graph(capi, step, 10, 2)
    return {"ms": ms_graph, "ms_eager_from_python": ms, "launches": 12 if fused_backward else 18,
            "note": "9 GEMMs (bias fused into the 3 forward ones), 2 relu, 2 relu-backward, "
            "cross-entropy fwd+bwd, 3 bias-gradient reductions; with each layer's dX, dW and db in one launch (rp_hip_linear_backward) "
            "that is 12 launches, issued separately 18 (`ms_separate_launches`); `ms` replays the step from a HIP graph, "
            "`ms_eager_from_python` launches it call by call through ctypes, `ms_through_python_api` is the same step through "
            "the drop-in recpulse_cuda tensors, recpulse.module.Linear and autograd (wall clock, allocation and graph bookkeeping included)"}


def mlp_step_time_dropin(reps=200, warmup=20):
    """Config 2 end to end through the drop-in Python API (recpulse_cuda tensors, recpulse.module.Linear, autograd):
    forward, mean cross-entropy, backward, zero_grad.  Wall-clock per step with one synchronising read at the end."""
    sys.path.insert(0, os.path.join(ROOT, "recpulse_amd", "dropin"))
    import recpulse_cuda as rp
    from recpulse.module import Linear, Module

    class MLP(Module):
        def __init__(self):
            super().__init__()
            self.fc1, self.fc2, self.fc3 = Linear(784, 256), Linear(256, 128), Linear(128, 10)

        def forward(self, x):
            return self.fc3(self.fc2(self.fc1(x).op_relu()).op_relu())

    rng = np.random.default_rng(1)
    rp.manual_seed(1)
    net = MLP().to(device="cuda")
    x = rp.from_numpy(rng.uniform(0, 1, (256, 784)).astype(np.float32)).to(device="cuda").requires_grad_(True)
    y = rng.integers(0, 10, 256).tolist()
    params = list(net.learnable().values())

    def step():
        loss = net(x).op_cross_entropy_loss(y)
        loss.backward()
        return loss

    for _ in range(warmup):
        loss = step()
        for p in params + [x]:
            p.zero_grad()
    loss.sum_all()
    t0 = time.perf_counter()
    for _ in range(reps):
        loss = step()
        for p in params + [x]:
            p.zero_grad()
    loss.sum_all()                      # device -> host read: everything before it has finished
    return (time.perf_counter() - t0) / reps * 1e3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--data", choices=["normal", "ints", "ones", "zeros"], default="normal",
                    help="operand values of the headline GEMMs: N(0,1) (the configuration) or low-toggle data, to show how far the "
                         "power-managed shader clock, and with it the throughput, depends on the values multiplied")
    ap.add_argument("--skinny-only", action="store_true",
                    help="run only the few-row bf16 GEMMs of configuration 5a and print their figures (for profiling that kernel alone)")
    ap.add_argument("--wide-only", action="store_true",
                    help="run only the fp32 (4096) and fp64 (2048, 4096) square GEMMs and print their figures (for profiling those kernels alone)")
    ap.add_argument("--memory-ceilings", action="store_true",
                    help="only the store / load / copy rates of the library's streaming kernels at footprints from 64 MB to 2 GB")
    ap.add_argument("--attention-only", action="store_true",
                    help="run only the configuration-4 attention launches in bf16, unfused and fused (for profiling those kernels alone)")
    ap.add_argument("--conv-only", action="store_true",
                    help="run only the conv2d layer's launches (for profiling those kernels alone), in --conv-dtype")
    ap.add_argument("--conv-dtype", choices=["bf16", "f32"], default="bf16")
    ap.add_argument("--mlp-only", action="store_true",
                    help="run only the configuration-2 MLP step (C ABI from a HIP graph, eager, and through the drop-in Python API)")
    ap.add_argument("--lstm-only", action="store_true",
                    help="time only the LSTM step (per-launch table and whole step), for profiling runs")
    ap.add_argument("--sustain", type=float, default=0.0,
                    help="run the forward 8192^3 bf16 GEMM back to back for this many seconds on --data operands while polling amd-smi "
                         "for shader clock and socket power, and print those figures (evidence for the power-limit reading of the headline)")
    ap.add_argument("--sustain-dtype", choices=["bf16", "f16"], default="bf16", help="16-bit type of the --sustain run")
    ap.add_argument("--sweep-only", action="store_true",
                    help="run only the configuration-3 sweep below the headline size: N = 1024 and 4096, bf16 and fp16, forward, dA, dB "
                         "(for profiling those kernels alone)")
    ap.add_argument("--f16-only", action="store_true",
                    help="run only the fp16 8192^3 forward GEMM (for profiling that kernel alone)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a plain copy kernel of known size (256 MiB in, 256 MiB out), the yardstick for FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    from recpulse_amd import capi
    if capi.device_count() < 1:
        print("bench.py needs a GPU and the built librp_hip.so; there is no CPU fallback", file=sys.stderr)
        sys.exit(1)
    capi.check(capi.lib().rp_hip_set_device(0), "rp_hip_set_device")

    if args.calibrate:
        n = 64 << 20
        src, dst = capi.DeviceBuffer(4 * n), capi.DeviceBuffer(4 * n)
        capi.check(capi.lib().rp_hip_fill(src.ptr, 1.0, n, capi.F32), "fill")
        for _ in range(3):
            capi.check(capi.lib().rp_hip_convert(dst.ptr, capi.F32, src.ptr, capi.F32, n), "copy")
        capi.synchronize()
        src.free(); dst.free()
    if args.sustain > 0:
        print(json.dumps({"sustained_gemm_8192": sustained(capi, args.sustain, args.data, dtype=args.sustain_dtype)}))
        return
    if args.skinny_only:
        print(json.dumps({"skinny": skinny_times(capi)}))
        return
    if args.sweep_only:
        print(json.dumps({"square_sweep": square_sweep(capi)}))
        return
    if args.f16_only:
        print(json.dumps({"gemm_f16_8192": f16_time(capi)}))
        return
    if args.memory_ceilings:
        print(json.dumps({"memory_ceilings": memory_ceilings(capi)}))
        return
    if args.attention_only:
        print(json.dumps({"attention_bf16": attention_times(capi, "bf16"), "attention_f32": attention_times(capi, "f32")}))
        return
    if args.lstm_only:
        print(json.dumps({"lstm_step_bf16": lstm_step_times(capi, "bf16"), "lstm_step_f32": lstm_step_times(capi, "f32")}))
        return
    if args.mlp_only:
        out = mlp_step_time(capi)
        out["ms_separate_launches"] = mlp_step_time(capi, fused_backward=False)["ms"]
        out["ms_through_python_api"] = mlp_step_time_dropin()
        print(json.dumps({"mlp_f32_step": out}))
        return
    if args.conv_only:
        print(json.dumps({"conv2d_" + args.conv_dtype: conv2d_times(capi, args.conv_dtype)}))
        return
    if args.wide_only:
        print(json.dumps({"wide": wide_times(capi, (("gemm_f32_4096", "f32", 4096), ("gemm_f64_2048", "f64", 2048), ("gemm_f64_4096", "f64", 4096)))}))
        return
    h = headline(capi, args.steps, args.warmup, data=args.data)
    a, b = h.pop("operands")
    line = {
        "metric": "GEMM TFLOP/s (bf16 8192^3, forward + both backward GEMMs per step)",
        "value": h["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": h["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic" if args.data == "normal" else f"synthetic ({args.data}: diagnostic, not the configuration)",
        "config": {"workload": "config 3 at N=8192: bf16 square GEMM, fp32 accumulate, bf16 output; "
                               "C=A·B, dA=dC·Bᵀ, dB=Aᵀ·dC with transposes as stride views; A,B,dC ~ N(0,1) seed 2",
                   "m": 8192, "n": 8192, "k": 8192, "gemms_per_step": 3},
        "roofline": {"bound": "mfma", "achieved": h["fwd_tflops"], "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                     "frac": h["fwd_tflops"] / PEAK_TFLOPS["bf16"], "traffic": forward_traffic(h["kernel"]),
                     "traffic_note": "bytes per launch below the L2s (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, scaled by a copy kernel), "
                                     "read from profiles/pmc_traffic_gemm_bf16_8192.md (null if that summary is of another kernel); "
                                     "algorithmic bytes are 4.027e8",
                     "kernel": h["kernel"] + " (forward, A row-major x B row-major)",
                     "avg_launch_ms": h["kernel_ms"]["fwd_nn"]},
        "kernel_ms": h["kernel_ms"], "sampled_rel_err": h["sampled_rel_err"],
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(a, b)
    del a, b
    if not args.no_secondary:
        line["secondary"] = secondary(capi)
        if not args.no_cpu:
            line["secondary"]["cpu_one_core"] = cpu_baseline_configs()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
