#!/usr/bin/env python3
"""Benchmark of the MI355X int8 path: one JSON line on stdout.

A step is one pass of the hot path over one batch of synthetic input that is
already resident in GPU memory: by default the MatMulInteger of the BERT-base
FFN-up projection (M=4096, K=768, N=3072, uint8 activations x int8 weights,
per-column fp32 dequantisation fused into the store) -- the shape the int8
target is quoted on.  The same line carries, under "extras", the
QuantizeLinear / DequantizeLinear / DynamicQuantizeLinear rates at
[8192, 32768] and the other GEMM shapes.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Every entry point is called through the C-ABI (include/om_mi355x.h).  Kernel
time is measured with HIP events recorded on the runtime's own stream around
the timed region; whole-job time with the host clock around the same region.
The headline is timed over exactly --steps launches after --warmup untimed
ones; before that, and before every other measurement, the same call is
launched untimed until the device has left its idle clocks (PREHEAT_MS, the
time spent is reported as "preheat_ms").  The other measurements time at least
MIN_LAUNCHES launches each, in separate event brackets, and report the mean
and the p10 / median / p90 of the bracket averages.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "onnx-mlir_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0        # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0      # MI355X published dense int8 MFMA rate (no sparsity)

METRIC = "int8 MatMulInteger TOPS (% MFMA peak) + Q/DQ GB/s (% HBM), 1 MI355X"

# The device leaves its idle clocks only after about 100 ms of work (the headline
# kernel measures 19.0 us after 200 launches from idle, 17.2 us in steady
# state).  Every timed group is therefore preceded by an untimed pre-heat of the
# same call until this much GPU time has passed; it is independent of --warmup
# and its length is reported with every result ("preheat_ms").
PREHEAT_MS = 120.0
# Launches an "extras" measurement times at least, in BRACKETS separate event
# brackets (p10 / median / p90 of the bracket averages show the spread).
MIN_LAUNCHES = 20
BRACKETS = 10


def traffic_record():
    """HBM bytes per launch of the headline kernel, from the rocprofv3 --pmc
    summary kept in profiles/headline_traffic.json (FETCH_SIZE and WRITE_SIZE,
    one run each, scaled by what the same counters read for a plain copy of
    known size).  The record names the kernel and the commit it was measured
    at; it is only used while the headline kernel still has that name."""
    try:
        with open(os.path.join(ROOT, "profiles", "headline_traffic.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return None


def preheat(rt, fn, min_ms=PREHEAT_MS):
    """Untimed launches of `fn` until `min_ms` of GPU time have passed.
    Returns (milliseconds spent, milliseconds per launch of the last batch)."""
    spent, batch, per = 0.0, 16, 1e-4
    while spent < min_ms:
        rt.timer_start()
        for _ in range(batch):
            fn()
        ms = rt.timer_stop()
        spent += ms
        per = max(ms / batch, 1e-4)
        batch = int(min(20000, max(16, (min_ms - spent) / per + 1)))
    return spent, per


def timed(rt, fn, steps, warmup, heat=True):
    """Returns (host seconds per step, event milliseconds per step, pre-heat ms)."""
    heat_ms = preheat(rt, fn)[0] if heat else 0.0
    for _ in range(warmup):
        fn()
    rt.synchronize()
    t0 = time.perf_counter()
    rt.timer_start()
    for _ in range(steps):
        fn()
    ev_ms = rt.timer_stop()          # waits for the last launch
    rt.synchronize()
    host = time.perf_counter() - t0
    return host / steps, ev_ms / steps, heat_ms


def measure(rt, fn, steps, warmup):
    """One extras measurement: pre-heat, warm-up, then at least MIN_LAUNCHES
    launches in BRACKETS event brackets of at least a millisecond each.
    kernel_ms is the mean over all timed launches; p10 / median / p90 are of the
    bracket averages."""
    heat_ms, est_ms = preheat(rt, fn)
    for _ in range(warmup):
        fn()
    # a bracket holds at least about a millisecond of launches: with fewer the
    # host's submission latency shows in the events of short kernels
    per = max(2, -(-max(steps, MIN_LAUNCHES) // BRACKETS), int(1.0 / est_ms) + 1)
    rt.synchronize()
    t0 = time.perf_counter()
    times = []
    for _ in range(BRACKETS):
        rt.timer_start()
        for _ in range(per):
            fn()
        times.append(rt.timer_stop() / per)
    host = (time.perf_counter() - t0) / (per * BRACKETS)
    q = np.percentile(np.array(times), [10, 50, 90])
    return {"ms_per_step": host * 1e3, "kernel_ms": float(np.mean(times)),
            "kernel_ms_p10": float(q[0]), "kernel_ms_median": float(q[1]), "kernel_ms_p90": float(q[2]),
            "launches": per * BRACKETS, "preheat_ms": heat_ms}


def gemm_case(rt, wl, name, M, K, N, w_i8, w_scale, steps, warmup, epilogue="f32", headline=False):
    rng = np.random.default_rng(0xC0FFEE00 + M + K + N)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    dA = rt.DeviceArray.from_numpy(A)
    dW = rt.DeviceArray.from_numpy(w_i8)
    dS = rt.DeviceArray.from_numpy(w_scale)
    dAs = rt.DeviceArray.from_numpy(np.array(0.0173, np.float32))
    dAz = rt.DeviceArray.from_numpy(np.array(131, np.uint8))
    rt.mark_constant(dW)             # weights: packed once, like any model constant
    if epilogue == "f32":
        dY = rt.DeviceArray((M, N), np.float32)
        fn = rt.PreparedCall("om_mi355x_MatMulIntegerDequant", dY, dA, dW, dAz, None, dAs, dS, None, 0)
    else:
        dY = rt.DeviceArray((M, N), np.int32)
        fn = rt.PreparedCall("om_mi355x_MatMulInteger", dY, dA, dW, dAz, None)
    ops = 2.0 * M * N * K
    res = {"name": name, "M": M, "K": K, "N": N, "epilogue": epilogue}
    if headline:
        # the contract's measurement: exactly `steps` launches in one bracket
        host_s, ev_ms, heat_ms = timed(rt, fn, steps, warmup)
        res.update({"ms_per_step": host_s * 1e3, "kernel_ms": ev_ms, "preheat_ms": heat_ms,
                    "tops": ops / host_s / 1e12})
    else:
        res.update(measure(rt, fn, steps, warmup))
        res["tops"] = ops / (res["ms_per_step"] * 1e-3) / 1e12
    fn.check()
    fn.close()
    res.update({"kernel": rt.last_gemm_kernel(), "kernel_tops": ops / (res["kernel_ms"] * 1e-3) / 1e12,
                "ops": ops, "hbm_bytes_algorithmic": M * K + K * N + 4 * M * N})
    for d in (dA, dW, dS, dAs, dAz, dY):
        d.free()
    return res


def rotated_case(rt, wl, M, K, N, w_i8, w_scale, steps, warmup, sets=6):
    """The headline GEMM rotating over `sets` activation/output buffer pairs,
    320 MB in all for M=4096, N=3072, so that no launch finds its output or its
    activations in the 256 MB last-level cache from the launch before."""
    rng = np.random.default_rng(0xC0FFEE00 + M + K + N)
    dW = rt.DeviceArray.from_numpy(w_i8)
    dS = rt.DeviceArray.from_numpy(w_scale)
    dAs = rt.DeviceArray.from_numpy(np.array(0.0173, np.float32))
    dAz = rt.DeviceArray.from_numpy(np.array(131, np.uint8))
    rt.mark_constant(dW)
    bufs, calls = [], []
    for _ in range(sets):
        dA = rt.DeviceArray.from_numpy(rng.integers(0, 256, (M, K), dtype=np.uint8))
        dY = rt.DeviceArray((M, N), np.float32)
        bufs += [dA, dY]
        calls.append(rt.PreparedCall("om_mi355x_MatMulIntegerDequant", dY, dA, dW, dAz, None, dAs, dS, None, 0))
    state = {"i": 0}

    def rotate():
        calls[state["i"] % sets]()
        state["i"] += 1

    res = measure(rt, rotate, max(steps, 10 * sets), warmup)
    for c in calls:
        c.check()
        c.close()
    for d in bufs + [dW, dS, dAs, dAz]:
        d.free()
    res.update({"buffer_sets": sets, "tops": 2.0 * M * N * K / (res["kernel_ms"] * 1e-3) / 1e12})
    return res


def decode_case(rt, wl, M, steps, warmup):
    c = wl.config5("up", M=M)
    K, N = c["W"].shape
    dX = rt.DeviceArray.from_numpy(c["X"])
    dW = rt.DeviceArray.from_numpy(c["W"])
    dS = rt.DeviceArray.from_numpy(c["w_scale"])
    dY = rt.DeviceArray((M, N), np.float32)
    rt.mark_constant(dW)
    fn = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dY, dX, dW, None, dS, None, 0)
    res = measure(rt, fn, steps, warmup)
    fn.check()
    fn.close()
    nbytes = K * N + M * K + 4 * M * N
    res.update({"name": f"config5 decode M={M}", "M": M, "K": K, "N": N,
                "gbs": nbytes / (res["kernel_ms"] * 1e-3) / 1e9, "bytes": nbytes,
                "hbm_frac": nbytes / (res["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS})
    for d in (dX, dW, dS, dY):
        d.free()
    return res


def chain_case(rt, wl, M, steps, warmup, limits):
    """Config 4's feed-forward block as two dynamically quantized layers in a
    row, FFN-up -> Gelu -> FFN-down, GPU-resident: two calls of
    om_mi355x_DynQuantMatMulDequant, or (limits) of
    om_mi355x_DynQuantMatMulDequantLimits with the first call's y_limits handed
    to the second as x_limits, so that the second layer's
    DynamicQuantizeLinear is one pass over its input."""
    up, down = wl.config4("ffn_up"), wl.config4("ffn_down")
    K, N = up["W"].shape
    N2 = down["W"].shape[1]
    dX = rt.DeviceArray.from_numpy(wl.normal_f32(4, 70, (M, K)))
    dW1, dS1 = rt.DeviceArray.from_numpy(up["W"]), rt.DeviceArray.from_numpy(up["w_scale"])
    dW2, dS2 = rt.DeviceArray.from_numpy(down["W"]), rt.DeviceArray.from_numpy(down["w_scale"])
    dH, dY = rt.DeviceArray((M, N), np.float32), rt.DeviceArray((M, N2), np.float32)
    dL = rt.DeviceArray((2,), np.float32)
    rt.mark_constant(dW1)
    rt.mark_constant(dW2)
    if limits:
        f1 = rt.PreparedCall("om_mi355x_DynQuantMatMulDequantLimits", dH, dL, dX, None, dW1, None, dS1, None, 2)
        f2 = rt.PreparedCall("om_mi355x_DynQuantMatMulDequantLimits", dY, None, dH, dL, dW2, None, dS2, None, 0)
    else:
        f1 = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dH, dX, dW1, None, dS1, None, 2)
        f2 = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dY, dH, dW2, None, dS2, None, 0)

    def fn():
        f1()
        f2()

    res = measure(rt, fn, steps, warmup)
    f1.check()
    f2.check()
    f1.close()
    f2.close()
    ops = 2.0 * M * N * K + 2.0 * M * N2 * N
    res.update({"name": f"config4 M={M} ffn_up -> Gelu -> ffn_down, " +
                        ("limits handed on" if limits else "two plain calls"),
                "M": M, "K": K, "N": N, "N2": N2, "kernel": rt.last_gemm_kernel(),
                "tops": ops / (res["kernel_ms"] * 1e-3) / 1e12})
    for d in (dX, dW1, dS1, dW2, dS2, dH, dY, dL):
        d.free()
    return res


def decode_limits_case(rt, wl, M, steps, warmup):
    """A decode step whose activation comes with its minimum and maximum (from
    the layer before): om_mi355x_DynQuantMatMulDequantLimits with x_limits."""
    c = wl.config5("up", M=M)
    K, N = c["W"].shape
    x = c["X"]
    dX = rt.DeviceArray.from_numpy(x)
    dL = rt.DeviceArray.from_numpy(np.array([x.min(), x.max()], np.float32))
    dW, dS = rt.DeviceArray.from_numpy(c["W"]), rt.DeviceArray.from_numpy(c["w_scale"])
    dY = rt.DeviceArray((M, N), np.float32)
    rt.mark_constant(dW)
    fn = rt.PreparedCall("om_mi355x_DynQuantMatMulDequantLimits", dY, None, dX, dL, dW, None, dS, None, 0)
    res = measure(rt, fn, steps, warmup)
    fn.check()
    fn.close()
    nbytes = K * N + M * K + 4 * M * N
    res.update({"name": f"config5 decode M={M}, limits of x known", "M": M, "K": K, "N": N,
                "kernel": rt.last_gemm_kernel(),
                "gbs": nbytes / (res["kernel_ms"] * 1e-3) / 1e9, "bytes": nbytes,
                "hbm_frac": nbytes / (res["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS})
    for d in (dX, dL, dW, dS, dY):
        d.free()
    return res


def qlinear_case(rt, wl, steps, warmup):
    """Config 3: QLinearMatMul, uint8 x uint8 -> uint8 with both zero points
    non-zero (row sums of A and the per-row correction are part of the step)."""
    c = wl.config3()
    M, K = c["A"].shape
    N = c["B"].shape[1]
    d = {k: rt.DeviceArray.from_numpy(np.asarray(c[k])) for k in
         ("A", "a_scale", "a_zp", "B", "b_scale", "b_zp", "y_scale", "y_zp")}
    dY = rt.DeviceArray((M, N), np.uint8)
    rt.mark_constant(d["B"])
    fn = rt.PreparedCall("om_mi355x_QLinearMatMul", dY, d["A"], d["a_scale"], d["a_zp"], d["B"],
                         d["b_scale"], d["b_zp"], d["y_scale"], d["y_zp"], rt.WRAP)
    res = measure(rt, fn, steps, warmup)
    fn.check()
    fn.close()
    ops = 2.0 * M * N * K
    res.update({"name": "config3 QLinearMatMul u8 x u8 -> u8", "M": M, "K": K, "N": N,
                "kernel": rt.last_gemm_kernel(), "tops": ops / (res["kernel_ms"] * 1e-3) / 1e12,
                "hbm_bytes_algorithmic": M * K + K * N + M * N})
    for a in list(d.values()) + [dY]:
        a.free()
    return res


def qlinear_ffn_up_case(rt, wl, steps, warmup):
    """QLinearMatMul at the headline shape (config 4 FFN-up, 4096 x 768 x 3072):
    uint8 activations with a zero point, symmetric int8 weights (b_zero_point
    a constant 0, per-tensor scales), uint8 out -- the requantizing epilogue on
    the kernel that holds the weights in registers."""
    c = wl.config4("ffn_up")
    K, N = c["W"].shape
    M = 4096
    A = wl.uniform_u8(4, 90, (M, K))
    ops_ = {"A": A, "a_scale": np.float32(0.0173), "a_zp": np.array(131, np.uint8), "B": c["W"],
            "b_scale": np.float32(0.004), "b_zp": np.array(0, np.int8), "y_scale": np.float32(0.9),
            "y_zp": np.array(127, np.uint8)}
    d = {k: rt.DeviceArray.from_numpy(np.asarray(v)) for k, v in ops_.items()}
    dY = rt.DeviceArray((M, N), np.uint8)
    rt.mark_constant(d["B"])
    rt.mark_constant(d["b_zp"])
    fn = rt.PreparedCall("om_mi355x_QLinearMatMul", dY, d["A"], d["a_scale"], d["a_zp"], d["B"],
                         d["b_scale"], d["b_zp"], d["y_scale"], d["y_zp"], rt.WRAP)
    res = measure(rt, fn, steps, warmup)
    fn.check()
    fn.close()
    rt.unmark_constant(d["b_zp"])
    ops = 2.0 * M * N * K
    res.update({"name": "config4 ffn_up QLinearMatMul u8 x i8 -> u8", "M": M, "K": K, "N": N,
                "kernel": rt.last_gemm_kernel(), "tops": ops / (res["kernel_ms"] * 1e-3) / 1e12,
                "hbm_bytes_algorithmic": M * K + K * N + M * N})
    for a in list(d.values()) + [dY]:
        a.free()
    return res


def fused_case(rt, wl, name, M, K, N, w_i8, w_scale, steps, warmup, X=None, activation=0):
    """DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul as one call: fp32
    activations in, fp32 out (the chain the quantized models contain);
    `activation` 1 / 2 adds the Relu / Gelu that follows an FFN-up projection."""
    if X is None:
        X = np.random.default_rng(0xF00D + M + K + N).normal(0, 1, (M, K)).astype(np.float32)
    dX = rt.DeviceArray.from_numpy(X)
    dW = rt.DeviceArray.from_numpy(w_i8)
    dS = rt.DeviceArray.from_numpy(np.asarray(w_scale, np.float32))
    dY = rt.DeviceArray((M, N), np.float32)
    rt.mark_constant(dW)
    fn = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dY, dX, dW, None, dS, None, activation)
    res = measure(rt, fn, steps, warmup)
    fn.check()
    fn.close()
    ops = 2.0 * M * N * K
    nbytes = 4 * M * K + K * N + 4 * M * N
    res.update({"name": name, "M": M, "K": K, "N": N, "kernel": rt.last_gemm_kernel(),
                "tops": ops / (res["kernel_ms"] * 1e-3) / 1e12, "hbm_bytes_algorithmic": nbytes,
                "hbm_frac_at_algorithmic_bytes": nbytes / (res["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS})
    for d in (dX, dW, dS, dY):
        d.free()
    return res


def config1_cases(rt, wl, steps, warmup, only=None):
    """Config 1 (A f32 [128,768] -> DynamicQuantizeLinear -> MatMulInteger with
    int8 B [768,768] -> Cast -> Mul): as the three separate calls of the
    unfused graph, tensors resident, and as the one fused call."""
    c = wl.config1()
    M, K = c["A"].shape
    N = c["B"].shape[1]
    dA = rt.DeviceArray.from_numpy(c["A"])
    dB = rt.DeviceArray.from_numpy(c["B"])
    dbs = rt.DeviceArray.from_numpy(np.asarray(c["b_scale"], np.float32))
    dbz = rt.DeviceArray.from_numpy(np.asarray(c["b_zp"]))
    dq, ds, dz = rt.DeviceArray((M, K), np.uint8), rt.DeviceArray((), np.float32), rt.DeviceArray((), np.uint8)
    dY = rt.DeviceArray((M, N), np.float32)
    rt.mark_constant(dB)
    calls = [rt.PreparedCall("om_mi355x_DynamicQuantizeLinear", dq, ds, dz, dA),
             rt.PreparedCall("om_mi355x_MatMulIntegerDequant", dY, dq, dB, dz, dbz, ds, dbs, None, 0)]

    def separate():
        for f in calls:
            f()

    fused = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dY, dA, dB, dbz, dbs, None, 0)
    out = {}
    if only in (None, "separate"):
        sep = measure(rt, separate, steps, warmup)
        sep["kernel"] = rt.last_gemm_kernel()
        out["DynamicQuantizeLinear + MatMulIntegerDequant (two calls)"] = sep
    if only in (None, "fused"):
        fus = measure(rt, fused, steps, warmup)
        fus["kernel"] = rt.last_gemm_kernel()
        out["DynQuantMatMulDequant (one call)"] = fus
    for f in calls + [fused]:
        f.check()
        f.close()
    ops = 2.0 * M * N * K
    nbytes = 4 * M * K + K * N + 4 * M * N
    for r in out.values():
        r.update({"M": M, "K": K, "N": N, "tops": ops / (r["kernel_ms"] * 1e-3) / 1e12,
                  "hbm_bytes_algorithmic": nbytes})
    for d in (dA, dB, dbs, dbz, dq, ds, dz, dY):
        d.free()
    return out


def qdq_cases(rt, wl, rows, cols, steps, warmup, only=None):
    c = wl.config2(rows, cols)
    n = rows * cols
    dX = rt.DeviceArray.from_numpy(c["X"])
    dS = rt.DeviceArray.from_numpy(c["scale"])
    dZ = rt.DeviceArray.from_numpy(c["zp"])
    dQ = rt.DeviceArray((rows, cols), np.uint8)
    dD = rt.DeviceArray((rows, cols), np.float32)
    dys = rt.DeviceArray((), np.float32)
    dyz = rt.DeviceArray((), np.uint8)
    s1 = rt.DeviceArray.from_numpy(np.array(0.02, np.float32))
    z1 = rt.DeviceArray.from_numpy(np.array(128, np.uint8))
    out = {}

    def run(name, fn, nbytes):
        if only is not None and name != only:
            fn.close()
            return
        r = measure(rt, fn, steps, warmup)
        fn.check()
        fn.close()
        r.update({"bytes": nbytes, "gbs": nbytes / (r["kernel_ms"] * 1e-3) / 1e9,
                  "hbm_frac": nbytes / (r["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS})
        out[name] = r

    P = rt.PreparedCall
    run("quantize_per_axis", P("om_mi355x_QuantizeLinear", dQ, dX, dS, dZ, 1, 1), 5 * n)
    run("dequantize_per_axis", P("om_mi355x_DequantizeLinear", dD, dQ, dS, dZ, 1), 5 * n)
    run("quantize_per_tensor", P("om_mi355x_QuantizeLinear", dQ, dX, s1, z1, 1, 1), 5 * n)
    run("dequantize_per_tensor", P("om_mi355x_DequantizeLinear", dD, dQ, s1, z1, 1), 5 * n)
    # two reads of X (min/max, then quantize) + one write: the tensor is far
    # larger than any on-chip cache
    run("dynamic_quantize", P("om_mi355x_DynamicQuantizeLinear", dQ, dys, dyz, dX), 9 * n)
    for d in (dX, dS, dZ, dQ, dD, dys, dyz, s1, z1):
        d.free()
    return out


def dql_activation_cases(rt, steps, warmup, only=None):
    """DynamicQuantizeLinear on activation-sized tensors (the first half of every
    dynamically quantized layer of config 4): one launch, X read once."""
    out = {}
    for rows, cols in ((4096, 768), (4096, 3072)):
        name = f"dynamic_quantize_{rows}x{cols}"
        if only is not None and only != name:
            continue
        rng = np.random.default_rng(rows + cols)
        dX = rt.DeviceArray.from_numpy(rng.standard_normal((rows, cols)).astype(np.float32))
        dQ = rt.DeviceArray((rows, cols), np.uint8)
        dys, dyz = rt.DeviceArray((), np.float32), rt.DeviceArray((), np.uint8)
        fn = rt.PreparedCall("om_mi355x_DynamicQuantizeLinear", dQ, dys, dyz, dX)
        r = measure(rt, fn, steps, warmup)
        fn.check()
        fn.close()
        nbytes = 5 * rows * cols        # X once, the 8-bit result once
        r.update({"bytes": nbytes, "gbs": nbytes / (r["kernel_ms"] * 1e-3) / 1e9,
                  "hbm_frac": nbytes / (r["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS})
        out[name] = r
        for d in (dX, dQ, dys, dyz):
            d.free()
    return out


def per_axis_layout_cases(rt, steps, warmup):
    """Per-axis QuantizeLinear / DequantizeLinear on layouts other than config 2's:
    an inner axis with slabs that are / are not whole float4, short rows, rows
    that are not whole float4.  Small tensors (cache-resident): the figures
    compare dispatch paths, they are not HBM rates."""
    rng = np.random.default_rng(0xA715)
    out = {}
    for shape in ((64, 2048, 7, 7), (256, 512, 14, 14), (8, 256, 57, 57), (1 << 20, 4), (1 << 18, 64),
                  (1 << 16, 256), (1 << 18, 65), (1 << 13, 2048)):
        C = shape[1]
        x = rng.normal(0, 1, shape).astype(np.float32)
        dX = rt.DeviceArray.from_numpy(x)
        dS = rt.DeviceArray.from_numpy(rng.uniform(0.01, 0.1, C).astype(np.float32))
        dZ = rt.DeviceArray.from_numpy(rng.integers(0, 255, C).astype(np.uint8))
        dQ, dY = rt.DeviceArray(shape, np.uint8), rt.DeviceArray(shape, np.float32)
        res = {}
        for name, fn in (("quantize", rt.PreparedCall("om_mi355x_QuantizeLinear", dQ, dX, dS, dZ, 1, 1)),
                         ("dequantize", rt.PreparedCall("om_mi355x_DequantizeLinear", dY, dQ, dS, dZ, 1))):
            r = measure(rt, fn, steps, warmup)
            fn.check()
            fn.close()
            res[name] = {"kernel_us": r["kernel_ms"] * 1e3, "gb_per_s": 5 * x.size / (r["kernel_ms"] * 1e-3) / 1e9}
        out["x".join(str(d) for d in shape)] = res
        for d in (dX, dS, dZ, dQ, dY):
            d.free()
    return out


def only_mode(rt, wl, what, steps, warmup):
    """One kernel, `steps` launches, nothing else on the GPU: the target of the
    rocprofv3 counter runs whose summaries are kept under profiles/."""
    import ctypes
    if what == "copy":
        # plain device-to-device copy of known size: calibrates FETCH_SIZE / WRITE_SIZE
        n = 1 << 30
        a, b = rt.DeviceArray((n,), np.uint8), rt.DeviceArray((n,), np.uint8)
        hip = ctypes.CDLL("libamdhip64.so")
        hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        for _ in range(steps):
            assert hip.hipMemcpy(b.ptr, a.ptr, n, 3) == 0
        hip.hipDeviceSynchronize()
        return {"only": what, "bytes_read": n, "bytes_written": n, "launches": steps}
    if what in ("gemm_ffn_up", "gemm_qkv", "gemm_ffn_down", "gemm_out"):
        layer = what[5:]
        k, n = wl.CONFIG4_SHAPES[layer]
        c = wl.config4(layer, M=8)
        r = gemm_case(rt, wl, f"config4 {layer}", 4096, k, n, c["W"], c["w_scale"], steps, warmup, "f32",
                      headline=True)
        return {"only": what, **r}
    if what == "per_axis_layouts":
        return {"only": what, **per_axis_layout_cases(rt, steps, warmup)}
    if what == "mfma_ceiling":
        return {"only": what, "random_operands": rt.mfma_ceiling(True),
                "small_constant_operands": rt.mfma_ceiling(False)}
    if what in ("fused_ffn_up", "fused_ffn_down", "fused_ffn_up_relu", "fused_ffn_up_gelu"):
        layer = "ffn_down" if what == "fused_ffn_down" else "ffn_up"
        act = {"relu": 1, "gelu": 2}.get(what.rsplit("_", 1)[1], 0)
        k, n = wl.CONFIG4_SHAPES[layer]
        c = wl.config4(layer, M=8)
        r = fused_case(rt, wl, f"config4 {layer} fused layer" + (f", activation {act}" if act else ""),
                       4096, k, n, c["W"], c["w_scale"], steps, warmup, activation=act)
        return {"only": what, **r}
    if what in ("decode", "decode4", "decode16"):
        return {"only": what, **decode_case(rt, wl, {"decode": 1, "decode4": 4, "decode16": 16}[what], steps, warmup)}
    if what in ("gemm_prefill_up", "gemm_prefill_down"):
        name = what[13:]
        k, n = wl.CONFIG5_SHAPES[name]
        c = wl.config5(name, M=8)
        r = gemm_case(rt, wl, f"config5 prefill {name}", 2048, k, n, c["W"], c["w_scale"], steps, warmup, "f32",
                      headline=True)
        return {"only": what, **r}
    if what == "config3":
        return {"only": what, **qlinear_case(rt, wl, steps, warmup)}
    if what in ("chain", "chain_limits", "chain128", "chain128_limits"):
        return {"only": what, **chain_case(rt, wl, 128 if "128" in what else 4096, steps, warmup,
                                           what.endswith("limits"))}
    if what == "decode16_limits":
        return {"only": what, **decode_limits_case(rt, wl, 16, steps, warmup)}
    if what == "qlinear_ffn_up":
        return {"only": what, **qlinear_ffn_up_case(rt, wl, steps, warmup)}
    if what in ("config1", "config1_two_calls"):
        r = config1_cases(rt, wl, steps, warmup, only="fused" if what == "config1" else "separate")
        return {"only": what, **r}
    if what.startswith("dynamic_quantize_"):
        return {"only": what, **dql_activation_cases(rt, steps, warmup, only=what)[what]}
    # "<op>" is the aligned config 2 tensor, "<op>_ragged" the [8191, 32767] one
    ragged = what.endswith("_ragged")
    op = what[:-len("_ragged")] if ragged else what
    rows, cols = (8191, 32767) if ragged else (8192, 32768)
    r = qdq_cases(rt, wl, rows, cols, steps, warmup, only=op)
    return {"only": what, "shape": [rows, cols], **r[op]}


def sig(x, digits=5):
    """Floats to `digits` significant digits, through any nesting."""
    if isinstance(x, float):
        return float(f"{x:.{digits}g}")
    if isinstance(x, dict):
        return {k: sig(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [sig(v, digits) for v in x]
    return x


# What a measurement keeps in the one JSON line; everything else (percentiles,
# launch counts, pre-heat times, byte counts) goes to the detail file.
_LINE_KEYS = ("name", "M", "K", "N", "kernel_us", "tops", "gbs", "hbm_frac", "hbm_frac_at_algorithmic_bytes",
              "kernel", "buffer_sets")


def for_line(x):
    """A measurement (or a nesting of them) reduced to the fields of _LINE_KEYS,
    the kernel time in microseconds."""
    if isinstance(x, list):
        return [for_line(v) for v in x]
    if isinstance(x, dict) and "kernel_ms" in x:
        y = dict(x, kernel_us=x["kernel_ms"] * 1e3)
        if "kernel" in y:
            y["kernel"] = y["kernel"].split(" (")[0]
        return {k: y[k] for k in _LINE_KEYS if k in y}
    if isinstance(x, dict):
        return {k: for_line(v) for k, v in x.items()}
    return x


def config_summary(main_res, extras):
    """The figures of the five benchmark configurations, compact enough to sit
    at the very end of the line (a reader that keeps only the line's last 2000
    characters still sees every configuration): kernel time in microseconds by
    HIP events, with TOP/s and the fraction of the 5 POP/s int8 peak for the
    GEMMs, GB/s and the fraction of 8 TB/s for the bandwidth-bound ops."""
    def us(r):
        return r["kernel_ms"] * 1e3

    def gemm(r):
        t = r.get("kernel_tops", r.get("tops"))
        return [us(r), t, t / INT8_PEAK_TOPS]

    def bw(r):
        return [us(r), r["gbs"], r["hbm_frac"]]

    out = {"units": "GEMM [us, TOP/s, frac of 5 POP/s]; Q/DQ and decode [us, GB/s, frac of 8 TB/s]"}
    c1 = extras.get("config1", {})
    if c1:
        out["c1_128x768x768"] = {("fused_one_call" if "one call" in k else "two_calls"): gemm(v) for k, v in c1.items()}
    for key, name in (("qdq_8192x32768", "c2_8192x32768"), ("qdq_8191x32767", "c2_8191x32767")):
        if key in extras:
            short = {"quantize_per_axis": "q_axis", "dequantize_per_axis": "dq_axis", "quantize_per_tensor": "q_tensor",
                     "dequantize_per_tensor": "dq_tensor", "dynamic_quantize": "dql"}
            out[name] = {short[k]: bw(v) for k, v in extras[key].items()}
    gemms = {g["name"]: g for g in extras.get("gemm", [])}
    fused = {g["name"]: g for g in extras.get("fused", [])}
    for k, g in gemms.items():
        if k.startswith("config3"):
            out["c3_512x1024x4096_qlinear"] = gemm(g)
    c4 = {"ffn_up": gemm(main_res)}
    for k, g in gemms.items():
        if k.startswith("config4") and "int32" not in k and "QLinear" not in k:
            c4.setdefault(k.split()[1], gemm(g))
        elif k.startswith("config4") and "QLinear" in k:
            c4["ffn_up_qlinear_u8_out"] = gemm(g)
    for k, g in fused.items():
        c4["fused_" + k.split()[1] + ("_gelu" if "Gelu" in k else "")] = gemm(g)
    if "ffn_block" in extras:
        c4["ffn_block_us"] = {k: v["kernel_ms"] * 1e3 for k, v in extras["ffn_block"].items()}
    out["c4_M4096"] = c4
    c5 = {}
    for k, g in gemms.items():
        if k.startswith("config5"):
            c5["prefill_" + k.split()[2]] = gemm(g)
    for d in extras.get("decode", []):
        c5[f"decode_M{d['M']}"] = bw(d)
    if c5:
        out["c5"] = c5
    return sig(out, 4)


def host_cpu():
    """Model name and logical CPU counts of the host (as the OS reports them)."""
    name = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    name = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count()
    return {"model": name, "logical_cpus": os.cpu_count(), "usable_cpus": usable}


def cpu_baseline_gemm(oracle, wl, M, K, N, budget_s=20.0):
    """The oracle's restatement of the reference's CPU pass structure for the
    same MatMulInteger + Cast + Mul, timed on this host's cores."""
    c = wl.config4("ffn_up", M=M)
    rng = np.random.default_rng(7)
    A = rng.integers(0, 256, (M, K), dtype=np.uint8)
    az = np.array(131, np.uint8)
    t0 = time.perf_counter()
    acc = oracle.matmul_integer(A, c["W"], az, None, passes=True)
    oracle.dequant_epilogue(acc, np.float32(0.0173), c["w_scale"])
    first = time.perf_counter() - t0
    reps = int(max(1, min(10, budget_s / max(first, 1e-3) - 1)))
    times = [first]
    for _ in range(reps):
        t0 = time.perf_counter()
        acc = oracle.matmul_integer(A, c["W"], az, None, passes=True)
        oracle.dequant_epilogue(acc, np.float32(0.0173), c["w_scale"])
        times.append(time.perf_counter() - t0)
    best = float(np.median(times))
    return {"value": 2.0 * M * N * K / best / 1e12, "unit": "TOPS", "cores": oracle.num_threads(),
            "kind": "port", "host": host_cpu(),
            "sample": f"full M={M} K={K} N={N} MatMulInteger+Cast+Mul, median of {len(times)} runs of the "
                      "oracle's restatement of the reference's CPU passes (int32 copies, zero-point "
                      "passes, 4x8x8-blocked int32 GEMM, OpenMP over row tiles); not onnx-mlir codegen",
            "seconds_per_step": best}


def onnx_mlir_leg(A, W, az, a_scale, w_scale, gpu_y, budget_s=20.0):
    """The reference's own CPU code for the headline op, when its compiler is
    installed on this host: `onnx-mlir -O3 --parallel` builds
    bench/models/cfg4_matmulinteger.mlir (MatMulInteger -> Cast -> Mul, the same
    graph the GPU number is for) into a shared library, whose run_main_graph is
    then called on the same operands through the OMTensor C API that every
    compiled model exports (include/OnnxMlirRuntime.h of the reference).  Returns
    None when there is no `onnx-mlir` on PATH -- the case on every box this was
    written on, so this leg has never run -- and a dict with "error" when a step
    of it fails."""
    import ctypes, shutil, subprocess, tempfile
    exe = shutil.which("onnx-mlir")
    if exe is None:
        return None
    model = os.path.join(ROOT, "bench", "models", "cfg4_matmulinteger.mlir")
    try:
        with tempfile.TemporaryDirectory() as tmp:
            base = os.path.join(tmp, "cfg4_matmulinteger")
            r = subprocess.run([exe, "-O3", "--parallel", model, "-o", base],
                               capture_output=True, text=True, timeout=600)
            if r.returncode != 0:
                return {"error": "onnx-mlir failed: " + r.stderr[-400:]}
            so = ctypes.CDLL(base + ".so")
            vp, i64 = ctypes.c_void_p, ctypes.c_int64
            so.omTensorCreate.restype, so.omTensorCreate.argtypes = vp, [vp, ctypes.POINTER(i64), i64, ctypes.c_int]
            so.omTensorListCreate.restype, so.omTensorListCreate.argtypes = vp, [ctypes.POINTER(vp), i64]
            so.run_main_graph.restype, so.run_main_graph.argtypes = vp, [vp]
            so.omTensorListGetOmtByIndex.restype, so.omTensorListGetOmtByIndex.argtypes = vp, [vp, i64]
            so.omTensorGetDataPtr.restype, so.omTensorGetDataPtr.argtypes = vp, [vp]
            so.omTensorListDestroy.restype, so.omTensorListDestroy.argtypes = None, [vp]
            onnx_type = {np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int8): 3}
            arrays = [np.ascontiguousarray(x) for x in
                      (A, W, az, np.array(a_scale, np.float32), np.asarray(w_scale, np.float32))]
            tensors = (vp * len(arrays))()
            shapes = []
            for i, x in enumerate(arrays):
                shp = (i64 * max(x.ndim, 1))(*x.shape)
                shapes.append(shp)
                tensors[i] = so.omTensorCreate(x.ctypes.data, shp, x.ndim, onnx_type[x.dtype])
            inputs = so.omTensorListCreate(tensors, len(arrays))

            def run():
                t0 = time.perf_counter()
                out = so.run_main_graph(inputs)
                dt = time.perf_counter() - t0
                if not out:
                    raise RuntimeError("run_main_graph returned NULL")
                return out, dt

            out, first = run()
            y = np.ctypeslib.as_array(ctypes.cast(so.omTensorGetDataPtr(so.omTensorListGetOmtByIndex(out, 0)),
                                                  ctypes.POINTER(ctypes.c_float)), shape=gpu_y.shape)
            same = bool(np.array_equal(y.view(np.uint32), gpu_y.view(np.uint32)))
            so.omTensorListDestroy(out)
            times = [first]
            for _ in range(int(max(1, min(10, budget_s / max(first, 1e-3) - 1)))):
                out, dt = run()
                so.omTensorListDestroy(out)
                times.append(dt)
        M, K = A.shape
        N = W.shape[1]
        best = float(np.median(times))
        return {"value": 2.0 * M * N * K / best / 1e12, "unit": "TOPS", "cores": host_cpu()["usable_cpus"],
                "kind": "reference", "host": host_cpu(), "seconds_per_step": best,
                "bit_identical_to_gpu_output": same,
                "sample": f"full M={M} K={K} N={N} MatMulInteger+Cast+Mul, median of {len(times)} calls of "
                          "run_main_graph of bench/models/cfg4_matmulinteger.mlir built by `onnx-mlir -O3 --parallel`"}
    except Exception as e:                                   # noqa: BLE001 -- an optional leg must not end the bench
        return {"error": f"{type(e).__name__}: {e}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="config4_ffn_up",
                    choices=["config4_ffn_up", "config4_ffn_up_i32"])
    ap.add_argument("--no-extras", action="store_true", help="skip the Q/DQ and other-shape measurements")
    ap.add_argument("--extras", default="config1,gemm,fused,decode,qdq", help="which extra groups to measure")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--only", default=None,
                    choices=["copy", "mfma_ceiling", "per_axis_layouts", "gemm_ffn_up", "gemm_qkv", "gemm_out", "gemm_ffn_down",
                             "gemm_prefill_up", "gemm_prefill_down", "fused_ffn_up", "fused_ffn_down",
                             "fused_ffn_up_relu", "fused_ffn_up_gelu",
                             "decode", "decode4", "decode16", "config1", "config1_two_calls", "config3", "qlinear_ffn_up", "chain", "chain_limits", "chain128", "chain128_limits", "decode16_limits",
                             "quantize_per_axis", "dequantize_per_axis",
                             "quantize_per_tensor", "dequantize_per_tensor", "dynamic_quantize",
                             "quantize_per_axis_ragged", "dequantize_per_axis_ragged",
                             "dynamic_quantize_4096x768", "dynamic_quantize_4096x3072"],
                    help="launch just this kernel --steps times (for rocprofv3 counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import om_mi355x as rt
    from om_mi355x import workloads as wl
    rt.load()                       # raises if the HIP library is not built
    info = rt.device_info()         # raises if there is no gfx950 device
    if args.only:
        print(json.dumps(only_mode(rt, wl, args.only, args.steps, args.warmup)))
        return

    M, K, N = 4096, 768, 3072
    c = wl.config4("ffn_up", M=8)   # weights and scales only; activations are made in gemm_case
    epi = "f32" if args.workload == "config4_ffn_up" else "i32"
    main_res = gemm_case(rt, wl, "config4 FFN-up", M, K, N, c["W"], c["w_scale"],
                         args.steps, args.warmup, epi, headline=True)

    extras = {}
    groups = set() if args.no_extras else set(args.extras.split(","))
    esteps, ewarm = args.steps, min(args.warmup, 50)   # every extra is pre-heated as well
    # The bandwidth-bound groups run first: after the seconds of matrix-core work
    # of the gemm group the weight-streaming decode kernel takes 1.8 us longer per
    # launch (10.5 against 8.7 us at M=1, the same in a kernel trace).
    if "decode" in groups:
        extras["decode"] = [decode_case(rt, wl, m, esteps, ewarm) for m in (1, 4, 16)]
    if "config1" in groups:
        extras["config1"] = config1_cases(rt, wl, esteps, ewarm)
    if "qdq" in groups:
        qsteps = min(max(MIN_LAUNCHES, args.steps // 10), 200)
        extras["qdq_8192x32768"] = qdq_cases(rt, wl, 8192, 32768, qsteps, 2)
        extras["qdq_8191x32767"] = qdq_cases(rt, wl, 8191, 32767, qsteps, 2)
    if "qdq" in groups:
        extras["dql_activations"] = dql_activation_cases(rt, esteps, ewarm)
    if "fused" in groups:
        fused = []
        for name, (k, n) in wl.CONFIG4_SHAPES.items():
            if name in ("ffn_up", "ffn_down"):
                cc = wl.config4(name, M=8)
                fused.append(fused_case(rt, wl, f"config4 {name} fused layer", 4096, k, n, cc["W"],
                                        cc["w_scale"], esteps, ewarm))
                if name == "ffn_up":   # the projection an activation function follows
                    fused.append(fused_case(rt, wl, f"config4 {name} fused layer, Gelu", 4096, k, n, cc["W"],
                                            cc["w_scale"], esteps, ewarm, activation=2))
        extras["fused"] = fused
        # the feed-forward block as two fused layers in a row, without and with
        # the first layer's limits handed to the second
        extras["ffn_block"] = {"plain": chain_case(rt, wl, 4096, esteps, ewarm, False),
                               "limits": chain_case(rt, wl, 4096, esteps, ewarm, True)}
    if "gemm" in groups:
        gemms = []
        for name, (k, n) in wl.CONFIG4_SHAPES.items():
            cc = wl.config4(name, M=8)
            gemms.append(gemm_case(rt, wl, f"config4 {name}", 4096, k, n, cc["W"], cc["w_scale"],
                                   esteps, ewarm, "f32"))
        gemms.append(gemm_case(rt, wl, "config4 FFN-up int32 out", M, K, N, c["W"], c["w_scale"],
                               esteps, ewarm, "i32"))
        for name, (k, n) in wl.CONFIG5_SHAPES.items():
            cc = wl.config5(name, M=8)
            gemms.append(gemm_case(rt, wl, f"config5 prefill {name}", 2048, k, n, cc["W"], cc["w_scale"],
                                   min(max(MIN_LAUNCHES, args.steps // 10), 500), 2, "f32"))
        gemms.append(qlinear_case(rt, wl, esteps, ewarm))
        gemms.append(qlinear_ffn_up_case(rt, wl, esteps, ewarm))
        extras["gemm"] = gemms
        extras["headline_rotated"] = rotated_case(rt, wl, M, K, N, c["W"], c["w_scale"], esteps, ewarm)

    cpu = None
    if not args.no_cpu:
        import oracle_lib
        cpu = cpu_baseline_gemm(oracle_lib.load(), wl, M, K, N)
        # The reference's own compiled model, where its compiler is installed.
        rng = np.random.default_rng(7)
        A = rng.integers(0, 256, (M, K), dtype=np.uint8)
        az, a_scale = np.array(131, np.uint8), np.float32(0.0173)
        gpu_y = rt.MatMulIntegerDequant(A, c["W"], az, None, a_scale, c["w_scale"], None)
        ref = onnx_mlir_leg(A, c["W"], az, a_scale, c["w_scale"], gpu_y)
        if ref is not None and "error" not in ref:
            ref["port"] = cpu
            cpu = ref
        else:
            cpu["onnx_mlir"] = ref if ref is not None else "not on PATH"

    traffic = None
    rec = traffic_record() if epi == "f32" else None
    if rec and rec.get("kernel") == main_res["kernel"]:
        traffic = rec.get("traffic_bytes")
    hbm_bytes = main_res["hbm_bytes_algorithmic"]
    # What the matrix cores of this device deliver fed from registers alone, a few
    # milliseconds each: the published peak assumes the top clock, which the device
    # does not hold once the operands are random bytes (as the benchmark's are).
    ceiling = {"random_operands": rt.mfma_ceiling(True), "small_constant_operands": rt.mfma_ceiling(False)}
    line = {
        "metric": METRIC,
        "value": main_res["tops"],
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": f"config4 FFN-up MatMulInteger M={M} K={K} N={N}, uint8 activations x int8 "
                               f"weights, a_zp scalar, {'per-column fp32 dequant' if epi == 'f32' else 'int32'} "
                               "output, operands resident in HBM, weights packed once",
                   "preheat_ms": main_res["preheat_ms"]},
        "roofline": {"bound": "mfma", "achieved": main_res["kernel_tops"], "peak": INT8_PEAK_TOPS,
                     "unit": "TOP/s", "frac": main_res["kernel_tops"] / INT8_PEAK_TOPS,
                     "traffic": traffic,
                     "traffic_source": ({"file": "profiles/headline_traffic.json", "commit": rec.get("commit")}
                                        if traffic else None),
                     "kernel": main_res["kernel"], "kernel_ms": main_res["kernel_ms"],
                     "algorithmic_ops": main_res["ops"],
                     "algorithmic_hbm_bytes": hbm_bytes,
                     "hbm_frac_at_algorithmic_bytes": hbm_bytes / (main_res["kernel_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "hbm_bound_tops": main_res["ops"] / (hbm_bytes / (HBM_PEAK_GBS * 1e9)) / 1e12,
                     "measured_mfma_ceiling": ceiling},
        "cpu_baseline": cpu,
        "device": info,
    }
    # Everything measured, in full, beside the line; the line itself carries the
    # extras reduced to their figures and ends with the per-configuration summary.
    detail = dict(line, extras=extras)
    try:
        os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
        with open(os.path.join(ROOT, "gpurun_out", "bench_detail.json"), "w") as f:
            json.dump(detail, f)
        line["detail_file"] = "gpurun_out/bench_detail.json"
    except OSError:
        line["detail_file"] = None
    # (the feed-forward block's pair is in the summary and in the detail file)
    line["extras"] = for_line({k: v for k, v in extras.items() if k != "ffn_block"})
    line["configs"] = config_summary(main_res, extras)
    print(json.dumps(sig(line), separators=(",", ":")))


if __name__ == "__main__":
    main()
