"""Run one benchmark graph through the runtime the way a compiled model would,
and report wall-clock inference times in the format of the reference's model
driver (utils/RunONNXModel.py:1083-1104, 1139-1160): per-iteration lines, then
min / max / mean / stdev over all iterations and over the middle two quartiles.

    python -m om_mi355x.run_config --config 4 --layer ffn_up -n 50 --warmup 5
    python -m om_mi355x.run_config --config 4 --layer ffn_up --plan fused
    python -m om_mi355x.run_config --config 2 --enable-fast-math --disable-quantization-zero-point

Plans (what the accelerator's compiler passes would have produced):
  unfused  one call per ONNX op; Cast and Mul, which are not offloaded, run on
           the host (numpy); every tensor is a host buffer
  kept     the same calls, the tensors that only offloaded ops touch backed by
           GPU memory (om_mi355x_KeepOnDevice / om_mi355x_Release around them)
  fused    the chain as one om_mi355x_DynQuantMatMulDequant call
Inputs and outputs of the graph are always host buffers, weights are declared
constant once, as a model does at its first inference.
"""
from __future__ import annotations

import argparse
import os
import sys
import time

import numpy as np

import om_mi355x as rt
from om_mi355x import workloads as wl


def ordinal(n: int) -> str:
    suffix = "th" if 10 <= n % 100 <= 20 else {1: "st", 2: "nd", 3: "rd"}.get(n % 10, "th")
    return f"{n}{suffix}"


def middle_quartiles(values):
    v = np.sort(np.asarray(values))
    cut = len(v) * 25 // 100
    return v[cut:len(v) - cut] if len(v) - 2 * cut > 0 else v


def linear_layer(x, w, w_scale, plan):
    """DynamicQuantizeLinear -> MatMulInteger -> Cast -> Mul(a_scale * w_scale)."""
    rt.mark_constant(w)
    w_scale = np.ascontiguousarray(w_scale, np.float32)
    if plan == "fused":
        rt.mark_constant(w_scale)
        return lambda: rt.DynQuantMatMulDequant(x, w, None, w_scale)
    M, N = x.shape[0], w.shape[1]
    aq = np.empty(x.shape, np.uint8)
    a_s = np.empty((), np.float32)
    a_z = np.empty((), np.uint8)
    acc = np.empty((M, N), np.int32)
    kept = [aq, a_z] if plan == "kept" else []      # a_s and acc are read by host ops

    def run():
        for t in kept:
            rt.keep_on_device(t)
        try:
            rt.DynamicQuantizeLinear(x, out=(aq, a_s, a_z))
            rt.MatMulInteger(aq, w, a_z, None, out=acc)
        finally:
            for t in kept:
                rt.release(t)
        return acc.astype(np.float32) * (a_s * w_scale)

    return run


def build(args):
    c, plan = args.config, args.plan
    if c == 1:
        d = wl.config1()
        return linear_layer(d["A"], d["B"], np.float32(d["b_scale"]), plan)
    if c == 2:
        d = wl.config2(args.rows, args.cols)
        x, sc, zp = d["X"], d["scale"], d["zp"]

        def run():
            q = rt.QuantizeLinear(x, sc, zp, axis=1)
            y = rt.DequantizeLinear(q, sc, zp, axis=1)
            return y, rt.DynamicQuantizeLinear(x)

        return run
    if c == 3:
        d = wl.config3()
        rt.mark_constant(d["B"])
        return lambda: rt.QLinearMatMul(d["A"], d["a_scale"], d["a_zp"], d["B"], d["b_scale"],
                                        d["b_zp"], d["y_scale"], d["y_zp"])
    if c == 4:
        d = wl.config4(args.layer or "ffn_up", M=args.m or 4096)
        return linear_layer(d["X"], d["W"], d["w_scale"], plan)
    if c == 5:
        d = wl.config5(args.layer or "up", M=args.m or 2048)
        return linear_layer(d["X"], d["W"], d["w_scale"], plan)
    raise SystemExit(f"unknown config {c}")


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--config", type=int, required=True, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--layer", default=None, help="config 4: qkv|out|ffn_up|ffn_down; config 5: up|down")
    ap.add_argument("--m", type=int, default=None, help="rows of the activation (configs 4 and 5)")
    ap.add_argument("--rows", type=int, default=8192, help="config 2")
    ap.add_argument("--cols", type=int, default=32768, help="config 2")
    ap.add_argument("--plan", default="unfused", choices=["unfused", "kept", "fused"])
    ap.add_argument("-n", "--n-iteration", type=int, default=10)
    ap.add_argument("-w", "--warmup", type=int, default=2)
    ap.add_argument("--enable-fast-math", action="store_true",
                    help="compute as a model compiled with -O3 --enable-fast-math does (quotient as x * (1 / scale))")
    ap.add_argument("--disable-quantization-zero-point", action="store_true",
                    help="compute as a model compiled with --disable-quantization-zero-point does")
    args = ap.parse_args(argv)

    rt.load()
    print("  device:", rt.device_info())
    # what the accelerator's patterns would put in front of the quantize ops
    rt.set_quant_mode((rt.QUANT_RECIPROCAL if args.enable_fast_math else 0) |
                      (rt.QUANT_NO_ZERO_POINT if args.disable_quantization_zero_point else 0))
    run = build(args)
    for i in range(args.warmup):
        t0 = time.perf_counter()
        run()
        print("  {} warmup: {} seconds".format(ordinal(i + 1), time.perf_counter() - t0))
    perf = []
    for i in range(args.n_iteration):
        t0 = time.perf_counter()
        run()
        perf.append(time.perf_counter() - t0)
        print("  {} iteration, {}, seconds".format(ordinal(i + 1), perf[-1]))
    if len(perf) > 1:
        for label, v in (("Statistics 1 (excluding warmup),", perf),
                         ("Statistics 2 (no warmup/quart.),", middle_quartiles(perf))):
            print("  {} min, {:.6e}, max, {:.6e}, mean, {:.6e}, stdev, {:.6e}".format(
                label, np.min(v), np.max(v), np.mean(v), np.std(v, dtype=np.float64)))
    return 0


if __name__ == "__main__":
    sys.exit(main())
