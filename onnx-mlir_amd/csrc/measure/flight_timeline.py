"""When the blocks of k_gemm_i8_flight / k_gemm_i8_flight_dq pass each of their
phases: a build of the runtime in which wave 0 of every block reads the 100 MHz
clock at fixed points of the kernel (measure/libom_mi355x.so, -DFLIGHT_TIMING)
runs one of three calls a few thousand times; the last launch's readings are
printed as minimum / median / maximum over the blocks, in ns from the first
block's entry.

    python flight_timeline.py --case fused  --shape 128x768x768    DynQuantMatMulDequant
    python flight_timeline.py --case f32    --shape 128x768x768    MatMulIntegerDequant (u8 x i8)
    python flight_timeline.py --case q8     --shape 512x1024x4096  QLinearMatMul (u8 x u8 -> u8)

The launch time printed with it is that of the instrumented kernel, a few
tenths of a microsecond more than the product's.
"""
import argparse
import ctypes
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
import om_mi355x as rt  # noqa: E402

PHASES = {
    "fused": ["entry", "share published", "weights requested / poll over", "limits known",
              "rows in LDS", "K loop done", "stores issued", "stores acknowledged"],
    "gemm": ["entry", "half of the weights requested", "half of the rows staged", "all requested, rows staged",
             "barrier passed", "K loop done", "stores issued", "stores acknowledged"],
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--case", choices=("fused", "f32", "q8"), default="fused")
    ap.add_argument("--shape", default="128x768x768")
    ap.add_argument("--launches", type=int, default=2000)
    ap.add_argument("--operands", choices=("random", "constant"), default="random",
                    help="constant: every byte of both operands the same small value (the matrix cores "
                         "draw less power on such data, see measure/mfma_ceiling.hip)")
    args = ap.parse_args()
    M, K, N = (int(v) for v in args.shape.split("x"))
    rt.LIB_PATH = os.path.join(HERE, "libom_mi355x.so")
    if not os.path.exists(rt.LIB_PATH):
        raise SystemExit(f"{rt.LIB_PATH} is not built (make -C onnx-mlir_amd/csrc all)")
    rng = np.random.default_rng(0)
    W = rng.integers(-127, 128, (K, N)).astype(np.int8)
    S = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
    dW, dS = (rt.DeviceArray.from_numpy(x) for x in (W, S))
    rt.mark_constant(dW)
    if args.case == "fused":
        dX = rt.DeviceArray.from_numpy(rng.normal(0, 1, (M, K)).astype(np.float32))
        dY = rt.DeviceArray((M, N), np.float32)
        fn = rt.PreparedCall("om_mi355x_DynQuantMatMulDequant", dY, dX, dW, None, dS, None, 0)
    elif args.case == "q8":
        A = rng.integers(0, 256, (M, K), dtype=np.uint8)
        Bu = rng.integers(0, 256, (K, N), dtype=np.uint8)
        if args.operands == "constant":
            A[:], Bu[:] = 129, 121
        d = [rt.DeviceArray.from_numpy(np.asarray(x)) for x in
             (A, np.float32(0.01), np.uint8(128), Bu, np.float32(0.005), np.uint8(120), np.float32(0.5), np.uint8(0))]
        rt.mark_constant(d[3])
        dY = rt.DeviceArray((M, N), np.uint8)
        fn = rt.PreparedCall("om_mi355x_QLinearMatMul", dY, d[0], d[1], d[2], d[3], d[4], d[5], d[6], d[7], 0)
    else:
        dA = rt.DeviceArray.from_numpy(rng.integers(0, 256, (M, K), dtype=np.uint8))
        dAs = rt.DeviceArray.from_numpy(np.array(0.0173, np.float32))
        dAz = rt.DeviceArray.from_numpy(np.array(131, np.uint8))
        dY = rt.DeviceArray((M, N), np.float32)
        fn = rt.PreparedCall("om_mi355x_MatMulIntegerDequant", dY, dA, dW, dAz, None, dAs, dS, None, 0)
    for _ in range(args.launches):
        fn()
    rt.synchronize()
    rt.timer_start()
    for _ in range(args.launches):
        fn()
    us = rt.timer_stop() / args.launches * 1e3
    kernel = rt.last_gemm_kernel()
    print(f"{args.case} {M}x{K}x{N}: {kernel}, {us:.2f} us per launch (instrumented)")
    if "flight" not in kernel:
        raise SystemExit("this shape does not take k_gemm_i8_flight: nothing recorded")
    lib = rt.load()
    slots = 12
    buf = np.zeros(1024 * slots, np.uint64)
    lib.om_dev_flight_ts.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    if lib.om_dev_flight_ts(buf.ctypes.data, buf.nbytes) != 0:
        raise SystemExit("could not read the timestamps")
    d = buf.reshape(1024, slots)
    d = d[d[:, 0] != 0]
    names = PHASES["fused" if args.case == "fused" else "gemm"]
    t0 = d[:, 0].min()
    t = (d[:, :len(names)].astype(np.int64) - int(t0)) * 10  # 100 MHz clock -> ns
    cycles = d[:, 11].astype(np.int64) - d[:, 10].astype(np.int64)
    ns = np.maximum(t[:, len(names) - 1] - t[:, 0], 1)
    print(f"blocks {len(d)}, shader clock {float(np.median(cycles / ns)):.2f} GHz over the kernel")
    print(f"{'phase (ns after the first entry)':36s} {'min':>6s} {'median':>7s} {'max':>6s}")
    for i, name in enumerate(names):
        print(f"{name:36s} {t[:, i].min():6d} {int(np.median(t[:, i])):7d} {t[:, i].max():6d}")
    print(f"span, first entry to last acknowledgement: {t[:, len(names) - 1].max()} ns")


if __name__ == "__main__":
    main()
