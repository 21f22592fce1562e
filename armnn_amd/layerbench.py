"""Time one quantized layer on the device through the C ABI and price it against its roofline.

  python -m armnn_amd.layerbench conv --n 64 --h 14 --w 14 --ci 512 --co 512 --k 1
  python -m armnn_amd.layerbench dw   --n 64 --h 112 --w 112 --c 32 --stride 1
  python -m armnn_amd.layerbench fc   --m 2048 --k 4096 --o 4096
  python -m armnn_amd.layerbench pad  --n 64 --h 112 --w 112 --c 64        (one row and column on every side)
  python -m armnn_amd.layerbench add  --n 16 --h 56 --w 56 --c 256         (Addition of two tensors with a fused ReLU)
  python -m armnn_amd.layerbench dwpw --n 64 --h 14 --w 14 --c 512 --co 512 --stride 1
                                                                           (3x3 depthwise + the 1x1 convolution behind it, as
                                                                            one launch: mi355x_conv2d_run_fused)
  python -m armnn_amd.layerbench tail --n 64 --h 7 --w 7 --c 1024 --o 1001 (global average pooling -> FullyConnected ->
                                                                            Softmax: three launches and one launch)

Prints one JSON line: kernel chosen, average launch time (HIP events on the launch stream), algorithmic
ops and bytes, and the fraction of the int8 MFMA peak (5.0 POP/s) or of the HBM peak (8 TB/s).
Inputs are seeded synthetic data; nothing is checked here (parity lives in tests/).
"""
from __future__ import annotations

import argparse
import json
import sys

import numpy as np

from . import shim, synth
from .tensor import DataType, QTensor, TensorInfo

INT8_PEAK = 5.0e15
HBM_PEAK = 8.0e12


def _same(in_size, k, stride):
    out = (in_size + stride - 1) // stride
    total = max((out - 1) * stride + k - in_size, 0)
    return out, total // 2


def _pad(dev, a, adt, zp):
    """A constant Pad of one row and column on every side of an NHWC tensor: one byte read per input element, one
    written per output element."""
    import ctypes as C
    xin = TensorInfo((a.n, a.h, a.w, a.c), adt, (0.0235,), zp)
    yout = TensorInfo((a.n, a.h + 2, a.w + 2, a.c), adt, (0.0235,), zp)
    d = shim.pad_desc(xin.shape, ((0, 0), (1, 1), (1, 1), (0, 0)), float(zp), xin, yout)
    lib = shim.load_library()
    xd = shim.DeviceBuffer(xin.num_elements).upload(synth.uniform_int(1, xin.shape, 0, 127, np.uint8))
    yd = shim.DeviceBuffer(yout.num_elements)
    stream = dev.stream()
    run = lambda: shim._chk(lib.mi355x_pad_run(C.byref(d), xd.ptr, yd.ptr, stream))
    for _ in range(a.warmup):
        run()
    e0, e1 = dev.event(), dev.event()
    dev.event_record(e0, stream)
    for _ in range(a.iters):
        run()
    dev.event_record(e1, stream)
    dev.event_sync(e1)
    ms = dev.elapsed_ms(e0, e1) / a.iters
    nbytes = xin.num_elements + yout.num_elements
    print(json.dumps({"layer": f"pad N={a.n} {a.h}x{a.w}x{a.c} by 1 on height and width", "kernel": "PadKernel", "us": ms * 1e3,
                      "GBps": nbytes / (ms * 1e-3) / 1e9, "frac_hbm_peak": nbytes / (ms * 1e-3) / HBM_PEAK, "bytes": nbytes}))
    return 0


def _timed(dev, stream, run, a):
    for _ in range(a.warmup):
        run()
    e0, e1 = dev.event(), dev.event()
    dev.event_record(e0, stream)
    for _ in range(a.iters):
        run()
    dev.event_record(e1, stream)
    dev.event_sync(e1)
    return dev.elapsed_ms(e0, e1) / a.iters


def _add(dev, a, adt, zp):
    """Addition of two NHWC tensors with a fused ReLU, quantization scales from --scales: two bytes read and one written per
    element."""
    import ctypes as C
    lo = 0 if a.u8 else -128
    shape = (a.n, a.h, a.w, a.c)
    s0, s1, so = a.scales
    q0, q1, qo = TensorInfo(shape, adt, (s0,), lo), TensorInfo(shape, adt, (s1,), lo), TensorInfo(shape, adt, (so,), lo)
    lib = shim.load_library()
    n = q0.num_elements
    x0 = shim.DeviceBuffer(n).upload(synth.uniform_int(1, shape, 0, 255, np.uint8))
    x1 = shim.DeviceBuffer(n).upload(synth.uniform_int(2, shape, 0, 255, np.uint8))
    y = shim.DeviceBuffer(n)
    stream = dev.stream()
    a0, a1, ao = shim._quant(q0), shim._quant(q1), shim._quant(qo)
    run = lambda: shim._chk(lib.mi355x_add_run(n, C.byref(a0), C.byref(a1), C.byref(ao), shim.ACT_RELU, 0.0, 0.0, x0.ptr, x1.ptr, y.ptr, stream))
    ms = _timed(dev, stream, run, a)
    print(json.dumps({"layer": f"add N={a.n} {a.h}x{a.w}x{a.c} + ReLU, scales {s0} + {s1} -> {so}", "kernel": shim.last_kernel(), "us": ms * 1e3, "elements": n,
                      "GBps": 3 * n / (ms * 1e-3) / 1e9, "frac_hbm_peak": 3 * n / (ms * 1e-3) / HBM_PEAK, "bytes": 3 * n}))
    return 0


def _dwpw(dev, a, adt, zp):
    """3x3 depthwise (ReLU6) + 1x1 convolution (ReLU6) over uint8-style activations, as MobileNetV1 has them, run as one
    launch; algorithmic bytes: input + output + both layers' constants (the tensor between them never exists)."""
    lo = 0 if a.u8 else -128
    ho, pt = _same(a.h, 3, a.stride)
    wo, pl = _same(a.w, 3, a.stride)
    xin = TensorInfo((a.n, a.h, a.w, a.c), adt, (0.0235,), lo)
    mid = TensorInfo((a.n, ho, wo, a.c), adt, (0.0235,), lo)
    yout = TensorInfo((a.n, ho, wo, a.co), adt, (0.0235,), lo)
    wsd = synth.scales(3, a.c) / np.float32(1.0)
    wd = QTensor(TensorInfo((1, 3, 3, a.c), DataType.QSymmS8, tuple(wsd), 0, 3), synth.int8_weights(2, (1, 3, 3, a.c)))
    bd = QTensor(TensorInfo((a.c,), DataType.Signed32, tuple(np.float32(0.0235) * wsd), 0, 0), synth.int32_bias(4, a.c))
    wsp = synth.scales(5, a.co) / np.float32(np.sqrt(a.c) / 3.0)
    wp = QTensor(TensorInfo((a.co, 1, 1, a.c), DataType.QSymmS8, tuple(wsp), 0, 0), synth.int8_weights(6, (a.co, 1, 1, a.c)))
    bp = QTensor(TensorInfo((a.co,), DataType.Signed32, tuple(np.float32(0.0235) * wsp), 0, 0), synth.int32_bias(7, a.co))
    act = (shim.ACT_BOUNDED_RELU, 6.0, 0.0)
    pdw = shim.Conv2dPlan(xin, wd, bd, mid, pad_top=pt, pad_left=pl, stride_x=a.stride, stride_y=a.stride, depthwise=True,
                          activation=act[0], act_a=act[1], act_b=act[2])
    ppw = shim.Conv2dPlan(mid, wp, bp, yout, activation=act[0], act_a=act[1], act_b=act[2])
    if not pdw.fusable_with(ppw):
        raise SystemExit("the pair is not fusable: " + shim.load_library().mi355x_last_error().decode())
    xd = shim.DeviceBuffer(xin.num_elements).upload(synth.uniform_int(1, xin.shape, 0, 255, np.uint8))
    yd = shim.DeviceBuffer(yout.num_elements)
    stream = dev.stream()
    ms = _timed(dev, stream, lambda: pdw.run_fused(ppw, a.n, xd.ptr, yd.ptr, stream), a)
    nbytes = xin.num_elements + yout.num_elements + 9 * a.c + 8 * a.c + a.c * a.co + 8 * a.co
    ops = 2.0 * a.n * ho * wo * a.co * a.c
    print(json.dumps({"layer": f"dw3x3 s{a.stride} + pw N={a.n} {a.h}x{a.w}x{a.c}->{a.co}", "kernel": shim.last_kernel(), "us": ms * 1e3,
                      "GBps": nbytes / (ms * 1e-3) / 1e9, "frac_hbm_peak": nbytes / (ms * 1e-3) / HBM_PEAK, "bytes": nbytes,
                      "pointwise_TOPS": ops / (ms * 1e-3) / 1e12, "recommended_by_the_library": bool(pdw.fusion_pays(ppw, a.n))}))
    return 0


def _tail(dev, a, adt, zp):
    """Global average pooling -> FullyConnected -> Softmax over a.n images of a.h x a.w x a.c with a.o classes: the three
    launches one behind the other, and the one launch of mi355x_tail_run (same bytes)."""
    import ctypes as C
    lo = 0 if a.u8 else -128
    lib = shim.load_library()
    xin = TensorInfo((a.n, a.h, a.w, a.c), adt, (0.0235,), lo)
    pooled = TensorInfo((a.n, a.c), adt, (0.0235,), lo)
    logits = TensorInfo((a.n, a.o), adt, (0.1,), lo + 70)
    probs = TensorInfo((a.n, a.o), adt, (1.0 / 256,), lo)
    ws = synth.scales(3, a.o)
    w = QTensor(TensorInfo((a.o, a.c), DataType.QSymmS8, tuple(ws), 0, 0), synth.int8_weights(2, (a.o, a.c)))
    b = QTensor(TensorInfo((a.o,), DataType.Signed32, tuple(np.float32(0.0235) * ws), 0, 0), synth.int32_bias(4, a.o))
    fc = shim.FullyConnectedPlan(pooled, w, b, logits)
    d = shim.Pool2dDesc(a.h, a.w, a.c, 1, 1, a.w, a.h, 1, 1, 0, 0, 0, 0, 1, 1, shim._quant(xin), shim._quant(pooled))
    tail = shim.ClassifierTail(d, fc, 1.0, probs)
    xd = shim.DeviceBuffer(xin.num_elements).upload(synth.uniform_int(1, xin.shape, 0, 255, np.uint8))
    pd, ld, yd = shim.DeviceBuffer(pooled.num_elements), shim.DeviceBuffer(logits.num_elements), shim.DeviceBuffer(probs.num_elements)
    stream = dev.stream()
    qi, qo = shim._quant(logits), shim._quant(probs)

    def three():
        shim._chk(lib.mi355x_pool2d_run(C.byref(d), a.n, xd.ptr, pd.ptr, stream))
        fc.run(a.n, pd.ptr, ld.ptr, stream)
        shim._chk(lib.mi355x_softmax_run(a.n, a.o, 1.0, C.byref(qi), C.byref(qo), ld.ptr, yd.ptr, stream))

    ms3 = _timed(dev, stream, three, a)
    ms1 = _timed(dev, stream, lambda: tail.run(a.n, xd.ptr, pd.ptr, ld.ptr, yd.ptr, stream), a)
    kernel = shim.last_kernel()
    print(json.dumps({"layer": f"tail N={a.n} {a.h}x{a.w}x{a.c} -> {a.o}", "three_launches_us": ms3 * 1e3, "one_launch_us": ms1 * 1e3,
                      "kernel": kernel, "waits_given_up": tail.gave_up()}))
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("op", choices=["conv", "dw", "fc", "pad", "add", "tail", "dwpw"])
    ap.add_argument("--n", type=int, default=64)
    ap.add_argument("--h", type=int, default=56)
    ap.add_argument("--w", type=int, default=56)
    ap.add_argument("--ci", type=int, default=64)
    ap.add_argument("--co", type=int, default=64)
    ap.add_argument("--c", type=int, default=32)
    ap.add_argument("--k", type=int, default=3, help="kernel size (conv/dw) or K (fc)")
    ap.add_argument("--stride", type=int, default=1)
    ap.add_argument("--m", type=int, default=256)
    ap.add_argument("--o", type=int, default=4096)
    ap.add_argument("--u8", action="store_true", help="QAsymmU8 activations (default QAsymmS8)")
    ap.add_argument("--wzp", type=int, default=None, metavar="ZERO_POINT",
                    help="per-tensor QAsymmU8 weights with this zero point (default: per-channel QSymmS8)")
    ap.add_argument("--wspread", type=int, default=1, metavar="FACTOR",
                    help="with --wzp: multiply the weight draws (std 30) by this before adding the zero point; 3 spreads the "
                         "codes over the whole uint8 range, so that weight minus zero point no longer fits int8")
    ap.add_argument("--scales", type=float, nargs=3, default=(0.0235, 0.1, 0.1), metavar=("IN0", "IN1", "OUT"),
                    help="add: the three quantization scales (the default, 0.0235 + 0.1 -> 0.1, makes one sum in 200 an exact tie)")
    ap.add_argument("--algo", type=int, default=0)
    ap.add_argument("--iters", type=int, default=500, help="timed launches; long enough for the clocks to settle")
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--opt", action="append", default=[], metavar="NAME=VALUE", help="mi355x_set_option before the plan is built")
    a = ap.parse_args(argv)
    for item in a.opt:
        name, value = item.split("=")
        shim.set_option(name, int(value))

    dev = shim.Device()
    adt = DataType.QAsymmU8 if a.u8 else DataType.QAsymmS8
    zp = 128 if a.u8 else -3
    if a.op == "pad":
        return _pad(dev, a, adt, zp)
    if a.op == "add":
        return _add(dev, a, adt, zp)
    if a.op == "tail":
        return _tail(dev, a, adt, zp)
    if a.op == "dwpw":
        return _dwpw(dev, a, adt, zp)
    act = (shim.ACT_BOUNDED_RELU, 6.0, 0.0)
    if a.op == "fc":
        k, o, m = a.k if a.k > 3 else 4096, a.o, a.m
        xin = TensorInfo((m, k), adt, (0.02,), zp)
        yout = TensorInfo((m, o), adt, (1.0,), 0)
        ws = synth.scales(3, o)
        w = QTensor(TensorInfo((o, k), DataType.QSymmS8, tuple(ws), 0, 0), synth.int8_weights(2, (o, k)))
        if a.wzp is not None:
            ws = ws[:1]
            w = QTensor(TensorInfo((o, k), DataType.QAsymmU8, tuple(ws), a.wzp, None),
                        np.clip(a.wspread * synth.int8_weights(2, (o, k)).astype(np.int32) + a.wzp, 0, 255).astype(np.uint8))
        b = QTensor(TensorInfo((o,), DataType.Signed32, tuple(np.float32(0.02) * ws), 0, 0 if a.wzp is None else None), synth.int32_bias(4, o))
        plan = shim.FullyConnectedPlan(xin, w, b, yout, algo=a.algo)
        batch, macs = m, m * k * o
        nbytes = m * k + m * o + k * o + 8 * o
        desc = f"fc M={m} K={k} O={o}"
    else:
        dw = a.op == "dw"
        ci = a.c if dw else a.ci
        co = a.c if dw else a.co
        ho, pt = _same(a.h, a.k, a.stride)
        wo, pl = _same(a.w, a.k, a.stride)
        xin = TensorInfo((a.n, a.h, a.w, ci), adt, (0.0235,), zp)
        yout = TensorInfo((a.n, ho, wo, co), adt, (0.0235,), 0 if a.u8 else -128)
        wshape = (1, a.k, a.k, co) if dw else (co, a.k, a.k, ci)
        taps = a.k * a.k * (1 if dw else ci)
        ws = synth.scales(3, co) / np.float32(np.sqrt(taps) / 3.0)
        w = QTensor(TensorInfo(wshape, DataType.QSymmS8, tuple(ws), 0, 3 if dw else 0), synth.int8_weights(2, wshape))
        if a.wzp is not None:
            ws = ws[:1]
            w = QTensor(TensorInfo(wshape, DataType.QAsymmU8, tuple(ws), a.wzp, None),
                        np.clip(a.wspread * synth.int8_weights(2, wshape).astype(np.int32) + a.wzp, 0, 255).astype(np.uint8))
        b = QTensor(TensorInfo((co,), DataType.Signed32, tuple(np.float32(0.0235) * ws), 0, 0 if a.wzp is None else None), synth.int32_bias(4, co))
        plan = shim.Conv2dPlan(xin, w, b, yout, pad_top=pt, pad_left=pl, stride_x=a.stride, stride_y=a.stride,
                               depthwise=dw, activation=act[0], act_a=act[1], act_b=act[2], algo=a.algo)
        batch, macs = a.n, a.n * ho * wo * co * taps
        nbytes = xin.num_elements + yout.num_elements + w.info.num_elements + 8 * co
        desc = f"{a.op} N={a.n} {a.h}x{a.w}x{ci}->{co} k{a.k} s{a.stride}"

    lo, hi = (0, 255) if a.u8 else (-128, 127)
    xd = shim.DeviceBuffer(xin.num_elements).upload(synth.uniform_int(1, xin.shape, lo, hi, np.uint8 if a.u8 else np.int8))
    yd = shim.DeviceBuffer(yout.num_elements)
    stream = dev.stream()
    for _ in range(a.warmup):
        plan.run(batch, xd.ptr, yd.ptr, stream)
    e0, e1 = dev.event(), dev.event()
    dev.event_record(e0, stream)
    for _ in range(a.iters):
        plan.run(batch, xd.ptr, yd.ptr, stream)
    dev.event_record(e1, stream)
    dev.event_sync(e1)
    ms = dev.elapsed_ms(e0, e1) / a.iters
    ops = 2.0 * macs
    out = {"layer": desc, "kernel": plan.algo()[1], "us": ms * 1e3, "TOPS": ops / (ms * 1e-3) / 1e12,
           "GBps": nbytes / (ms * 1e-3) / 1e9, "frac_mfma_peak": ops / (ms * 1e-3) / INT8_PEAK,
           "frac_hbm_peak": nbytes / (ms * 1e-3) / HBM_PEAK, "ops": ops, "bytes": nbytes,
           "arithmetic_intensity": ops / nbytes}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
