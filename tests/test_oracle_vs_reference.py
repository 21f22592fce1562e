"""The C restatement must equal the reference's own code bit for bit on seeded inputs (no GPU).

Skipped where oracle/_ref is not built (it is built wherever the reference tree is mounted)."""
import numpy as np
import pytest

from armnn_amd import synth
from armnn_amd.tensor import DataType, QTensor, TensorInfo
from oracle import cpuref
from tests import cases

CONV = cases.small_conv_cases()
FC = cases.small_fc_cases()


@pytest.mark.parametrize("case", CONV, ids=[c.name for c in CONV])
def test_conv_bit_exact(port, reference, case):
    ref = reference.conv2d(case.x, case.w, case.b, case.out_info, **case.params)
    for fast in (False, True):
        got = port.conv2d(case.x, case.w, case.b, case.out_info, fast=fast, **case.params)
        np.testing.assert_array_equal(got.data, ref.data)
    fn, a, b = case.act
    if fn:
        np.testing.assert_array_equal(port.activation(ref, case.out_info, fn, a, b).data,
                                      reference.activation(ref, case.out_info, fn, a, b).data)


def test_conv_nchw_bit_exact(port, reference):
    c = cases.make_conv_case("nchw", 400, h=9, w=7, ci=5, co=6)
    x = QTensor(TensorInfo((1, 5, 9, 7), c.x.info.dtype, c.x.info.scales, c.x.info.offset), c.x.data.transpose(0, 3, 1, 2))
    w = QTensor(TensorInfo((6, 5, 3, 3), c.w.info.dtype, c.w.info.scales, 0, 0), c.w.data.transpose(0, 3, 1, 2))
    oi = TensorInfo((1, 6, 9, 7), c.out_info.dtype, c.out_info.scales, c.out_info.offset)
    r = reference.conv2d(x, w, c.b, oi, data_layout=cpuref.NCHW, **c.params)
    g = port.conv2d(x, w, c.b, oi, data_layout=cpuref.NCHW, **c.params)
    np.testing.assert_array_equal(g.data, r.data)
    # and NCHW agrees with NHWC up to the permutation (same taps, different order of cIn/ky/kx only in memory)
    nhwc = port.conv2d(c.x, c.w, c.b, c.out_info, **c.params)
    np.testing.assert_array_equal(g.data.transpose(0, 2, 3, 1), nhwc.data)


@pytest.mark.parametrize("case", FC, ids=[c.name for c in FC])
def test_fc_bit_exact(port, reference, case):
    ref = reference.fully_connected(case.x, case.w, case.b, case.out_info, transpose_weights=case.transpose_weights)
    for fast in (False, True):
        got = port.fully_connected(case.x, case.w, case.b, case.out_info, transpose_weights=case.transpose_weights, fast=fast)
        np.testing.assert_array_equal(got.data, ref.data)


@pytest.mark.parametrize("dtype,lo,hi", [(DataType.QAsymmS8, -128, 127), (DataType.QAsymmU8, 0, 255)])
def test_scalar_quantize_dequantize(port, reference, dtype, lo, hi):
    vals = synth.normal(7, (4000,), 0.0, 40.0).astype(np.float32)
    scs = synth.scales(8, 4000, 0.01, 1.0)
    offs = synth.uniform_int(9, (4000,), lo, hi, np.int64)
    for v, s, o in zip(vals, scs, offs):
        assert port.quantize(v, s, o, dtype) == reference.quantize(v, s, o, dtype)
    for q in range(lo, hi + 1):
        assert port.dequantize(q, 0.0235, 17, dtype) == reference.dequantize(q, 0.0235, 17, dtype)


@pytest.mark.parametrize("fn,a,b", [(cpuref.ACT_RELU, 0, 0), (cpuref.ACT_BOUNDED_RELU, 6, 0), (cpuref.ACT_BOUNDED_RELU, 1, -1)])
@pytest.mark.parametrize("dtype,lo,hi", [(DataType.QAsymmS8, -128, 127), (DataType.QAsymmU8, 0, 255)])
def test_activation_all_codes(port, reference, fn, a, b, dtype, lo, hi):
    """Exhaustive over the 256 codes: the layer equals an integer clamp (closed form), and port == reference."""
    codes = np.arange(lo, hi + 1)
    for scale in (0.0235, 0.05, 0.1, 1.0, 2.0):
        for zp in (lo, lo + 3, (lo + hi) // 2, hi - 5):
            info = TensorInfo((256,), dtype, (scale,), zp)
            x = QTensor(info, codes)
            r = reference.activation(x, info, fn, a, b).data
            p = port.activation(x, info, fn, a, b).data
            np.testing.assert_array_equal(p, r)
            qlo = port.quantize(b if fn == cpuref.ACT_BOUNDED_RELU else 0.0, scale, zp, dtype)
            qhi = port.quantize(a, scale, zp, dtype) if fn == cpuref.ACT_BOUNDED_RELU else hi
            np.testing.assert_array_equal(p.astype(np.int32), np.clip(codes, qlo, qhi))


POOL = [
    dict(pool_type=cpuref.POOL_AVERAGE, pool_w=7, pool_h=7, stride_x=1, stride_y=1, shape=(2, 7, 7, 16), pads=(0, 0, 0, 0)),
    dict(pool_type=cpuref.POOL_MAX, pool_w=3, pool_h=3, stride_x=2, stride_y=2, shape=(1, 12, 12, 8), pads=(0, 1, 0, 1)),
    dict(pool_type=cpuref.POOL_MAX, pool_w=3, pool_h=3, stride_x=2, stride_y=2, shape=(1, 11, 13, 5), pads=(1, 1, 1, 1)),
    dict(pool_type=cpuref.POOL_AVERAGE, pool_w=3, pool_h=2, stride_x=2, stride_y=1, shape=(1, 9, 10, 4), pads=(1, 1, 1, 0)),
]


@pytest.mark.parametrize("cfg", POOL)
@pytest.mark.parametrize("method", [cpuref.PAD_EXCLUDE, cpuref.PAD_IGNORE_VALUE])
@pytest.mark.parametrize("dtype", [DataType.QAsymmS8, DataType.QAsymmU8])
def test_pooling_bit_exact(port, reference, cfg, method, dtype):
    n, h, w, c = cfg["shape"]
    pl, pr, pt, pb = cfg["pads"]
    lo, hi = (0, 255) if dtype == DataType.QAsymmU8 else (-128, 127)
    x = QTensor(TensorInfo(cfg["shape"], dtype, (0.05,), lo + 20), synth.uniform_int(11, cfg["shape"], lo, hi, np.int64))
    ho = (h + pt + pb - cfg["pool_h"]) // cfg["stride_y"] + 1
    wo = (w + pl + pr - cfg["pool_w"]) // cfg["stride_x"] + 1
    oi = TensorInfo((n, ho, wo, c), dtype, (0.07,), lo + 9)
    kw = dict(pool_type=cfg["pool_type"], pool_w=cfg["pool_w"], pool_h=cfg["pool_h"], stride_x=cfg["stride_x"],
              stride_y=cfg["stride_y"], pad_left=pl, pad_right=pr, pad_top=pt, pad_bottom=pb, padding_method=method)
    np.testing.assert_array_equal(port.pooling2d(x, oi, **kw).data, reference.pooling2d(x, oi, **kw).data)


@pytest.mark.parametrize("dtype", [DataType.QAsymmS8, DataType.QAsymmU8])
def test_softmax_and_add_bit_exact(port, reference, dtype):
    lo, hi = (0, 255) if dtype == DataType.QAsymmU8 else (-128, 127)
    x = QTensor(TensorInfo((4, 1001), dtype, (0.1,), lo + 60), synth.uniform_int(21, (4, 1001), lo, hi, np.int64))
    oi = TensorInfo((4, 1001), dtype, (1.0 / 256,), lo)
    np.testing.assert_array_equal(port.softmax(x, oi).data, reference.softmax(x, oi).data)
    a = QTensor(TensorInfo((2, 5, 5, 16), dtype, (0.03,), lo + 10), synth.uniform_int(22, (2, 5, 5, 16), lo, hi, np.int64))
    b = QTensor(TensorInfo((2, 5, 5, 16), dtype, (0.05,), lo + 90), synth.uniform_int(23, (2, 5, 5, 16), lo, hi, np.int64))
    oi = TensorInfo((2, 5, 5, 16), dtype, (0.06,), lo + 50)
    np.testing.assert_array_equal(port.add(a, b, oi).data, reference.add(a, b, oi).data)
    b1 = QTensor(TensorInfo((1, 1, 1, 16), dtype, (0.05,), lo + 90), synth.uniform_int(24, (1, 1, 1, 16), lo, hi, np.int64))
    np.testing.assert_array_equal(port.add(a, b1, oi).data, reference.add(a, b1, oi).data)


PAD = [
    # (input shape, (before, after) per dimension, pad value, output quantization or None for the input's)
    ((2, 5, 6, 8), ((0, 0), (1, 2), (2, 1), (0, 0)), 3.0, None),
    ((1, 9, 7, 16), ((0, 0), (0, 1), (0, 1), (0, 0)), -7.0, None),
    ((2, 4, 4, 3), ((1, 0), (1, 1), (1, 1), (2, 3)), 2.5, None),          # every dimension padded; 2.5 rounds to 3
    ((3, 7), ((1, 0), (2, 3)), -300.0, (0.07, 5)),                          # saturating pad code, re-quantized elements
    ((4,), ((2, 1),), -3.5, None),
    ((2, 3, 4), ((1, 0), (0, 1), (2, 0)), 1000.0, (0.031, -2)),
]


@pytest.mark.parametrize("cfg", PAD, ids=[str(c[0]) for c in PAD])
@pytest.mark.parametrize("dtype", [DataType.QAsymmS8, DataType.QAsymmU8])
def test_pad_bit_exact(port, reference, cfg, dtype):
    shape, pads, value, outq = cfg
    lo, hi = (0, 255) if dtype == DataType.QAsymmU8 else (-128, 127)
    x = QTensor(TensorInfo(shape, dtype, (0.05,), lo + 20), synth.uniform_int(13, shape, lo, hi, np.int64))
    oshape = tuple(s + b + a for s, (b, a) in zip(shape, pads))
    oi = TensorInfo(oshape, dtype, (outq[0],), lo + 20 + outq[1]) if outq else TensorInfo(oshape, dtype, (0.05,), lo + 20)
    before = [b for b, _ in pads]
    p = port.pad(x, oi, before, value).data
    np.testing.assert_array_equal(p, reference.pad(x, oi, before, value).data)
    if outq is None:
        # closed form: numpy's constant padding with the saturated, rounded code
        code = int(np.clip(np.sign(value) * np.floor(abs(value) + 0.5), lo, hi))
        np.testing.assert_array_equal(p, np.pad(x.data, pads, constant_values=code))


@pytest.mark.parametrize("dtype", [DataType.QAsymmS8, DataType.QAsymmU8])
@pytest.mark.parametrize("shape", [(2, 7, 7, 64), (3, 14, 14, 37), (1, 5, 3, 8), (2, 1, 1, 16), (1, 9, 9, 1024)])
def test_mean_over_height_and_width_equals_global_average_pooling(port, reference, dtype, shape):
    """What lets the device run the Mean layer on its pooling kernel: the reference's Reduce (Reduce.cpp:69-173) and an
    average Pooling2d over the whole feature map give the same bytes, for any output quantization."""
    lo = 0 if dtype == DataType.QAsymmU8 else -128
    n, h, w, c = shape
    x = QTensor(TensorInfo(shape, dtype, (0.05,), lo + 20), synth.uniform_int(100, shape, lo, lo + 255, np.int64))
    for so, zo in ((0.05, lo + 3), (0.031, lo + 77), (0.2, lo + 250)):
        oi = TensorInfo((n, 1, 1, c), dtype, (so,), zo)
        pooled = port.pooling2d(x, oi, pool_type=cpuref.POOL_AVERAGE, pool_w=w, pool_h=h, stride_x=1, stride_y=1, padding_method=cpuref.PAD_EXCLUDE)
        np.testing.assert_array_equal(pooled.data, reference.mean(x, oi, [1, 2]).data)
