"""Pooling2d, Add, Activation and Softmax on the device against the oracle (<= 1 LSB; pooling, add and activation are
expected exact: the device follows the reference's float operations element for element)."""
import numpy as np
import pytest

from armnn_amd import shim, synth
from armnn_amd.tensor import DataType, QTensor, TensorInfo
from oracle import cpuref
from tests.helpers import lsb_diff

pytestmark = pytest.mark.gpu

S8, U8 = DataType.QAsymmS8, DataType.QAsymmU8


def _rand(seed, shape, dtype, scale, offset):
    lo, hi = (0, 255) if dtype == U8 else (-128, 127)
    return QTensor(TensorInfo(shape, dtype, (scale,), offset), synth.uniform_int(seed, shape, lo, hi, np.int64))


POOLS = [
    # (name, shape, pool_type, pw, ph, sx, sy, pads l r t b)  -- channel counts hit the 4-channel and the scalar kernel
    ("max3x3s2_c64", (2, 23, 21, 64), cpuref.POOL_MAX, 3, 3, 2, 2, (1, 1, 1, 1)),
    ("max3x3s2_c5", (1, 11, 13, 5), cpuref.POOL_MAX, 3, 3, 2, 2, (1, 1, 1, 1)),
    ("avg7x7_global_c1024", (3, 7, 7, 1024), cpuref.POOL_AVERAGE, 7, 7, 1, 1, (0, 0, 0, 0)),
    ("max14x14_global_c300", (2, 14, 14, 300), cpuref.POOL_MAX, 14, 14, 1, 1, (0, 0, 0, 0)),
    ("avg3x5_global_c8", (5, 5, 3, 8), cpuref.POOL_AVERAGE, 3, 5, 2, 2, (0, 0, 0, 0)),
    ("avg3x2_pad_c12", (1, 9, 10, 12), cpuref.POOL_AVERAGE, 3, 2, 2, 1, (1, 1, 1, 0)),
    ("avg2x2_c8", (2, 8, 8, 8), cpuref.POOL_AVERAGE, 2, 2, 2, 2, (0, 0, 0, 0)),
    ("max9x9_big_window_c8", (1, 12, 12, 8), cpuref.POOL_MAX, 9, 9, 3, 3, (4, 4, 4, 4)),
    ("avg5x5_pad2_c16", (1, 10, 10, 16), cpuref.POOL_AVERAGE, 5, 5, 1, 1, (2, 2, 2, 2)),
]


@pytest.mark.parametrize("cfg", POOLS, ids=[c[0] for c in POOLS])
@pytest.mark.parametrize("method", [cpuref.PAD_EXCLUDE, cpuref.PAD_IGNORE_VALUE])
@pytest.mark.parametrize("dtype", [S8, U8])
def test_pooling(port, cfg, method, dtype):
    name, shape, ptype, pw, ph, sx, sy, (pl, pr, pt, pb) = cfg
    print("pool", name, method, dtype, flush=True)
    n, h, w, c = shape
    lo = 0 if dtype == U8 else -128
    x = _rand(31, shape, dtype, 0.05, lo + 20)
    ho = (h + pt + pb - ph) // sy + 1
    wo = (w + pl + pr - pw) // sx + 1
    oi = TensorInfo((n, ho, wo, c), dtype, (0.07,), lo + 9)
    kw = dict(pool_type=ptype, pool_w=pw, pool_h=ph, stride_x=sx, stride_y=sy, pad_left=pl, pad_right=pr, pad_top=pt,
              pad_bottom=pb, padding_method=method)
    want = port.pooling2d(x, oi, **kw)
    got = shim.pooling2d(x, oi, **kw)
    np.testing.assert_array_equal(got.data, want.data)


@pytest.mark.parametrize("dtype", [S8, U8])
@pytest.mark.parametrize("shape", [(2, 14, 14, 256), (1, 5, 5, 3), (3, 7, 9, 20)])
@pytest.mark.parametrize("act", [(0, 0.0, 0.0), (1, 0.0, 0.0), (2, 6.0, 0.0)])
def test_add(port, dtype, shape, act):
    print("add", dtype, shape, act, flush=True)
    lo = 0 if dtype == U8 else -128
    a = _rand(41, shape, dtype, 0.03, lo + 10)
    b = _rand(42, shape, dtype, 0.05, lo + 90)
    oi = TensorInfo(shape, dtype, (0.06,), lo + 50)
    want = port.add(a, b, oi)
    if act[0]:
        want = port.activation(want, oi, *act)
    got = shim.add(a, b, oi, activation=act[0], act_a=act[1], act_b=act[2])
    np.testing.assert_array_equal(got.data, want.data)


@pytest.mark.parametrize("dtype", [S8, U8])
@pytest.mark.parametrize("cols", [10, 1001, 1500, 3000])
def test_softmax(port, dtype, cols):
    print("softmax", dtype, cols, flush=True)
    lo = 0 if dtype == U8 else -128
    x = _rand(51, (5, cols), dtype, 0.1, lo + 60)
    oi = TensorInfo((5, cols), dtype, (1.0 / 256,), lo)
    want = port.softmax(x, oi)
    got = shim.softmax(x, oi)
    mx, exact = lsb_diff(got.data, want.data)
    print(f"  max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99


@pytest.mark.parametrize("dtype", [S8, U8])
@pytest.mark.parametrize("act", [(1, 0.0, 0.0), (2, 6.0, 0.0), (2, 1.0, -1.0)])
def test_activation_requantizing(port, dtype, act):
    lo = 0 if dtype == U8 else -128
    x = _rand(61, (2, 9, 9, 24), dtype, 0.04, lo + 100)
    oi = TensorInfo((2, 9, 9, 24), dtype, (0.03,), lo + 7)
    want = port.activation(x, oi, *act)
    got = shim.activation(x, oi, *act)
    np.testing.assert_array_equal(got.data, want.data)
