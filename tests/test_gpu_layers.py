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
    # (name, shape, pool_type, pw, ph, sx, sy, pads l r t b)  -- channel counts hit the 16-channel max kernel, the 4-channel and the scalar kernel
    ("max3x3s2_c64", (2, 23, 21, 64), cpuref.POOL_MAX, 3, 3, 2, 2, (1, 1, 1, 1)),
    ("max3x3s2_c5", (1, 11, 13, 5), cpuref.POOL_MAX, 3, 3, 2, 2, (1, 1, 1, 1)),
    ("max3x3s1_c16_pad", (1, 6, 7, 16), cpuref.POOL_MAX, 3, 3, 1, 1, (1, 1, 1, 1)),
    ("max2x2s2_c32", (3, 9, 8, 32), cpuref.POOL_MAX, 2, 2, 2, 2, (0, 1, 0, 1)),
    ("max3x2s3_c48_window_in_the_padding", (2, 5, 4, 48), cpuref.POOL_MAX, 3, 2, 3, 3, (3, 3, 2, 2)),
    ("avg7x7_global_c1024", (3, 7, 7, 1024), cpuref.POOL_AVERAGE, 7, 7, 1, 1, (0, 0, 0, 0)),
    ("max14x14_global_c300", (2, 14, 14, 300), cpuref.POOL_MAX, 14, 14, 1, 1, (0, 0, 0, 0)),
    ("avg3x5_global_c8", (5, 5, 3, 8), cpuref.POOL_AVERAGE, 3, 5, 2, 2, (0, 0, 0, 0)),
    ("max7x7_global_c1001_odd_channels", (4, 7, 7, 1001), cpuref.POOL_MAX, 7, 7, 1, 1, (0, 0, 0, 0)),
    ("avg8x8_global_c2048_64_taps", (16, 8, 8, 2048), cpuref.POOL_AVERAGE, 8, 8, 1, 1, (0, 0, 0, 0)),
    ("avg1x1_global_c7", (3, 1, 1, 7), cpuref.POOL_AVERAGE, 1, 1, 1, 1, (0, 0, 0, 0)),
    ("avg13x5_global_c40_65_taps", (2, 5, 13, 40), cpuref.POOL_AVERAGE, 13, 5, 1, 1, (0, 0, 0, 0)),
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
    if ph == h and pw == w and (pl, pr, pt, pb) == (0, 0, 0, 0) and h * w <= 64:
        # a whole small image: the kernel that requests a channel's taps at once ran; the LDS-staged kernel gives the same
        assert shim.last_kernel().startswith("GlobalPoolSmallKernel")
        shim.set_option("pool_small", 0)
        try:
            staged = shim.pooling2d(x, oi, **kw)
            assert not shim.last_kernel().startswith("GlobalPoolSmallKernel")
        finally:
            shim.set_option("pool_small", 1)
        np.testing.assert_array_equal(staged.data, want.data)


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


ADD_QUANTS = [
    # (name, dtype, (scale, offset) of input 0, of input 1, of the output, activation)
    ("resnet_like_relu", S8, (0.0235, -128), (0.1, -128), (0.1, -128), (1, 0.0, 0.0)),
    ("generic", S8, (0.05, 3), (0.03, -7), (0.06, 10), (0, 0.0, 0.0)),
    ("halves_all_ties", U8, (0.02, 128), (0.02, 128), (0.04, 128), (0, 0.0, 0.0)),
    ("unit_scales", S8, (1.0, 0), (1.0, 0), (1.0, 0), (0, 0.0, 0.0)),
    ("mostly_saturating", S8, (0.3, 5), (0.001, -100), (0.01, 0), (0, 0.0, 0.0)),
    ("bounded_relu_inside_the_range", U8, (0.031, 7), (0.047, 201), (0.05, 10), (2, 6.0, 0.0)),
    ("thirds", S8, (0.1, -3), (0.2, 4), (0.3, -1), (0, 0.0, 0.0)),
    ("quarters_and_eighths", U8, (0.125, 0), (0.25, 255), (0.5, 100), (1, 0.0, 0.0)),
    ("tiny_output_scale", S8, (0.004, 17), (0.006, -50), (0.0009, -128), (0, 0.0, 0.0)),
]


@pytest.mark.parametrize("cfg", ADD_QUANTS, ids=[c[0] for c in ADD_QUANTS])
def test_add_of_every_pair_of_codes(port, cfg):
    """All 256 x 256 pairs of input codes: the Addition's fast path (a two-sided bracket around the reference's fp32 value)
    and its fallback together give the reference's byte everywhere, ties included."""
    name, dtype, (sa, oa), (sb, ob), (so, oo), act = cfg
    lo = 0 if dtype == U8 else -128
    codes = np.arange(256, dtype=np.int64) + lo
    a = QTensor(TensorInfo((256, 256), dtype, (sa,), oa), np.repeat(codes, 256).reshape(256, 256))
    b = QTensor(TensorInfo((256, 256), dtype, (sb,), ob), np.tile(codes, 256).reshape(256, 256))
    oi = TensorInfo((256, 256), dtype, (so,), oo)
    want = port.add(a, b, oi)
    if act[0]:
        want = port.activation(want, oi, *act)
    got = shim.add(a, b, oi, activation=act[0], act_a=act[1], act_b=act[2])
    assert shim.last_kernel() == "AddVec16Kernel"
    np.testing.assert_array_equal(got.data, want.data)
    print(name, "distinct output codes:", len(np.unique(got.data)), flush=True)


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


PADS = [
    # (name, input shape, (before, after) per dimension, pad value, output (scale, offset shift) or None)
    ("nhwc_hw_c64_16B", (2, 14, 14, 64), ((0, 0), (1, 1), (1, 1), (0, 0)), None, None),      # 16-byte units
    ("nhwc_same_s2_c32", (3, 112, 112, 32), ((0, 0), (0, 1), (0, 1), (0, 0)), None, None),
    ("nhwc_hw_c12_4B", (2, 9, 7, 12), ((0, 0), (2, 1), (1, 3), (0, 0)), 5.0, None),          # 4-byte units
    ("nhwc_hw_c3_1B", (1, 10, 11, 3), ((0, 0), (1, 2), (3, 0), (0, 0)), -2.5, None),         # byte units; rounds to -3
    ("all_dims", (2, 4, 4, 3), ((1, 0), (1, 1), (1, 1), (2, 3)), 300.0, None),               # saturating code
    ("requantized", (2, 6, 5, 16), ((0, 0), (1, 1), (2, 2), (0, 0)), 1.0, (0.07, 5)),
    ("requantized_bytes", (3, 7), ((1, 0), (2, 3)), -300.0, (0.031, -2)),
    ("rank1", (37,), ((2, 1),), 4.0, None),
    ("rank3", (2, 3, 40), ((1, 0), (0, 1), (8, 0)), 0.0, None),
    ("no_padding", (2, 5, 5, 8), ((0, 0), (0, 0), (0, 0), (0, 0)), 0.0, None),
    ("batch_padded", (2, 3, 3, 16), ((1, 2), (0, 0), (0, 0), (0, 0)), 9.0, None),
]


@pytest.mark.parametrize("cfg", PADS, ids=[c[0] for c in PADS])
@pytest.mark.parametrize("dtype", [S8, U8])
def test_pad(port, cfg, dtype):
    """Bytes are moved or re-coded one at a time: exact against the checker, and against numpy's constant padding
    wherever input and output share one quantization."""
    name, shape, pads, value, outq = cfg
    print("pad", name, dtype, flush=True)
    lo, hi = (0, 255) if dtype == U8 else (-128, 127)
    zp = lo + 20
    x = _rand(61, shape, dtype, 0.05, zp)
    if value is None:
        value = float(zp)                                   # the neutral element a folded convolution would use
    oshape = tuple(s + b + a for s, (b, a) in zip(shape, pads))
    oi = TensorInfo(oshape, dtype, (outq[0],), zp + outq[1]) if outq else TensorInfo(oshape, dtype, (0.05,), zp)
    want = port.pad(x, oi, [b for b, _ in pads], value)
    got = shim.pad(x, oi, pads, value)
    np.testing.assert_array_equal(got.data, want.data)
    if outq is None:
        code = int(np.clip(np.sign(value) * np.floor(abs(value) + 0.5), lo, hi))
        np.testing.assert_array_equal(got.data, np.pad(x.data, pads, constant_values=code))


def test_pad_rejects_what_it_cannot_run():
    with pytest.raises(shim.ShimError):
        d = shim.PadDesc()
        d.rank = 5
        shim._chk(shim.load_library().mi355x_pad_run(shim.C.byref(d), None, None, None))
    with pytest.raises(shim.ShimError):
        shim.pad(_rand(63, (4,), S8, 0.05, 0), TensorInfo((6,), S8, (0.05,), 0), ((1, 1),), float("nan"))


FOLDS = [
    # (name, make_conv_case keywords): the layer's own padding is what a Pad layer in front of it would have added
    ("conv3x3", dict(n=2, h=13, w=15, ci=16, co=32, padding=(1, 2, 2, 1))),
    ("conv3x3_s2_u8", dict(n=1, h=14, w=14, ci=32, co=16, stride=(2, 2), padding=(0, 1, 0, 1), in_dtype=U8, in_offset=7, out_offset=0)),
    ("depthwise3x3_s2", dict(n=2, h=28, w=28, ci=64, depthwise=True, stride=(2, 2), padding=(0, 1, 0, 1))),
    ("depthwise3x3", dict(n=1, h=9, w=9, ci=24, depthwise=True, padding=(2, 2, 2, 2))),
    ("conv1x1_padded", dict(n=1, h=6, w=6, ci=64, co=64, kh=1, kw=1, padding=(1, 1, 1, 1))),
    ("stem7x7_s2", dict(n=2, h=32, w=32, ci=3, co=64, kh=7, kw=7, stride=(2, 2), padding=(3, 3, 3, 3))),
]


@pytest.mark.parametrize("cfg", FOLDS, ids=[c[0] for c in FOLDS])
def test_padding_inside_the_convolution_equals_a_pad_layer_in_front_of_it(cfg):
    """What folding a Pad layer into the convolution relies on: padding with the input's zero point and then running
    the unpadded convolution gives the bytes of the convolution with that padding as its own."""
    from tests.cases import make_conv_case
    name, kw = cfg
    print("fold", name, flush=True)
    c = make_conv_case(name, 901, **kw)
    pt, pb, pl, pr = kw["padding"]
    folded = shim.conv2d(c.x, c.w, c.b, c.out_info, activation=c.act[0], act_a=c.act[1], act_b=c.act[2], **c.params)
    n, h, w, ci = c.x.info.shape
    pinfo = TensorInfo((n, h + pt + pb, w + pl + pr, ci), c.x.info.dtype, c.x.info.scales, c.x.info.offset)
    padded = shim.pad(c.x, pinfo, ((0, 0), (pt, pb), (pl, pr), (0, 0)), float(c.x.info.offset))
    params = dict(c.params, pad_top=0, pad_left=0)
    apart = shim.conv2d(padded, c.w, c.b, c.out_info, activation=c.act[0], act_a=c.act[1], act_b=c.act[2], **params)
    np.testing.assert_array_equal(folded.data, apart.data)


def test_async_copies_need_memory_the_device_reaches_and_keep_stream_order():
    """mi355x_memcpy_h2d_async / _d2h_async: pinned memory goes up and comes back unchanged behind a kernel queued in
    between; pageable memory is refused, not copied some slower way."""
    import ctypes as C
    lib = shim.load_library()
    dev = shim.Device()
    stream = dev.stream()
    n = 1 << 20
    src, dst = C.c_void_p(), C.c_void_p()
    shim._chk(lib.mi355x_host_alloc(C.byref(src), n))
    shim._chk(lib.mi355x_host_alloc(C.byref(dst), n))
    data = np.random.default_rng(5).integers(0, 256, n, dtype=np.uint8)
    C.memmove(src.value, data.ctypes.data, n)
    a, b = shim.DeviceBuffer(n), shim.DeviceBuffer(n)
    shim._chk(lib.mi355x_memcpy_h2d_async(a.ptr, src, n, stream))
    shim._chk(lib.mi355x_memcpy_d2d(b.ptr, a.ptr, n, stream))
    shim._chk(lib.mi355x_memcpy_d2h_async(dst, b.ptr, n, stream))
    dev.stream_sync(stream)
    back = np.ctypeslib.as_array(C.cast(dst.value, C.POINTER(C.c_uint8)), shape=(n,)).copy()
    np.testing.assert_array_equal(back, data)
    pageable = np.zeros(4096, dtype=np.uint8)
    assert lib.mi355x_memcpy_h2d_async(a.ptr, pageable.ctypes.data, 4096, stream) != 0
    assert lib.mi355x_memcpy_d2h_async(pageable.ctypes.data, a.ptr, 4096, stream) != 0
    assert lib.mi355x_memcpy_h2d_async(a.ptr, src, 0, stream) == 0
    a.free(); b.free()
    shim._chk(lib.mi355x_host_free(src)); shim._chk(lib.mi355x_host_free(dst))
    dev.stream_destroy(stream)


@pytest.mark.parametrize("chunk", range(4))
def test_random_pooling_add_softmax_pad(port, chunk):
    """Seeded draws over the bandwidth-bound layers: window, stride, padding (also wider than the window), padding method,
    channel counts on and off the vector paths, quantizations, pad lists of every rank."""
    for k in range(25 * chunk, 25 * chunk + 25):
        rng = np.random.default_rng(37000 + k)
        pick = lambda xs: xs[int(rng.integers(len(xs)))]
        dtype = pick([S8, U8])
        lo = 0 if dtype == U8 else -128
        q = lambda: (float(np.exp(rng.uniform(np.log(0.01), np.log(0.2)))), lo + int(rng.integers(0, 256)))
        kind = pick(["pool", "pool", "add", "softmax", "pad"])
        print(f"layer case {k}: {kind} {dtype.name}", flush=True)
        if kind == "pool":
            n, h, w, c = int(rng.integers(1, 4)), int(rng.integers(1, 20)), int(rng.integers(1, 20)), pick([1, 3, 4, 8, 12, 16, 64, 100, 256])
            pw, ph, sx, sy = int(rng.integers(1, 6)), int(rng.integers(1, 6)), int(rng.integers(1, 4)), int(rng.integers(1, 4))
            pl, pr, pt, pb = (int(rng.integers(0, pw + 1)), int(rng.integers(0, pw + 1)), int(rng.integers(0, ph + 1)), int(rng.integers(0, ph + 1)))
            if h + pt + pb < ph or w + pl + pr < pw:
                continue
            s, z = q()
            x = _rand(38000 + k, (n, h, w, c), dtype, s, z)
            so, zo = q()
            oi = TensorInfo((n, (h + pt + pb - ph) // sy + 1, (w + pl + pr - pw) // sx + 1, c), dtype, (so,), zo)
            kw = dict(pool_type=pick([cpuref.POOL_MAX, cpuref.POOL_AVERAGE]), pool_w=pw, pool_h=ph, stride_x=sx, stride_y=sy, pad_left=pl,
                      pad_right=pr, pad_top=pt, pad_bottom=pb, padding_method=pick([cpuref.PAD_EXCLUDE, cpuref.PAD_IGNORE_VALUE]))
            np.testing.assert_array_equal(shim.pooling2d(x, oi, **kw).data, port.pooling2d(x, oi, **kw).data, err_msg=f"case {k} {kw}")
        elif kind == "add":
            shape = tuple(int(rng.integers(1, 12)) for _ in range(3)) + (pick([1, 3, 8, 16, 50, 128]),)
            (s0, z0), (s1, z1), (so, zo) = q(), q(), q()
            a, b = _rand(39000 + k, shape, dtype, s0, z0), _rand(39500 + k, shape, dtype, s1, z1)
            oi = TensorInfo(shape, dtype, (so,), zo)
            act = pick([(0, 0.0, 0.0), (1, 0.0, 0.0), (2, 6.0, 0.0)])
            want = port.add(a, b, oi)
            if act[0]:
                want = port.activation(want, oi, *act)
            np.testing.assert_array_equal(shim.add(a, b, oi, activation=act[0], act_a=act[1], act_b=act[2]).data, want.data, err_msg=f"case {k}")
        elif kind == "softmax":
            rows, cols = int(rng.integers(1, 9)), pick([1, 2, 10, 100, 1000, 1001, 1025, 2048, 3000])
            s, z = q()
            x = _rand(40000 + k, (rows, cols), dtype, s, z)
            oi = TensorInfo((rows, cols), dtype, (1.0 / 256,), lo)
            beta = float(rng.uniform(0.5, 2.0))
            mx, _ = lsb_diff(shim.softmax(x, oi, beta).data, port.softmax(x, oi, beta).data)
            assert mx <= 1, k
        else:
            rank = int(rng.integers(1, 5))
            shape = tuple(int(rng.integers(1, 10)) for _ in range(rank - 1)) + (pick([1, 4, 7, 16, 32]),)
            pads = tuple((int(rng.integers(0, 3)), int(rng.integers(0, 3))) if rng.integers(2) else (0, 0) for _ in range(rank))
            s, z = q()
            x = _rand(41000 + k, shape, dtype, s, z)
            so, zo = (s, z) if rng.integers(3) else q()
            oi = TensorInfo(tuple(d + b + a for d, (b, a) in zip(shape, pads)), dtype, (so,), zo)
            value = float(rng.integers(-300, 300)) + pick([0.0, 0.5])
            np.testing.assert_array_equal(shim.pad(x, oi, pads, value).data, port.pad(x, oi, [b for b, _ in pads], value).data, err_msg=f"case {k}")
