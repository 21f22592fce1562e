"""Depthwise 3x3 + pointwise 1x1 as one kernel, and pointwise 1x1 + the depthwise 3x3 after it as one kernel: bytes must
equal the two layers run one after the other, and the pair must stay within 1 LSB of the oracle per layer (the second
layer judged on the first layer's actual output)."""
import ctypes as C

import numpy as np
import pytest

from armnn_amd import shim
from armnn_amd.tensor import DataType, QTensor, TensorInfo, numpy_dtype
from tests import cases
from tests.helpers import lsb_diff

pytestmark = pytest.mark.gpu

S8, U8 = DataType.QAsymmS8, DataType.QAsymmU8

# (name, n, h, w, c, co, stride, dtype, act after dw, act after pw)
PAIRS = [
    ("s1_c32_co64_u8", 2, 37, 45, 32, 64, 1, U8, cases.RELU6, cases.RELU6),
    ("s2_c64_co128_s8", 3, 41, 30, 64, 128, 2, S8, cases.RELU6, cases.RELU6),
    ("s1_c128_co128_s8", 1, 19, 23, 128, 128, 1, S8, cases.RELU6, (0, 0.0, 0.0)),
    ("s2_c128_co256_u8", 2, 28, 28, 128, 256, 2, U8, cases.RELU, cases.RELU6),
    ("s1_c256_co256_s8", 2, 14, 14, 256, 256, 1, S8, (0, 0.0, 0.0), cases.RELU6),
    ("s1_c512_co512_s8", 2, 14, 14, 512, 512, 1, S8, cases.RELU6, cases.RELU6),
    ("s1_c96_co192_s8_tiny", 1, 5, 3, 96, 192, 1, S8, cases.RELU6, cases.RELU6),
]


# pairs the one-block-per-tile-over-all-channels kernel takes: 256 or 512 channels in between, 256 or 512 out, stride 1 (or
# stride 2 from 256 to 512 channels)
PANEL_PAIRS = [
    ("panel_c512_co512_u8_14", 5, 14, 14, 512, 512, 1, U8, cases.RELU6, cases.RELU6),      # the MobileNetV1 pairs dw7+pw7 ... dw11+pw11
    ("panel_c256_co256_u8_28", 3, 28, 28, 256, 256, 1, U8, cases.RELU6, cases.RELU6),      # dw5+pw5
    ("panel_c256_co512_s8_ragged", 2, 13, 9, 256, 512, 1, S8, cases.RELU, (0, 0.0, 0.0)),
    ("panel_c512_co256_s8_tiny", 1, 3, 5, 512, 256, 1, S8, (0, 0.0, 0.0), cases.RELU6),
    ("panel_c512_co512_s8_17x23", 2, 17, 23, 512, 512, 1, S8, cases.RELU6, cases.RELU),
    ("panel_c256_co512_u8_28_s2", 5, 28, 28, 256, 512, 2, U8, cases.RELU6, cases.RELU6),   # dw6+pw6
    ("panel_c256_co512_s8_ragged_s2", 3, 19, 25, 256, 512, 2, S8, cases.RELU, cases.RELU6),
]


# pairs the persistent kernel with resident pointwise weights takes (32 -> 64, 64 -> 128 at stride 2, 128 -> 128, 128 -> 256
# at stride 2): enough
# images that a block walks several items, ragged maps, both activation types
STREAM_PAIRS = [
    ("stream_c32_co64_u8_112", 12, 112, 112, 32, 64, 1, U8, cases.RELU6, cases.RELU6),      # MobileNetV1 dw1+pw1
    ("stream_c64_co128_u8_112_s2", 12, 112, 112, 64, 128, 2, U8, cases.RELU6, cases.RELU6),  # dw2+pw2
    ("stream_c128_co128_u8_56", 12, 56, 56, 128, 128, 1, U8, cases.RELU6, cases.RELU6),      # dw3+pw3
    ("stream_c128_co256_u8_56_s2", 20, 56, 56, 128, 256, 2, U8, cases.RELU6, cases.RELU6),   # dw4+pw4
    ("stream_c128_co256_s8_ragged_s2", 30, 23, 31, 128, 256, 2, S8, cases.RELU, cases.RELU6),
    ("stream_c32_co64_s8_ragged", 30, 50, 35, 32, 64, 1, S8, cases.RELU, (0, 0.0, 0.0)),
    ("stream_c64_co128_s8_ragged_s2", 25, 45, 51, 64, 128, 2, S8, (0, 0.0, 0.0), cases.RELU6),
    ("stream_c128_co128_s8_ragged", 40, 13, 29, 128, 128, 1, S8, cases.RELU6, cases.RELU),
    ("stream_c32_co64_s8_tiny", 1, 3, 5, 32, 64, 1, S8, cases.RELU6, cases.RELU6),
]


@pytest.mark.parametrize("pair", STREAM_PAIRS + PAIRS[:4], ids=[p[0] for p in STREAM_PAIRS + PAIRS[:4]])
def test_stream_kernel_is_taken_and_equals_the_older_fused_kernel(pair):
    shim.Device()
    dw, pw = _make(*pair)
    pdw, ppw = _plan(dw), _plan(pw)
    n = dw.x.info.shape[0]
    xd = shim.DeviceBuffer(dw.x.data.nbytes).upload(dw.x.data)
    ya, yb = shim.DeviceBuffer(pw.out_info.num_elements), shim.DeviceBuffer(pw.out_info.num_elements)
    pdw.run_fused(ppw, n, xd.ptr, ya.ptr)
    assert shim.last_kernel().startswith("DwPwStreamKernel<"), shim.last_kernel()
    shim.set_option("dwpw_stream", 0)
    try:
        pdw.run_fused(ppw, n, xd.ptr, yb.ptr)
        assert shim.last_kernel().startswith("DwPwKernel<"), shim.last_kernel()
    finally:
        shim.set_option("dwpw_stream", 1)
    a = ya.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    b = yb.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    assert len(np.unique(a)) > 8
    np.testing.assert_array_equal(a, b)


def _make(name, n, h, w, c, co, stride, dt, act_dw, act_pw):
    zp_in = 120 if dt == U8 else -8
    zp_mid = 0 if dt == U8 else -128
    dw = cases.make_conv_case(name + "_dw", 900 + c, n=n, h=h, w=w, ci=c, depthwise=True, stride=(stride, stride), in_dtype=dt,
                              in_scale=0.0235, in_offset=zp_in, out_scale=0.0235, out_offset=zp_mid, act=act_dw,
                              w_scale_range=(0.01, 0.05))
    ho, wo = dw.out_info.shape[1], dw.out_info.shape[2]
    pw = cases.make_conv_case(name + "_pw", 901 + co, n=n, h=ho, w=wo, ci=c, co=co, kh=1, kw=1, in_dtype=dt, in_scale=0.0235,
                              in_offset=zp_mid, out_scale=0.03, out_offset=zp_mid + 5, act=act_pw)
    return dw, pw


def _plan(c):
    fn, a, b = c.act
    return shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, activation=fn, act_a=a, act_b=b, **c.params)


@pytest.mark.parametrize("pair", PANEL_PAIRS, ids=[p[0] for p in PANEL_PAIRS])
def test_panel_kernel_is_taken_and_equals_the_older_fused_kernel(pair):
    shim.Device()
    dw, pw = _make(*pair)
    pdw, ppw = _plan(dw), _plan(pw)
    n = dw.x.info.shape[0]
    xd = shim.DeviceBuffer(dw.x.data.nbytes).upload(dw.x.data)
    ya, yb = shim.DeviceBuffer(pw.out_info.num_elements), shim.DeviceBuffer(pw.out_info.num_elements)
    pdw.run_fused(ppw, n, xd.ptr, ya.ptr)
    assert shim.last_kernel().startswith("DwPwPanelKernel<"), shim.last_kernel()
    shim.set_option("dwpw_panel", 0)
    try:
        pdw.run_fused(ppw, n, xd.ptr, yb.ptr)
        assert shim.last_kernel().startswith("DwPwKernel<"), shim.last_kernel()
    finally:
        shim.set_option("dwpw_panel", 1)
    a = ya.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    b = yb.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    np.testing.assert_array_equal(a, b)


@pytest.mark.parametrize("pair", PAIRS + PANEL_PAIRS + STREAM_PAIRS[4:], ids=[p[0] for p in PAIRS + PANEL_PAIRS + STREAM_PAIRS[4:]])
def test_fused_equals_two_layers(port, pair):
    print("pair", pair, flush=True)
    shim.Device()
    dw, pw = _make(*pair)
    pdw, ppw = _plan(dw), _plan(pw)
    assert pdw.fusable_with(ppw), shim.load_library().mi355x_last_error().decode()
    n = dw.x.info.shape[0]
    xd = shim.DeviceBuffer(dw.x.data.nbytes).upload(dw.x.data)
    mid = shim.DeviceBuffer(dw.out_info.num_elements)
    y2 = shim.DeviceBuffer(pw.out_info.num_elements)
    yf = shim.DeviceBuffer(pw.out_info.num_elements)
    pdw.run(n, xd.ptr, mid.ptr)
    ppw.run(n, mid.ptr, y2.ptr)
    pdw.run_fused(ppw, n, xd.ptr, yf.ptr)
    mid_h = mid.download(dw.out_info.shape, numpy_dtype(dw.out_info.dtype))
    two = y2.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    fused = yf.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    np.testing.assert_array_equal(fused, two)
    assert len(np.unique(fused)) > 8
    # and the two layers themselves against the oracle
    fn, a, b = dw.act
    want_mid = port.activation(port.conv2d(dw.x, dw.w, dw.b, dw.out_info, **dw.params), dw.out_info, fn, a, b) if fn else \
        port.conv2d(dw.x, dw.w, dw.b, dw.out_info, **dw.params)
    mx, exact = lsb_diff(mid_h, want_mid.data)
    assert mx <= 1 and exact >= 0.99
    pw.x = QTensor(pw.x.info, mid_h)
    fn, a, b = pw.act
    want = port.conv2d(pw.x, pw.w, pw.b, pw.out_info, **pw.params)
    if fn:
        want = port.activation(want, pw.out_info, fn, a, b)
    mx, exact = lsb_diff(fused, want.data)
    print(f"  fused vs oracle on the device's intermediate: max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99


def test_unfusable_pairs_are_refused():
    shim.Device()
    dw, pw = _make("x", 1, 9, 9, 32, 64, 1, S8, cases.RELU6, cases.RELU6)
    pdw, ppw = _plan(dw), _plan(pw)
    assert pdw.fusable_with(ppw)
    assert not ppw.fusable_with(pdw)                      # wrong order
    # the shared tensor's quantization differs
    pw2 = cases.make_conv_case("x_pw2", 5, n=1, h=9, w=9, ci=32, co=64, kh=1, kw=1, in_scale=0.05, in_offset=-128)
    assert not pdw.fusable_with(_plan(pw2))
    # channel counts do not chain
    pw3 = cases.make_conv_case("x_pw3", 6, n=1, h=9, w=9, ci=64, co=64, kh=1, kw=1, in_scale=0.0235, in_offset=-128)
    assert not pdw.fusable_with(_plan(pw3))
    # 3x3 consumer is not pointwise
    c3 = cases.make_conv_case("x_c3", 7, n=1, h=9, w=9, ci=32, co=64, in_scale=0.0235, in_offset=-128)
    assert not pdw.fusable_with(_plan(c3))
    with pytest.raises(shim.ShimError):
        xd = shim.DeviceBuffer(dw.x.data.nbytes).upload(dw.x.data)
        yd = shim.DeviceBuffer(c3.out_info.num_elements)
        pdw.run_fused(_plan(c3), 1, xd.ptr, yd.ptr)


# ---- the other order: 1x1 convolution, then the 3x3 depthwise that consumes it, whole images per block ------------------
# (name, n, h, w, ci, c, depthwise stride, dtype, act after pw, act after dw)
PW_DW = [
    ("14x14_k512_c512_s1_s8", 3, 14, 14, 512, 512, 1, S8, cases.RELU6, cases.RELU6),
    ("14x14_k256_c128_s2_u8", 2, 14, 14, 256, 128, 2, U8, cases.RELU6, cases.RELU),
    ("7x7_k512_c128_s1_s8_last_block_has_one_image", 5, 7, 7, 512, 128, 1, S8, cases.RELU6, cases.RELU6),
    ("7x7_k128_c64_s1_u8_four_images_one_block", 4, 7, 7, 128, 64, 1, U8, (0, 0.0, 0.0), cases.RELU6),
    ("9x11_k128_c64_s2_s8_odd_sizes", 2, 9, 11, 128, 64, 2, S8, cases.RELU, (0, 0.0, 0.0)),
    ("6x5_k384_c192_s1_u8", 7, 6, 5, 384, 192, 1, U8, cases.RELU6, cases.RELU6),
    ("1x1_k128_c64_s1_s8", 9, 1, 1, 128, 64, 1, S8, cases.RELU6, cases.RELU6),
    ("14x16_k128_c64_s1_s8_exactly_224_rows", 2, 14, 16, 128, 64, 1, S8, cases.RELU6, cases.RELU6),
]


def _make_pw_dw(name, n, h, w, ci, c, stride, dt, act_pw, act_dw):
    zp_in = 3 if dt == U8 else -128
    zp_mid = 7 if dt == U8 else -121
    pw = cases.make_conv_case(name + "_pw", 700 + ci, n=n, h=h, w=w, ci=ci, co=c, kh=1, kw=1, in_dtype=dt, in_scale=0.0235,
                              in_offset=zp_in, out_scale=0.04, out_offset=zp_mid, act=act_pw)
    dw = cases.make_conv_case(name + "_dw", 701 + c, n=n, h=h, w=w, ci=c, depthwise=True, stride=(stride, stride), in_dtype=dt,
                              in_scale=0.04, in_offset=zp_mid, out_scale=0.0235, out_offset=zp_in, act=act_dw,
                              w_scale_range=(0.01, 0.05))
    return pw, dw


@pytest.mark.parametrize("pair", PW_DW, ids=[p[0] for p in PW_DW])
def test_pointwise_then_depthwise_fused_equals_two_layers(port, pair):
    print("pair", pair, flush=True)
    shim.Device()
    pw, dw = _make_pw_dw(*pair)
    ppw, pdw = _plan(pw), _plan(dw)
    assert ppw.fusable_with(pdw), shim.load_library().mi355x_last_error().decode()
    n = pw.x.info.shape[0]
    xd = shim.DeviceBuffer(pw.x.data.nbytes).upload(pw.x.data)
    mid = shim.DeviceBuffer(pw.out_info.num_elements)
    y2 = shim.DeviceBuffer(dw.out_info.num_elements)
    yf = shim.DeviceBuffer(dw.out_info.num_elements)
    ppw.run(n, xd.ptr, mid.ptr)
    pdw.run(n, mid.ptr, y2.ptr)
    ppw.run_fused(pdw, n, xd.ptr, yf.ptr)
    assert shim.last_kernel().startswith("PwDwKernel")
    first = yf.download(dw.out_info.shape, numpy_dtype(dw.out_info.dtype))
    _, h, w, _ = pw.x.info.shape
    for mf in (2, 4):                                        # smaller blocks, where an image fits them, give the same bytes
        shim.set_option("pwdw_mf", mf)
        try:
            ppw.run_fused(pdw, n, xd.ptr, yf.ptr)
            kernel = shim.last_kernel()
        finally:
            shim.set_option("pwdw_mf", 0)
        assert kernel.startswith(f"PwDwKernel<{mf}," if h * w <= mf * 32 else "PwDwKernel<7,"), kernel
        np.testing.assert_array_equal(yf.download(dw.out_info.shape, numpy_dtype(dw.out_info.dtype)), first, err_msg=f"{mf} fragments per block")
    mid_h = mid.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    two = y2.download(dw.out_info.shape, numpy_dtype(dw.out_info.dtype))
    fused = yf.download(dw.out_info.shape, numpy_dtype(dw.out_info.dtype))
    np.testing.assert_array_equal(fused, two)
    assert len(np.unique(fused)) > 8
    # the padding the depthwise layer sees is its input zero point: border outputs against the oracle on the device's own
    # intermediate tensor, like every other output
    dw.x = QTensor(dw.x.info, mid_h)
    fn, a, b = dw.act
    want = port.conv2d(dw.x, dw.w, dw.b, dw.out_info, **dw.params)
    if fn:
        want = port.activation(want, dw.out_info, fn, a, b)
    mx, exact = lsb_diff(fused, want.data)
    print(f"  fused vs oracle on the device's intermediate: max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    fn, a, b = pw.act
    want_mid = port.conv2d(pw.x, pw.w, pw.b, pw.out_info, **pw.params)
    if fn:
        want_mid = port.activation(want_mid, pw.out_info, fn, a, b)
    mx, exact = lsb_diff(mid_h, want_mid.data)
    assert mx <= 1 and exact >= 0.99


def test_pointwise_then_depthwise_pairs_outside_the_kernels_shape_are_refused():
    shim.Device()
    lib = shim.load_library()
    # 15 x 15 = 225 pixels: one image no longer fits the block's 224 rows
    pw, dw = _make_pw_dw("big", 1, 15, 15, 128, 64, 1, S8, cases.RELU6, cases.RELU6)
    assert not _plan(pw).fusable_with(_plan(dw))
    assert "whole images" in lib.mi355x_last_error().decode()
    # 96 channels are not whole 64-channel blocks
    pw, dw = _make_pw_dw("c96", 1, 7, 7, 128, 96, 1, S8, cases.RELU6, cases.RELU6)
    assert not _plan(pw).fusable_with(_plan(dw))
    # 64 input channels: no whole 128-byte k-tile
    pw, dw = _make_pw_dw("k64", 1, 7, 7, 64, 64, 1, S8, cases.RELU6, cases.RELU6)
    assert not _plan(pw).fusable_with(_plan(dw))
    # the shared tensor's quantization differs
    pw, dw = _make_pw_dw("q", 1, 7, 7, 128, 64, 1, S8, cases.RELU6, cases.RELU6)
    other = cases.make_conv_case("q_dw2", 3, n=1, h=7, w=7, ci=64, depthwise=True, in_scale=0.05, in_offset=-121)
    assert not _plan(pw).fusable_with(_plan(other))
    with pytest.raises(shim.ShimError):
        xd = shim.DeviceBuffer(pw.x.data.nbytes).upload(pw.x.data)
        yd = shim.DeviceBuffer(other.out_info.num_elements)
        _plan(pw).run_fused(_plan(other), 1, xd.ptr, yd.ptr)


# ---- a 1x1 convolution and the pooling over its whole output image as one launch ----------------------------------------
# (name, n, h, w, ci, c, dtype, act after the convolution, pool type (0 max, 1 average), pooled scale, pooled offset)
PW_POOL = [
    ("7x7_k1024_c1024_s8_avg_as_mobilenet_ends", 6, 7, 7, 1024, 1024, S8, cases.RELU6, 1, 0.0235, -128),
    ("7x7_k512_c128_u8_avg_last_block_has_one_image", 5, 7, 7, 512, 128, U8, cases.RELU6, 1, 0.03, 2),
    ("7x7_k128_c64_s8_max", 4, 7, 7, 128, 64, S8, (0, 0.0, 0.0), 0, 0.04, -121),
    ("14x14_k256_c128_u8_avg_one_image_per_block", 3, 14, 14, 256, 128, U8, cases.RELU, 1, 0.02, 0),
    ("4x5_k128_c192_s8_avg_eleven_images_per_block", 13, 4, 5, 128, 192, S8, cases.RELU6, 1, 0.05, -100),
    ("1x1_k128_c64_u8_max", 9, 1, 1, 128, 64, U8, cases.RELU6, 0, 0.04, 7),
    ("10x10_k384_c64_s8_avg_wider_output_scale", 3, 10, 10, 384, 64, S8, (0, 0.0, 0.0), 1, 0.01, 5),
]


def _make_pw_pool(name, n, h, w, ci, c, dt, act_pw, pool_type, pooled_scale, pooled_offset):
    zp_in = 3 if dt == U8 else -128
    zp_mid = 7 if dt == U8 else -121
    pw = cases.make_conv_case(name + "_pw", 900 + ci, n=n, h=h, w=w, ci=ci, co=c, kh=1, kw=1, in_dtype=dt, in_scale=0.0235,
                              in_offset=zp_in, out_scale=0.04, out_offset=zp_mid, act=act_pw)
    pooled = TensorInfo((n, 1, 1, c), dt, pooled_scale, pooled_offset)
    d = shim.Pool2dDesc(h, w, c, 1, 1, w, h, 1, 1, 0, 0, 0, 0, pool_type, 1, shim._quant(pw.out_info), shim._quant(pooled))
    return pw, pooled, d


@pytest.mark.parametrize("cfg", PW_POOL, ids=[c[0] for c in PW_POOL])
def test_pointwise_then_global_pooling_fused_equals_two_layers(port, cfg):
    print("pair", cfg, flush=True)
    shim.Device()
    lib = shim.load_library()
    pw, pooled, d = _make_pw_pool(*cfg)
    ppw = _plan(pw)
    assert ppw.pool_fusable(d), lib.mi355x_last_error().decode()
    n, h, w, _ = pw.x.info.shape
    xd = shim.DeviceBuffer(pw.x.data.nbytes).upload(pw.x.data)
    mid = shim.DeviceBuffer(pw.out_info.num_elements)
    y2 = shim.DeviceBuffer(pooled.num_elements)
    yf = shim.DeviceBuffer(pooled.num_elements + 64)
    shim._chk(lib.mi355x_fill_u8(yf.ptr, 0x5A, pooled.num_elements + 64, None))
    ppw.run(n, xd.ptr, mid.ptr)
    shim._chk(lib.mi355x_pool2d_run(C.byref(d), n, mid.ptr, y2.ptr, None))
    ppw.run_pooled(d, n, xd.ptr, yf.ptr)
    assert shim.last_kernel().startswith("PwDwKernel") and shim.last_kernel().endswith("true>")
    first = yf.download((pooled.num_elements + 64,), np.uint8)
    for mf in (2, 4, 7):                                     # every block size the kernel comes in gives the same bytes
        shim.set_option("pwdw_mf", mf)
        try:
            shim._chk(lib.mi355x_fill_u8(yf.ptr, 0x5A, pooled.num_elements + 64, None))
            ppw.run_pooled(d, n, xd.ptr, yf.ptr)
            kernel = shim.last_kernel()
        finally:
            shim.set_option("pwdw_mf", 0)
        if h * w <= mf * 32:
            assert kernel.startswith(f"PwDwKernel<{mf},"), kernel
        np.testing.assert_array_equal(yf.download((pooled.num_elements + 64,), np.uint8), first, err_msg=f"{mf} fragments per block")
    two = y2.download(pooled.shape, numpy_dtype(pooled.dtype))
    got = yf.download((pooled.num_elements + 64,), np.uint8)
    fused = got[:pooled.num_elements].view(numpy_dtype(pooled.dtype)).reshape(pooled.shape)
    np.testing.assert_array_equal(fused, two)
    assert (got[pooled.num_elements:] == 0x5A).all()         # nothing written behind the pooled tensor
    assert len(np.unique(fused)) > 4
    # against the oracle's pooling of the device's own intermediate tensor
    mid_h = mid.download(pw.out_info.shape, numpy_dtype(pw.out_info.dtype))
    want = port.pooling2d(QTensor(pw.out_info, mid_h), pooled, pool_type=d.pool_type, pool_w=w, pool_h=h, stride_x=1, stride_y=1)
    mx, exact = lsb_diff(fused, want.data)
    print(f"  fused vs oracle on the device's intermediate: max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99


def test_pointwise_then_pooling_pairs_outside_the_kernels_shape_are_refused():
    shim.Device()
    lib = shim.load_library()
    pw, pooled, d = _make_pw_pool("ok", 2, 7, 7, 128, 64, S8, cases.RELU6, 1, 0.04, -121)
    plan = _plan(pw)
    assert plan.pool_fusable(d)
    assert not plan.pool_fusion_pays(d, 2)                   # one block: two launches are no slower
    xd = shim.DeviceBuffer(pw.x.data.nbytes).upload(pw.x.data)
    yd = shim.DeviceBuffer(pooled.num_elements)

    def changed(**kw):
        e = shim.Pool2dDesc.from_buffer_copy(d)
        for k, v in kw.items():
            setattr(e, k, v)
        return e
    for e, why in ((changed(pool_w=3, pool_h=3, out_h=5, out_w=5), "whole"),        # a window smaller than the image
                   (changed(pad_left=1), "whole"),
                   (changed(channels=128), "chain"),
                   (changed(pool_type=2), "pooling algorithm"),
                   (changed(input=shim.Quant(int(S8), 0.05, -121)), "quantization")):
        assert not plan.pool_fusable(e)
        assert why in lib.mi355x_last_error().decode(), lib.mi355x_last_error().decode()
        with pytest.raises(shim.ShimError):
            plan.run_pooled(e, 2, xd.ptr, yd.ptr)
    # 15 x 15 = 225 pixels exceed what a block holds; 96 channels are not whole 64-channel blocks; 64 input channels are no
    # whole k-tile; a 3x3 convolution is not pointwise
    for args in (("big", 1, 15, 15, 128, 64), ("c96", 1, 7, 7, 128, 96), ("k64", 1, 7, 7, 64, 64)):
        pw2, _, d2 = _make_pw_pool(*args, S8, cases.RELU6, 1, 0.04, -121)
        assert not _plan(pw2).pool_fusable(d2), args
    c3 = cases.make_conv_case("c3", 7, n=1, h=7, w=7, ci=128, co=64, in_scale=0.0235, in_offset=-128, out_scale=0.04, out_offset=-121)
    assert not _plan(c3).pool_fusable(d)
    # a misaligned input pointer
    with pytest.raises(shim.ShimError):
        plan.run_pooled(d, 1, xd.ptr + 4, yd.ptr)
    # the pooled tensor inside the input's range: one launch would read what it writes
    with pytest.raises(shim.ShimError):
        plan.run_pooled(d, 2, xd.ptr, xd.ptr + 2 * 7 * 7 * 128 - 64)
    assert "overlap" in lib.mi355x_last_error().decode()
    plan.run_pooled(d, 2, xd.ptr, yd.ptr)
    # an empty batch is no work and no error
    plan.run_pooled(d, 0, xd.ptr, yd.ptr)


# ---- a convolution and the Addition that consumes it (residual connection) as one launch ------------------------------------
# (name, n, h, w, ci, co, kernel, stride, dtype, activation of the Addition, kernel the launch should resolve to or None)
CONV_ADD = [
    ("pointwise_k64_co256_s8_relu", 2, 56, 56, 64, 256, 1, 1, S8, cases.RELU, "PwGemmKernel"),
    ("pointwise_k128_co512_u8", 3, 28, 28, 128, 512, 1, 1, U8, (0, 0.0, 0.0), "PwGemmKernel"),
    ("pointwise_k256_co1024_s8_relu", 2, 14, 14, 256, 1024, 1, 1, S8, cases.RELU, "IgemmLdsKernel"),
    ("projection_k256_co512_stride2_u8_relu6", 2, 56, 56, 256, 512, 1, 2, U8, cases.RELU6, "IgemmLdsKernel"),
    ("pointwise_k512_co2048_ragged_rows_s8", 3, 7, 7, 512, 2048, 1, 1, S8, cases.RELU, "IgemmLdsKernel"),
    ("conv3x3_c64_falls_back_to_two_launches", 2, 20, 20, 64, 64, 3, 1, S8, cases.RELU, None),
    ("pointwise_co40_not_whole_chunks_falls_back", 1, 9, 9, 128, 40, 1, 1, U8, cases.RELU, None),
]


@pytest.mark.parametrize("cfg", CONV_ADD, ids=[c[0] for c in CONV_ADD])
def test_convolution_with_fused_addition_equals_two_layers(port, cfg):
    name, n, h, w, ci, co, k, stride, dt, act, kernel = cfg
    print("conv+add", cfg, flush=True)
    shim.Device()
    zp = 3 if dt == U8 else -120
    c = cases.make_conv_case(name, 1300 + co, n=n, h=h, w=w, ci=ci, co=co, kh=k, kw=k, stride=(stride, stride), in_dtype=dt, in_scale=0.0235,
                             in_offset=zp, out_scale=0.06, out_offset=zp + 90)
    plan = _plan(c)
    rng = np.random.default_rng(77)
    lo, hi = (0, 255) if dt == U8 else (-128, 127)
    other_info = TensorInfo(c.out_info.shape, dt, (0.043,), zp + 60)
    other = QTensor(other_info, rng.integers(lo, hi + 1, size=c.out_info.shape).astype(numpy_dtype(dt)))
    sum_info = TensorInfo(c.out_info.shape, dt, (0.09,), zp + 5)
    xd = shim.DeviceBuffer(c.x.data.nbytes).upload(c.x.data)
    od = shim.DeviceBuffer(other.data.nbytes).upload(other.data)
    mid = shim.DeviceBuffer(c.out_info.num_elements)
    yf = shim.DeviceBuffer(c.out_info.num_elements)
    plan.run(n, xd.ptr, mid.ptr)
    conv_out = QTensor(c.out_info, mid.download(c.out_info.shape, numpy_dtype(dt)))
    fn, a, b = act
    two = shim.add(conv_out, other, sum_info, activation=fn, act_a=a, act_b=b)
    plan.run_add(n, xd.ptr, od.ptr, other_info, sum_info, yf.ptr, activation=fn, act_a=a, act_b=b)
    last = shim.last_kernel()
    fused = yf.download(c.out_info.shape, numpy_dtype(dt))
    print(f"  {last}; distinct codes {len(np.unique(fused))}", flush=True)
    if kernel is None:
        assert last.startswith("Add"), last               # the Addition ran as a launch of its own
    else:
        assert last.startswith(kernel), last
    np.testing.assert_array_equal(fused, two.data)
    assert len(np.unique(fused)) > 8
    # and the Addition itself against the oracle, on the device's convolution output
    want = port.add(conv_out, other, sum_info)
    if fn:
        want = port.activation(want, sum_info, fn, a, b)
    np.testing.assert_array_equal(fused, want.data)


@pytest.mark.parametrize("tile", [96, 128, 256, 512])
def test_fused_addition_in_the_large_tiles_equals_two_layers(tile):
    """The implicit-GEMM kernel forced to 128x64, 128x128, 256x128 and 256x256 tiles (a thread then writes two to sixteen
    16-byte pieces of the output; with more than four it requests the Addition's other input after the requantization
    instead of before it): same bytes as the convolution followed by the Addition, ragged last row tile included."""
    print("conv+add tile", tile, flush=True)
    shim.Device()
    c = cases.make_conv_case(f"pointwise_k256_co512_tile{tile}", 1900 + tile, n=2, h=33, w=31, ci=256, co=512, kh=1, kw=1, in_dtype=S8, in_scale=0.0235,
                             in_offset=-7, out_scale=0.06, out_offset=11)
    shim.set_option("igemm_tile", tile)
    try:
        plan = _plan(c)
    finally:
        shim.set_option("igemm_tile", 0)
    n = c.x.info.shape[0]
    rng = np.random.default_rng(78)
    other_info = TensorInfo(c.out_info.shape, S8, (0.043,), -20)
    other = QTensor(other_info, rng.integers(-128, 128, size=c.out_info.shape).astype(np.int8))
    sum_info = TensorInfo(c.out_info.shape, S8, (0.09,), -128)
    xd = shim.DeviceBuffer(c.x.data.nbytes).upload(c.x.data)
    od = shim.DeviceBuffer(other.data.nbytes).upload(other.data)
    mid = shim.DeviceBuffer(c.out_info.num_elements)
    yf = shim.DeviceBuffer(c.out_info.num_elements)
    plan.run(n, xd.ptr, mid.ptr)
    conv_out = QTensor(c.out_info, mid.download(c.out_info.shape, np.int8))
    fn, a, b = cases.RELU
    two = shim.add(conv_out, other, sum_info, activation=fn, act_a=a, act_b=b)
    plan.run_add(n, xd.ptr, od.ptr, other_info, sum_info, yf.ptr, activation=fn, act_a=a, act_b=b)
    last = shim.last_kernel()
    print(f"  {last}", flush=True)
    assert last.startswith("IgemmLdsKernel<"), last
    np.testing.assert_array_equal(yf.download(c.out_info.shape, np.int8), two.data)
