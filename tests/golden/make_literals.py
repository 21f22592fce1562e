"""Writes tests/golden/reference_literals.json: known-answer vectors held by the reference's own tests.

Every case below is DATA transcribed from a test in the Arm NN 35.0.0 tree (inputs, quantization
parameters and expected outputs); the `source` field cites where it lives.  Nothing is executed from
the reference to make this file.  Run: python tests/golden/make_literals.py
"""
import json
import os

import numpy as np

S8, U8, QS8, S32 = "QAsymmS8", "QAsymmU8", "QSymmS8", "Signed32"


def t(shape, dtype, data, scales=(1.0,), offset=0, quant_dim=None):
    return {"shape": list(shape), "dtype": dtype, "data": [int(v) for v in np.asarray(data).reshape(-1)],
            "scales": [float(s) for s in scales], "offset": int(offset), "quant_dim": quant_dim}


def quantize(values, scale, offset, lo, hi):
    # armnnUtils::QuantizedVector -> armnn::Quantize (src/armnn/TypesUtils.cpp:29-45); the literals used here
    # are exactly representable so float32 division needs no special care beyond half-away rounding.
    v = np.asarray(values, dtype=np.float32) / np.float32(scale)
    r = np.where(v >= 0, np.floor(v + np.float32(0.5)), np.ceil(v - np.float32(0.5)))
    return np.clip(r + offset, lo, hi).astype(np.int64)


cases = []

# ---------------------------------------------------------------------------------------------------
cases.append({
    "name": "Convolution2dPerAxisQuantTest",
    "source": "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:3562-3669",
    "op": "conv2d", "tolerance": 1, "exact_on_cpuref": True,
    "params": {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1,
               "depthwise": False, "layout": "NHWC"},
    "input": t((1, 3, 1, 2), U8, [138, 108, 138, 108, 138, 108], (0.5,), 128),
    "weights": t((3, 1, 1, 2), QS8, [1, 2, 1, 2, 1, 2], (0.5, 0.75, 1.0), 0, 0),
    "bias": t((3,), S32, [4, 4, 4], (0.25, 0.375, 0.5), 0, 0),
    "output": t((1, 3, 1, 3), U8, [121, 118, 115] * 3, (1.0,), 128),
})

cases.append({
    "name": "DepthwiseConvolution2dPerAxisQuantTest",
    "source": "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:3826-3951",
    "op": "conv2d", "tolerance": 1, "exact_on_cpuref": True,
    "params": {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1,
               "depthwise": True, "layout": "NHWC"},
    "input": t((1, 3, 3, 2), U8, [129, 130] * 9, (0.5,), 128),
    "weights": t((1, 2, 2, 4), QS8, [1] * 16, (1.0, 0.5, 1.0, 0.5), 0, 3),
    "bias": t((4,), S32, [4, 4, 4, 4], (0.5, 0.25, 0.5, 0.25), 0, 0),
    "output": t((1, 2, 2, 4), U8, [132, 130, 134, 131] * 4, (1.0,), 128),
})

# ---------------------------------------------------------------------------------------------------
# FullyConnectedTest<QAsymmU8>: asymmetric WEIGHTS (offset 93), input offset 63.
fc_in = quantize([-1.2, 6.1, -3.5, 18.8, -5.5, 2.9], 0.1, 63, 0, 255)
fc_w = quantize([-8.4, 20.0, -10.4, -8, 16.4, -11.8, 23.4, 10.4, -14.0, -3.8, -11.8, 11.4], 0.2, 93, 0, 255)
for bias_enabled in (True, False):
    out_off = -50 if bias_enabled else 10
    exp = quantize([80.0, 1460.0] if bias_enabled else [-107.04, 110.0], 5.0, out_off, 0, 255)
    cases.append({
        "name": f"FullyConnectedTest_QAsymmU8_bias{int(bias_enabled)}",
        "source": "src/backends/backendsCommon/test/layerTests/FullyConnectedTestImpl.cpp:87-163",
        "op": "fully_connected", "tolerance": 1, "exact_on_cpuref": True,
        "params": {"transpose_weights": True},
        "input": t((1, 1, 2, 3), U8, fc_in, (0.1,), 63),
        "weights": t((2, 6), U8, fc_w, (0.2,), 93),
        "bias": t((2,), S32, [9250, 67500], (np.float32(0.1) * np.float32(0.2),), 0) if bias_enabled else None,
        "output": t((1, 2), U8, exp, (5.0,), out_off),
    })

# ---------------------------------------------------------------------------------------------------
# SimpleConvolution2d3x5Uint8Test: NCHW-described data, all tensors scale 0.5 / offset 50, bias scale 0.25.
img = np.empty((3, 8, 16), dtype=np.float32)
img[0] = 0.5
img[0, 1] = 0.0
img[1] = 0.0
img[1, :, 2] = 1.0
img[2] = -1.0
ker = np.zeros((2, 3, 5, 3), dtype=np.float32)
ker[0, 0] = 1.0
ker[0, 0, 1, 1] = -1.0
ker[0, 2] = 2.0
ker[1, 1] = 1.0
exp35 = np.zeros((2, 4, 14), dtype=np.float32)
exp35[0, 0], exp35[0, 1], exp35[0, 2], exp35[0, 3] = -24.0, -25.0, -23.5, -23.5
exp35[1, :, :3] = 5.0
for bias_enabled in (False, True):
    e = exp35.copy()
    if bias_enabled:
        e[1] += 2.0       # Bias2 = {0, 2}, applied to the expected values by ApplyBias (Conv2dTestImpl.cpp)
    cases.append({
        "name": f"SimpleConvolution2d3x5Uint8Test_bias{int(bias_enabled)}",
        "source": "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:38-63,752-838,3433-3442",
        "op": "conv2d", "tolerance": 1, "exact_on_cpuref": True,
        "params": {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1,
                   "depthwise": False, "layout": "NCHW"},
        "input": t((1, 3, 8, 16), U8, quantize(img, 0.5, 50, 0, 255), (0.5,), 50),
        "weights": t((2, 3, 5, 3), U8, quantize(ker, 0.5, 50, 0, 255), (0.5,), 50),
        "bias": t((2,), S32, quantize([0.0, 2.0], 0.25, 0, -2**31, 2**31 - 1), (0.25,), 0) if bias_enabled else None,
        "output": t((1, 2, 4, 14), U8, quantize(e, 0.5, 50, 0, 255), (0.5,), 50),
    })

# ---------------------------------------------------------------------------------------------------
# The reference registers most layer tests once per data layout and permutes the NCHW-described data itself for the NHWC
# variant (armnnUtils::Permute in the test implementations); both variants are written here the same way.
def nhwc(a):
    return np.transpose(np.asarray(a), (0, 2, 3, 1))


def conv_pair(name, source, x, w, bias, e, q, params, b_scale, lo=0, hi=255, dtype=U8, exact=True):
    """x (N,C,H,W), w (O,I,H,W), e (N,O,H,W) as real numbers; q = (scale, offset) shared by all three tensors.  `params`
    names the padding before the first row and column; the padding after the last ones follows from the output's shape."""
    scale, offset = q
    qx, qw, qe = (quantize(v, scale, offset, lo, hi) for v in (x, w, e))
    qb = t((len(bias),), S32, quantize(bias, b_scale, 0, -2**31, 2**31 - 1), (b_scale,), 0) if bias is not None else None
    for layout in ("NCHW", "NHWC"):
        f = (lambda a: a) if layout == "NCHW" else nhwc
        cases.append({
            "name": name + ("" if layout == "NCHW" else "Nhwc"), "source": source,
            "op": "conv2d", "tolerance": 1, "exact_on_cpuref": exact,
            "params": dict(params, depthwise=False, layout=layout),
            "input": t(f(qx).shape, dtype, f(qx), (scale,), offset),
            "weights": t(f(qw).shape, dtype, f(qw), (scale,), offset),
            "bias": qb,
            "output": t(f(qe).shape, dtype, f(qe), (scale,), offset),
        })


NO_PAD = {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1}

# SimpleConvolution2d3x3Uint8Test (registered with bias, both layouts): the 3x8x16 image of the 3x5 test, two 3x3 filters.
ker33 = np.zeros((2, 3, 3, 3), dtype=np.float32)
ker33[0, 0] = 1.0
ker33[0, 0, 1, 1] = -1.0
ker33[0, 2] = 2.0
ker33[1, 1] = 1.0
exp33 = np.zeros((1, 2, 6, 14), dtype=np.float32)
exp33[0, 0, 0], exp33[0, 0, 1], exp33[0, 0, 2:] = -15.0, -16.0, -14.5
exp33[0, 1, :, :3] = 3.0
exp33[0, 1] += 2.0                      # Bias2 = {0, 2} through ApplyBias
conv_pair("SimpleConvolution2d3x3Uint8Test", "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:38-63,842-918,3488-3497; "
          "src/backends/reference/test/RefLayerTests.cpp:44,48",
          img[None], ker33, [0.0, 2.0], exp33, (0.5, 50), NO_PAD, 0.25)

# Dilation tests (Convolution2d3x3DilationTestCommon: every tensor scale 0.1 / offset 128, registered without bias).
blob = np.zeros((1, 1, 10, 10), dtype=np.float32)
blob[0, 0, 3:6, 4:7] = 1.0
k19 = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
DIL3 = dict(NO_PAD, dilation_x=3, dilation_y=3)
DIL_SRC = "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:1060-1142,%s; src/backends/reference/test/RefLayerTests.cpp:%s"
conv_pair("Convolution2d3x3Dilation3x3Uint8Test", DIL_SRC % ("1150-1205", "91-98"), blob, k19, None,
          np.array([[6, 5, 5, 5]] * 3 + [[3, 2, 2, 2]], dtype=np.float32).reshape(1, 1, 4, 4), (0.1, 128), DIL3, 0.01)
conv_pair("Convolution2d2x3x3Dilation3x3Uint8Test", DIL_SRC % ("1208-1278", "124-131"), np.concatenate([blob, blob], axis=1),
          np.concatenate([k19, k19], axis=1), None,
          np.array([[12, 10, 10, 10]] * 3 + [[6, 4, 4, 4]], dtype=np.float32).reshape(1, 1, 4, 4), (0.1, 128), DIL3, 0.01)
conv_pair("Convolution2d2x2Dilation2x2Padding2x2Stride3x3Uint8Test", DIL_SRC % ("1281-1347", "157-164"),
          np.ones((1, 1, 10, 10), dtype=np.float32), np.array([1, 2, 3, 4], dtype=np.float32).reshape(1, 1, 2, 2), None,
          np.array([[4, 7, 7, 3], [6, 10, 10, 4], [6, 10, 10, 4], [2, 3, 3, 1]], dtype=np.float32).reshape(1, 1, 4, 4), (0.1, 128),
          {"pad_top": 1, "pad_left": 1, "stride_x": 3, "stride_y": 3, "dilation_x": 2, "dilation_y": 2}, 0.01)
# The QAsymmS8 instances use the same scale 0.1 / offset 128: every value saturates at code 127 on the way in, and the
# expected output saturates likewise.  Transcribed as the reference holds them.
conv_pair("Convolution2d3x3Dilation3x3Int8Test", DIL_SRC % ("1150-1205", "83-90"), blob, k19, None,
          np.array([[6, 5, 5, 5]] * 3 + [[3, 2, 2, 2]], dtype=np.float32).reshape(1, 1, 4, 4), (0.1, 128), DIL3, 0.01, -128, 127, S8)
conv_pair("Convolution2d2x2Dilation2x2Padding2x2Stride3x3Int8Test", DIL_SRC % ("1281-1347", "149-156"),
          np.ones((1, 1, 10, 10), dtype=np.float32), np.array([1, 2, 3, 4], dtype=np.float32).reshape(1, 1, 2, 2), None,
          np.array([[4, 7, 7, 3], [6, 10, 10, 4], [6, 10, 10, 4], [2, 3, 3, 1]], dtype=np.float32).reshape(1, 1, 4, 4), (0.1, 128),
          {"pad_top": 1, "pad_left": 1, "stride_x": 3, "stride_y": 3, "dilation_x": 2, "dilation_y": 2}, 0.01,
          -128, 127, S8)

# RefConvolution2dInt8Test (Convolution2dEndToEnd through INetwork/Optimize/IRuntime): registered with QSymmS8 tensors that
# carry offset 10; the QSymmS8 decoder and encoder apply scale and offset exactly as the QAsymmS8 ones do
# (src/backends/reference/workloads/Decoders.hpp, Encoders.hpp), so the case is held as QAsymmS8, the type this path takes.
e2e_in = [1, 5, 2, 3, 5, 8, 7, 3, 6, 3, 3, 3, 9, 1, 9, 4, 1, 8, 1, 3, 6, 8, 1, 9, 2]
e2e_out = [v + 1 for v in (65, 76, 91, 107, 99, 89, 116, 98, 118)]
cases.append({
    "name": "RefConvolution2dInt8Test",
    "source": "src/backends/backendsCommon/test/Convolution2dEndToEndTestImpl.hpp:50-118; src/backends/reference/test/RefEndToEndTests.cpp:722-727",
    "op": "conv2d", "tolerance": 1, "exact_on_cpuref": True,
    "params": dict(NO_PAD, depthwise=False, layout="NHWC"),
    "input": t((1, 5, 5, 1), S8, quantize(e2e_in, 1.0, 10, -128, 127), (1.0,), 10),
    "weights": t((1, 3, 3, 1), S8, quantize([4, 5, 6, 0, 0, 0, 3, 2, 1], 1.0, 10, -128, 127), (1.0,), 10),
    "bias": t((1,), S32, [1], (1.0,), 0),
    "output": t((1, 3, 3, 1), S8, quantize(e2e_out, 1.0, 10, -128, 127), (1.0,), 10),
})

# DepthwiseConvolution2dUint8Test: 2 channels, depth multiplier 2, 5x3 kernel, stride (2, 1), padding top/bottom 1; all
# tensors scale 0.5 / offset 50.  The kernel values are written filter by filter in the test but bound to a [1, 5, 3, 4]
# TensorInfo unpermuted for CpuRef, and are transcribed in that flat order.
dw_in = np.empty((1, 2, 8, 16), dtype=np.float32)
dw_in[0, 0] = 0.5
dw_in[0, 0, 1] = 0.0
dw_in[0, 1] = 0.0
dw_in[0, 1, :, 2] = 1.0
dw_k_flat = [1, 1, 1, 1, -1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1] + [2] * 15 + [0, 0, 0, 0, -1, 0] + [0] * 9 + [0] * 7 + [1] + [0] * 7
dw_exp = np.array(
    [3] * 14 + [5] * 7 + [5.5] * 7 + [5.5] * 7 + [5] * 7 +
    [2.5] * 7 + [3.5] * 7 + [4.5] * 7 + [6] * 7 + [6] * 14 +
    [1, 3, 0, 0, 0, 0, 0] + [2, 4, 0, 0, 0, 0, 0] * 6 + [3, 5, 0, 0, 0, 0, 0] * 5, dtype=np.float32).reshape(1, 4, 6, 7)
for bias_enabled in (True, False):
    e = dw_exp.copy()
    if bias_enabled:
        e += np.array([0, 2, 1, -1], dtype=np.float32).reshape(1, 4, 1, 1)
    for layout in ("NCHW", "NHWC"):
        f = (lambda a: a) if layout == "NCHW" else nhwc
        cases.append({
            "name": ("" if bias_enabled else "Unbiased") + "DepthwiseConvolution2dUint8Test" + ("" if layout == "NCHW" else "Nhwc"),
            "source": "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:2020-2237,3768-3777; "
                      "src/backends/reference/test/RefLayerTests.cpp:294-310",
            "op": "conv2d", "tolerance": 1, "exact_on_cpuref": True,
            "params": {"pad_top": 1, "pad_left": 0, "stride_x": 2, "stride_y": 1,
                       "dilation_x": 1, "dilation_y": 1, "depthwise": True, "layout": layout},
            "input": t(f(dw_in).shape, U8, f(quantize(dw_in, 0.5, 50, 0, 255)), (0.5,), 50),
            "weights": t((1, 5, 3, 4), U8, quantize(dw_k_flat, 0.5, 50, 0, 255), (0.5,), 50),
            "bias": t((4,), S32, quantize([0, 2, 1, -1], 0.25, 0, -2**31, 2**31 - 1), (0.25,), 0) if bias_enabled else None,
            "output": t(f(e).shape, U8, f(quantize(e, 0.5, 50, 0, 255)), (0.5,), 50),
        })

# DepthwiseConvolution2dDepthMul1Uint8Test: 2 channels of a 3x3 image under a 3x3 kernel, expected 0 (+ bias {0, 2}).
dm1_in = np.array([1, 2, 1, 2, 1, 2, 1, 2, 1] * 2, dtype=np.float32).reshape(1, 2, 3, 3)
dm1_k_flat = [1, 0, 1, 0, 0, 0, -1, 0, -1] * 2
for bias_enabled in (True, False):
    e = np.zeros((1, 2, 1, 1), dtype=np.float32) + (np.array([0, 2], dtype=np.float32).reshape(1, 2, 1, 1) if bias_enabled else 0)
    for layout in ("NCHW", "NHWC"):
        f = (lambda a: a) if layout == "NCHW" else nhwc
        cases.append({
            "name": ("" if bias_enabled else "Unbiased") + "DepthwiseConvolution2dDepthMul1Uint8Test" + ("" if layout == "NCHW" else "Nhwc"),
            "source": "src/backends/backendsCommon/test/layerTests/Conv2dTestImpl.cpp:1848-2017,3779-3788; "
                      "src/backends/reference/test/RefLayerTests.cpp:393-428",
            "op": "conv2d", "tolerance": 1, "exact_on_cpuref": True,
            "params": dict(NO_PAD, depthwise=True, layout=layout),
            "input": t(f(dm1_in).shape, U8, f(quantize(dm1_in, 0.5, 50, 0, 255)), (0.5,), 50),
            "weights": t((1, 3, 3, 2), U8, quantize(dm1_k_flat, 0.5, 50, 0, 255), (0.5,), 50),
            "bias": t((2,), S32, quantize([0, 2], 0.25, 0, -2**31, 2**31 - 1), (0.25,), 0) if bias_enabled else None,
            "output": t(f(e).shape, U8, f(quantize(e, 0.5, 50, 0, 255)), (0.5,), 50),
        })

# ---------------------------------------------------------------------------------------------------
# TfLite-delegate vectors (expected values come from the TfLite integer kernels; tolerance 1 in the reference).
cases.append({
    "name": "Conv2DPerChannelInt8Test",
    "source": "delegate/test/Convolution2dTest.cpp:216-289 (SAME padding per src/armnnTfLiteParser/TfLiteParser.cpp:406-427)",
    "op": "conv2d", "tolerance": 1, "exact_on_cpuref": False,
    "params": {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1,
               "depthwise": False, "layout": "NHWC"},
    "input": t((1, 4, 4, 2), S8, [-11, 40, -26, 11, -28, 8, 0, -8, -10, 34, 47, 0, -33, -14, 28, 35,
                                   6, -28, -26, 8, 13, 33, -31, -41, 31, -20, -31, -16, 8, -18, -44, 0], (0.388235,), 1),
    "weights": t((4, 2, 2, 2), QS8, [13, -44, 5, -14, 21, -45, 36, -25, -42, -2, 24, -30, -31, 35, 43, -30,
                                     -20, -5, 25, 17, 18, 20, 4, -46, -49, 9, -3, -20, 46, 5, 7, -15],
                 (1.858268, 2.0, 1.992126, 1.905512), 0, 0),
    "bias": t((4,), S32, [0, 0, 0, 0], (0.721445, 0.7764700055, 0.773414, 0.739787), 0, 0),
    "output": t((1, 4, 4, 4), S8, [-1, 9, 3, 5, 1, -1, 5, 9, 2, 7, -1, 2, 2, 4, 5, 6, 1, 1, 4, 4, 2, 0, -4, -3,
                                   0, 6, 12, 6, 3, 0, -1, -2, 7, -4, 4, 4, 3, 6, 6, 2, 0, -3, -1, 4, 4, 8, 3, 1,
                                   5, 0, 0, 1, 4, 7, 4, 6, 4, 0, 1, 2, 2, 7, 5, 7], (401.960785,), 3),
})

cases.append({
    "name": "Conv2DWithBiasesRelu6Uint8Test",
    "source": "delegate/test/Convolution2dTest.cpp:168-213 (+ generic quantization 1.0/0 -> out scale 2.0, "
              "delegate/test/ConvolutionTestHelper.hpp defaults)",
    "op": "conv2d", "tolerance": 1, "exact_on_cpuref": False,
    "activation": {"function": "BoundedReLu", "a": 6.0, "b": 0.0},
    "params": {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1,
               "depthwise": False, "layout": "NHWC"},
    "input": t((1, 2, 2, 1), U8, [1, 2, 4, 1], (1.0,), 0),
    "weights": t((1, 2, 2, 1), U8, [2, 1, 0, 6], (1.0,), 0),
    "bias": t((1,), S32, [0], (1.0,), 0),
    "output": t((1, 2, 2, 1), U8, [3, 2, 3, 1], (2.0,), 0),
})

cases.append({
    "name": "DepthwiseConv2dSameInt8PerChannelTest",
    "source": "delegate/test/DepthwiseConvolution2dTest.cpp:128-220",
    "op": "conv2d", "tolerance": 1, "exact_on_cpuref": False,
    "params": {"pad_top": 0, "pad_left": 0, "stride_x": 1, "stride_y": 1, "dilation_x": 1, "dilation_y": 1,
               "depthwise": True, "layout": "NHWC"},
    "input": t((1, 4, 4, 4), S8, [3, 3, 3, 4, 4, 4, 0, 0, 0, 3, 4, 3, 0, 2, 2, 3, 3, 0, 3, 0, 0, 3, 2, 1, 4, 1, 2, 2, 0, 0, 0, 4,
                                   3, 2, 2, 2, 2, 1, 0, 4, 4, 3, 2, 4, 3, 2, 0, 0, 4, 1, 4, 4, 1, 0, 4, 3, 3, 2, 0, 3, 1, 1, 0, 2],
               (1.0,), 0),
    "weights": t((1, 2, 2, 16), QS8, [12, 20, 10, 3, 2, 24, 9, 10, 5, 16, 30, 12, 3, 10, 4, 32,
                                      8, 0, 30, 3, 0, 16, 12, 15, 20, 12, 0, 3, 9, 20, 8, 8,
                                      12, 15, 20, 0, 0, 0, 3, 15, 15, 8, 40, 12, 9, 5, 2, 24,
                                      4, 0, 0, 6, 6, 0, 3, 5, 20, 8, 20, 3, 6, 15, 4, 0],
                 (0.25, 0.2, 0.1, 0.3333333333, 0.5, 0.125, 0.33333333, 0.2,
                  0.2, 0.25, 0.1, 0.333333333, 0.3333333333, 0.2, 0.5, 0.125), 0, 3),
    "bias": t((16,), S32, [0] * 16,
              (0.25, 0.2, 0.1, 0.3333333333, 0.5, 0.125, 0.33333333, 0.2,
               0.2, 0.25, 0.1, 0.333333333, 0.3333333333, 0.2, 0.5, 0.125), 0, 0),
    "output": t((1, 4, 4, 16), S8, [
        26, 21, 21, 7, 12, 17, 28, 21, 20, 22, 25, 26, 6, 11, 10, 16,
        16, 16, 4, 12, 7, 18, 28, 27, 30, 20, 12, 14, 16, 19, 17, 6,
        12, 12, 8, 0, 3, 13, 18, 15, 18, 26, 20, 26, 26, 32, 28, 21,
        0, 0, 0, 0, 2, 6, 6, 4, 2, 8, 6, 8, 15, 10, 10, 24,
        20, 21, 9, 7, 3, 6, 15, 16, 17, 22, 17, 22, 17, 18, 14, 7,
        18, 6, 16, 12, 12, 11, 17, 15, 18, 18, 10, 12, 27, 26, 22, 18,
        27, 28, 12, 10, 7, 3, 8, 13, 8, 12, 14, 16, 26, 24, 24, 24,
        9, 9, 6, 0, 0, 0, 2, 6, 0, 0, 0, 0, 4, 8, 8, 16,
        26, 24, 17, 7, 2, 8, 11, 10, 30, 24, 30, 28, 32, 33, 30, 24,
        20, 11, 16, 12, 7, 9, 17, 13, 20, 14, 16, 18, 31, 36, 33, 29,
        28, 25, 19, 9, 6, 13, 20, 19, 2, 8, 6, 8, 17, 17, 15, 25,
        12, 15, 5, 3, 2, 6, 7, 7, 0, 0, 0, 0, 6, 2, 2, 6,
        14, 16, 7, 5, 1, 3, 3, 2, 20, 28, 12, 20, 13, 20, 20, 19,
        9, 4, 10, 4, 0, 4, 8, 6, 4, 16, 12, 16, 12, 18, 18, 15,
        11, 12, 6, 4, 2, 8, 10, 7, 0, 0, 0, 0, 9, 14, 14, 14,
        3, 4, 1, 1, 1, 3, 3, 2, 0, 0, 0, 0, 2, 4, 4, 8], (1.0,), 0),
})

# ---------------------------------------------------------------------------------------------------
# Per-channel decoder literals (float outputs).
decode_cases = [
    {"name": "RefPerChannelDecoderTest1", "source": "src/backends/reference/test/RefPerChannelDecoderTests.cpp:40-60",
     "tensor": t((2, 2, 2, 3), QS8, list(range(24)), (1.0, 2.0), 0, 0), "is_depthwise": False,
     "expected": [float(i) for i in range(12)] + [float(2 * i) for i in range(12, 24)]},
    {"name": "RefPerChannelDecoderTest2", "source": "src/backends/reference/test/RefPerChannelDecoderTests.cpp:63-87",
     "tensor": t((4, 1, 2, 2), QS8, list(range(16)), (1.0, 2.0, 3.0, 4.0), 0, 0), "is_depthwise": True,
     "expected": [float(i * (i // 4 + 1)) for i in range(16)]},
    {"name": "RefPerChannelDecoderTest3", "source": "src/backends/reference/test/RefPerChannelDecoderTests.cpp:90-119",
     "tensor": t((6, 1, 2, 2), QS8, list(range(24)), (1.0, 2.0, 3.0, 4.0, 5.0, 6.0), 0, 0), "is_depthwise": True,
     "expected": [float(i * (i // 4 + 1)) for i in range(24)]},
    {"name": "RefPerChannelDecoderTest4", "source": "src/backends/reference/test/RefPerChannelDecoderTests.cpp:122-152",
     "tensor": t((6, 1, 2, 2), S32, list(range(24)), (1.0, 2.0, 3.0, 4.0, 5.0, 6.0), 0, 0), "is_depthwise": True,
     "expected": [float(i * (i // 4 + 1)) for i in range(24)]},
]

out = {"cases": cases, "decode_cases": decode_cases}
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_literals.json")
with open(path, "w") as f:
    json.dump(out, f, indent=1)
print(f"wrote {path}: {len(cases)} layer cases, {len(decode_cases)} decoder cases")
