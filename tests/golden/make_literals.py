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
