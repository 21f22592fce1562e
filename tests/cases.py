"""Seeded random layer cases shared by the CPU-checker tests and the GPU parity tests."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np

from armnn_amd import synth
from armnn_amd.tensor import DataType, QTensor, TensorInfo


def same_padding(in_size, k, stride, dilation=1):
    """TfLite SAME padding as the parser computes it (src/armnnTfLiteParser/TfLiteParser.cpp:406-427)."""
    out = (in_size + stride - 1) // stride
    dk = dilation * (k - 1) + 1
    total = max((out - 1) * stride + dk - in_size, 0)
    front = total // 2
    return out, front, total - front


def out_size(in_size, k, stride, pad_a, pad_b, dilation=1):
    """Convolution2dLayer.cpp:64-115: 1 + (in + padA + padB - dilatedK) / stride."""
    dk = dilation * (k - 1) + 1
    return 1 + (in_size + pad_a + pad_b - dk) // stride


@dataclass
class ConvCase:
    name: str
    x: QTensor
    w: QTensor
    b: Optional[QTensor]
    out_info: TensorInfo
    params: dict
    act: tuple = (0, 0.0, 0.0)     # (function, a, b)


def make_conv_case(name, seed, *, n=1, h=8, w=8, ci=8, co=8, kh=3, kw=3, stride=(1, 1), dilation=(1, 1),
                   padding="same", depthwise=False, mult=1, in_dtype=DataType.QAsymmS8, in_scale=0.02, in_offset=-3,
                   w_dtype=DataType.QSymmS8, per_axis=True, w_offset=0, w_scale_range=(0.002, 0.02), bias=True,
                   bias_scale_matches=True, out_scale=0.05, out_offset=-128, out_dtype=None, act=(0, 0.0, 0.0),
                   w_std=30.0):
    sx, sy = stride
    dx, dy = dilation
    if padding == "same":
        ho, pt, pb = same_padding(h, kh, sy, dy)
        wo, pl, pr = same_padding(w, kw, sx, dx)
    elif padding == "valid":
        pt = pb = pl = pr = 0
        ho, wo = out_size(h, kh, sy, 0, 0, dy), out_size(w, kw, sx, 0, 0, dx)
    else:
        pt, pb, pl, pr = padding
        ho, wo = out_size(h, kh, sy, pt, pb, dy), out_size(w, kw, sx, pl, pr, dx)
    if depthwise:
        co = ci * mult
    lo, hi = (0, 255) if in_dtype == DataType.QAsymmU8 else (-128, 127)
    xd = synth.uniform_int(seed + 1, (n, h, w, ci), lo, hi, np.int64)
    x = QTensor(TensorInfo((n, h, w, ci), in_dtype, (in_scale,), in_offset), xd)
    wshape = (1, kh, kw, co) if depthwise else (co, kh, kw, ci)
    if w_dtype == DataType.QSymmS8:
        wd = synth.int8_weights(seed + 2, wshape, w_std)
    elif w_dtype == DataType.QAsymmU8:
        wd = np.clip(np.rint(synth.normal(seed + 2, wshape, w_offset, w_std)), 0, 255)
    else:
        wd = np.clip(np.rint(synth.normal(seed + 2, wshape, w_offset, w_std)), -128, 127)
    if per_axis:
        ws = synth.scales(seed + 3, co, *w_scale_range)
        winfo = TensorInfo(wshape, w_dtype, tuple(ws), w_offset, 3 if depthwise else 0)
    else:
        ws = synth.scales(seed + 3, 1, *w_scale_range)
        winfo = TensorInfo(wshape, w_dtype, tuple(ws), w_offset, None)
    wt = QTensor(winfo, wd)
    bt = None
    if bias:
        bd = synth.int32_bias(seed + 4, co)
        if bias_scale_matches:
            bs = (np.float32(in_scale) * ws.astype(np.float32)).astype(np.float32)
        else:
            bs = synth.scales(seed + 5, len(ws), 1e-4, 1e-3)
        binfo = TensorInfo((co,), DataType.Signed32, tuple(bs), 0, 0 if per_axis else None)
        bt = QTensor(binfo, bd)
    out_info = TensorInfo((n, ho, wo, co), out_dtype if out_dtype is not None else in_dtype, (out_scale,), out_offset)
    params = dict(pad_top=pt, pad_left=pl, stride_x=sx, stride_y=sy, dilation_x=dx, dilation_y=dy, depthwise=depthwise)
    return ConvCase(name, x, wt, bt, out_info, params, act)


@dataclass
class FcCase:
    name: str
    x: QTensor
    w: QTensor
    b: Optional[QTensor]
    out_info: TensorInfo
    transpose_weights: bool = True
    act: tuple = (0, 0.0, 0.0)


def make_fc_case(name, seed, *, m=4, k=64, o=32, in_dtype=DataType.QAsymmS8, in_scale=0.02, in_offset=5,
                 w_dtype=DataType.QSymmS8, per_axis=True, w_offset=0, transpose=True, bias=True, out_scale=None,
                 out_offset=0, in_shape=None, act=(0, 0.0, 0.0)):
    lo, hi = (0, 255) if in_dtype == DataType.QAsymmU8 else (-128, 127)
    shape = in_shape if in_shape is not None else (m, k)
    xd = synth.uniform_int(seed + 1, shape, lo, hi, np.int64)
    x = QTensor(TensorInfo(shape, in_dtype, (in_scale,), in_offset), xd)
    wshape = (o, k) if transpose else (k, o)
    if w_dtype == DataType.QSymmS8:
        wd = synth.int8_weights(seed + 2, wshape)
    else:
        l2, h2 = (0, 255) if w_dtype == DataType.QAsymmU8 else (-128, 127)
        wd = np.clip(np.rint(synth.normal(seed + 2, wshape, w_offset, 30.0)), l2, h2)
    if per_axis:
        ws = synth.scales(seed + 3, o)
        winfo = TensorInfo(wshape, w_dtype, tuple(ws), w_offset, 0 if transpose else 1)
    else:
        ws = synth.scales(seed + 3, 1)
        winfo = TensorInfo(wshape, w_dtype, tuple(ws), w_offset, None)
    wt = QTensor(winfo, wd)
    bt = None
    if bias:
        bs = (np.float32(in_scale) * ws.astype(np.float32)).astype(np.float32)
        bt = QTensor(TensorInfo((o,), DataType.Signed32, tuple(bs), 0, 0 if per_axis else None), synth.int32_bias(seed + 4, o))
    if out_scale is None:
        # pre-quantization sum has std ~ sqrt(K) * (30*0.011) * (74*in_scale); keep +-4 sigma inside the int8 range
        out_scale = float(np.sqrt(k) * 0.33 * 74 * in_scale * 4 / 127)
    out_info = TensorInfo((shape[0], o), in_dtype, (out_scale,), out_offset)
    return FcCase(name, x, wt, bt, out_info, transpose, act)


S8, U8, QS8 = DataType.QAsymmS8, DataType.QAsymmU8, DataType.QSymmS8
RELU6 = (2, 6.0, 0.0)
RELU = (1, 0.0, 0.0)


def small_conv_cases():
    """A spread of small shapes covering every branch of the reference's loop nest."""
    c = []
    c.append(make_conv_case("s8_3x3_same", 100, ci=8, co=8))
    c.append(make_conv_case("s8_3x3_same_relu6", 101, ci=16, co=16, act=RELU6))
    c.append(make_conv_case("u8_3x3_same_relu6", 102, ci=16, co=24, in_dtype=U8, in_scale=0.0235, in_offset=128,
                            out_scale=0.0235, out_offset=0, act=RELU6))
    c.append(make_conv_case("s8_1x1_pointwise", 103, h=7, w=9, ci=32, co=64, kh=1, kw=1, act=RELU))
    c.append(make_conv_case("s8_3x3_stride2_same_even", 104, h=12, w=12, ci=8, co=8, stride=(2, 2)))
    c.append(make_conv_case("s8_3x3_stride2_same_odd", 105, h=11, w=13, ci=4, co=12, stride=(2, 2)))
    c.append(make_conv_case("s8_5x3_dilated", 106, h=14, w=15, ci=3, co=5, kh=5, kw=3, dilation=(2, 3)))
    c.append(make_conv_case("s8_valid_stride_xy", 107, h=13, w=17, ci=6, co=7, stride=(3, 2), padding="valid"))
    c.append(make_conv_case("s8_explicit_asym_pad", 108, h=9, w=9, ci=5, co=6, padding=(2, 0, 1, 3)))
    c.append(make_conv_case("s8_per_tensor_weights", 109, ci=8, co=8, per_axis=False))
    c.append(make_conv_case("s8_no_bias", 110, ci=8, co=8, bias=False))
    c.append(make_conv_case("s8_bias_scale_mismatch", 111, ci=8, co=8, bias_scale_matches=False))
    c.append(make_conv_case("u8_asym_u8_weights", 112, ci=8, co=8, in_dtype=U8, in_offset=120, w_dtype=U8, per_axis=False,
                            w_offset=93, out_offset=10))
    c.append(make_conv_case("s8_asym_s8_weights", 113, ci=8, co=8, w_dtype=S8, per_axis=False, w_offset=-7))
    c.append(make_conv_case("s8_batch3", 114, n=3, h=6, w=5, ci=8, co=16))
    c.append(make_conv_case("s8_7x7_stride2_stem", 115, h=20, w=20, ci=3, co=16, kh=7, kw=7, stride=(2, 2)))
    c.append(make_conv_case("u8_3x3_stem_ci3", 116, h=16, w=16, ci=3, co=32, stride=(2, 2), in_dtype=U8, in_offset=128,
                            in_scale=0.0235, out_scale=0.0235, out_offset=0, act=RELU6))
    c.append(make_conv_case("s8_wide_64x64", 117, h=6, w=6, ci=64, co=64, act=RELU6))
    c.append(make_conv_case("s8_1x1_k128_n96", 118, h=5, w=5, ci=128, co=96, kh=1, kw=1))
    # K = 3*3*512 = 4608 taps: the longest accumulation of the ResNet-50 layers (fp32 summation order in the reference)
    c.append(make_conv_case("s8_3x3_ci512_k4608", 119, h=5, w=4, ci=512, co=24, act=RELU))
    # weight-stationary pointwise GEMM kernel: several tiles per wave, ragged M, every chunk depth
    c.append(make_conv_case("pw_u8_k64_n128_m3200", 120, n=2, h=40, w=40, ci=64, co=128, kh=1, kw=1, in_dtype=U8, in_scale=0.0235,
                            in_offset=0, out_scale=0.0235, out_offset=0, act=RELU6))
    c.append(make_conv_case("pw_u8_k256_n512_m189", 121, n=3, h=9, w=7, ci=256, co=512, kh=1, kw=1, in_dtype=U8, in_scale=0.0235,
                            in_offset=0, out_scale=0.0235, out_offset=0, act=RELU6))
    c.append(make_conv_case("pw_s8_k32_n64_m12544", 122, n=1, h=112, w=112, ci=32, co=64, kh=1, kw=1, act=RELU6))
    c.append(make_conv_case("pw_s8_k96_n48", 123, n=1, h=13, w=11, ci=96, co=48, kh=1, kw=1))
    c.append(make_conv_case("pw_s8_k512_n32", 124, n=2, h=14, w=14, ci=512, co=32, kh=1, kw=1, in_offset=-128))
    c.append(make_conv_case("pw_u8_k1024_n1024", 125, n=1, h=7, w=7, ci=1024, co=1024, kh=1, kw=1, in_dtype=U8, in_scale=0.0235,
                            in_offset=0, out_scale=0.0235, out_offset=0, act=RELU6))
    c.append(make_conv_case("pw_s8_stride2_not_pointwise", 126, n=1, h=14, w=14, ci=64, co=64, kh=1, kw=1, stride=(2, 2)))
    # depthwise
    c.append(make_conv_case("dw_u8_3x3_m1", 200, ci=16, depthwise=True, in_dtype=U8, in_scale=0.0235, in_offset=128,
                            out_scale=0.0235, out_offset=0, act=RELU6, w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw_s8_3x3_m1_stride2", 201, h=12, w=10, ci=32, depthwise=True, stride=(2, 2),
                            w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw_s8_3x3_m2", 202, ci=6, depthwise=True, mult=2, w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw_s8_2x2_m4_valid", 203, h=5, w=5, ci=4, depthwise=True, mult=4, kh=2, kw=2, padding="valid",
                            w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw_s8_per_tensor", 204, ci=8, depthwise=True, per_axis=False, w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw_s8_dilated", 205, h=12, w=12, ci=8, depthwise=True, dilation=(2, 2),
                            w_scale_range=(0.01, 0.05)))
    # the v_dot4 + LDS-halo depthwise kernel (channels % 32 == 0, 3x3, stride 1/2) incl. ragged tile edges
    c.append(make_conv_case("dw3_u8_c32_s1", 210, h=19, w=21, ci=32, depthwise=True, in_dtype=U8, in_scale=0.0235, in_offset=128,
                            out_scale=0.0235, out_offset=0, act=RELU6, w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw3_u8_c64_s2_even", 211, n=2, h=20, w=18, ci=64, depthwise=True, stride=(2, 2), in_dtype=U8,
                            in_scale=0.0235, in_offset=3, out_scale=0.0235, out_offset=0, act=RELU6, w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw3_s8_c32_s2_odd", 212, h=17, w=23, ci=32, depthwise=True, stride=(2, 2),
                            w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw3_s8_c96_s1_valid", 213, h=9, w=37, ci=96, depthwise=True, padding="valid",
                            w_scale_range=(0.01, 0.05)))
    c.append(make_conv_case("dw3_s8_c32_pad2", 214, h=10, w=10, ci=32, depthwise=True, padding=(2, 2, 2, 2),
                            w_scale_range=(0.01, 0.05)))
    # stems on the small-Ci v_dot4 kernel
    c.append(make_conv_case("stem_u8_3x3_s2_224", 220, n=2, h=47, w=45, ci=3, co=32, stride=(2, 2), in_dtype=U8, in_offset=128,
                            in_scale=0.0078, out_scale=0.0235, out_offset=0, act=RELU6, w_scale_range=(0.005, 0.02)))
    c.append(make_conv_case("stem_s8_7x7_s2", 221, h=45, w=50, ci=3, co=64, kh=7, kw=7, stride=(2, 2), in_scale=0.0078,
                            in_offset=0, act=RELU, w_scale_range=(0.002, 0.008)))
    c.append(make_conv_case("stem_s8_3x3_s1_ci1", 222, h=20, w=33, ci=1, co=8, in_offset=-100))
    c.append(make_conv_case("stem_s8_5x5_ci4", 223, h=21, w=18, ci=4, co=12, kh=5, kw=5, padding=(1, 2, 0, 3)))
    c.append(make_conv_case("stem_s8_1x1_ci4", 224, h=9, w=9, ci=4, co=16, kh=1, kw=1))
    # several tiles in x and y, rows and images that start at odd byte addresses, a lone last column
    c.append(make_conv_case("stem_u8_3x3_s1_ci3_wide", 225, n=3, h=37, w=71, ci=3, co=20, in_dtype=U8, in_offset=77,
                            out_offset=3))
    c.append(make_conv_case("stem_s8_3x3_s2_ci2", 226, n=2, h=35, w=131, ci=2, co=48, stride=(2, 2), in_offset=5))
    # 32 or 64 output channels: the matrix-core variant (the other counts above stay on v_dot4)
    c.append(make_conv_case("stem_s8_3x3_s1_ci3_co64", 227, n=2, h=33, w=70, ci=3, co=64, in_offset=-20, act=RELU6))
    c.append(make_conv_case("stem_u8_7x7_s2_ci3_co32", 228, n=2, h=39, w=45, ci=3, co=32, kh=7, kw=7, stride=(2, 2), in_dtype=U8,
                            in_offset=111, out_offset=9, w_scale_range=(0.002, 0.008)))
    c.append(make_conv_case("stem_s8_3x3_s2_ci4_co32", 229, n=1, h=18, w=40, ci=4, co=32, stride=(2, 2)))
    # aligned geometry (image rows whole 16-byte chunks, no left padding): the 16-byte staging path, with tiles that reach past
    # the right and bottom edges, on both small-Ci kernels
    c.append(make_conv_case("stem_u8_3x3_s2_ci3_aligned_co32", 230, n=3, h=50, w=80, ci=3, co=32, stride=(2, 2), in_dtype=U8,
                            in_offset=120, out_offset=4, act=RELU6))
    c.append(make_conv_case("stem_s8_3x3_s2_ci4_aligned_co24", 231, n=2, h=34, w=140, ci=4, co=24, stride=(2, 2), in_offset=-9))
    c.append(make_conv_case("stem_s8_3x3_s1_ci4_nopad_co64", 232, n=2, h=21, w=36, ci=4, co=64, padding="valid"))
    c.append(make_conv_case("dw_u8_5x5_c20", 206, h=9, w=9, ci=20, depthwise=True, kh=5, kw=5, in_dtype=U8,
                            in_offset=100, out_offset=3, w_scale_range=(0.005, 0.02)))
    return c


def small_fc_cases():
    c = []
    c.append(make_fc_case("fc_s8_per_axis", 300))
    c.append(make_fc_case("fc_s8_per_tensor", 301, per_axis=False))
    c.append(make_fc_case("fc_u8_asym_weights", 302, in_dtype=U8, in_offset=63, w_dtype=U8, per_axis=False, w_offset=93,
                          out_offset=100))
    c.append(make_fc_case("fc_s8_not_transposed", 303, transpose=False))
    c.append(make_fc_case("fc_s8_no_bias", 304, bias=False))
    c.append(make_fc_case("fc_s8_4d_input", 305, in_shape=(3, 2, 4, 8), k=64, o=10))
    c.append(make_fc_case("fc_s8_m1_k1024_o1001", 306, m=1, k=1024, o=1001))
    c.append(make_fc_case("fc_s8_k4096", 307, m=3, k=4096, o=40))
    c.append(make_fc_case("fc_s8_relu", 308, m=5, k=100, o=33, act=RELU))
    # few rows: the weight-streaming matrix-vector kernel (1..4 rows, K % 16 == 0), ragged output counts
    c.append(make_fc_case("fc_u8_m2_k80_o10", 309, m=2, k=80, o=10, in_dtype=U8, in_offset=131, out_offset=7, act=RELU6))
    c.append(make_fc_case("fc_s8_m4_k2048_o203", 310, m=4, k=2048, o=203))
    c.append(make_fc_case("fc_s8_m1_k48_o5_not_transposed", 311, m=1, k=48, o=5, transpose=False, bias=False))
    # a few dozen rows: 32x32 tiles with K split over the waves (5..64 rows, K % 16 == 0, K >= 128)
    c.append(make_fc_case("fc_s8_m32_k1024_o1001", 312, m=32, k=1024, o=1001))
    c.append(make_fc_case("fc_u8_m33_k144_o36", 313, m=33, k=144, o=36, in_dtype=U8, in_offset=120, out_offset=3, act=RELU6))
    c.append(make_fc_case("fc_s8_m64_k2048_o100", 314, m=64, k=2048, o=100, per_axis=False))
    c.append(make_fc_case("fc_s8_m5_k128_o7_no_bias", 315, m=5, k=128, o=7, bias=False))
    return c
