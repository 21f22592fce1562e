"""The two synthetic int8 benchmark networks, as plain layer lists with seeded random-init constants.

A network is a list of ``Layer`` records in execution order.  Each layer names its input tensors and its output
tensor; ``Network.tensors`` maps tensor names to TensorInfo.  The same record drives the device executor
(armnn_amd/executor.py) and the CPU checker, so both see identical constants and quantization parameters.

Quantization rule (recorded here because the benchmark configuration only fixes shapes and distributions):
  * weights: int8 = clip(round(N(0,30)), -127, 127), QSymmS8, one scale per output channel,
      s_w[c] = u_c * G / (30 * sqrt(K) * r_in),   u_c ~ U[0.5, 1.5), K = taps per output,
    so that the pre-activation has standard deviation about G (=2.0) when the input has rms r_in;
  * bias: int32 = round(N(0,500)), scale s_in * s_w[c], offset 0;
  * MobileNetV1: activations QAsymmU8; every ReLU6 output has scale 6/255 and offset 0 (its exact range);
    the image has scale 2/255, offset 128 (i.e. [-1, 1]);
  * ResNet-50: activations QAsymmS8; ReLU outputs scale 0.05 offset -128; linear (pre-add) outputs scale 0.1
    offset 0; residual-add outputs (after ReLU) scale 0.1 offset -128; softmax output scale 1/256 with offset 0 (QAsymmU8) / -128 (QAsymmS8) as the optimizer forces
    (src/armnn/Network.cpp:821-835).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import synth
from .tensor import DataType, QTensor, TensorInfo

G_TARGET = 2.0
RELU6_SCALE = float(np.float32(6.0 / 255.0))


def same_padding(in_size, k, stride, dilation=1):
    """TfLite SAME padding (src/armnnTfLiteParser/TfLiteParser.cpp:406-427): front = total // 2."""
    out = (in_size + stride - 1) // stride
    dk = dilation * (k - 1) + 1
    total = max((out - 1) * stride + dk - in_size, 0)
    return out, total // 2, total - total // 2


@dataclass
class Layer:
    op: str                       # conv | depthwise | fc | pool | add | pad | activation | softmax | reshape
    name: str
    inputs: Tuple[str, ...]
    output: str
    weights: Optional[QTensor] = None
    bias: Optional[QTensor] = None
    params: dict = field(default_factory=dict)
    act: Tuple[int, float, float] = (0, 0.0, 0.0)     # fused activation (function, a, b)

    @property
    def macs_per_image(self) -> int:
        return self.params.get("_macs", 0)


@dataclass
class Network:
    name: str
    input: str
    output: str
    tensors: Dict[str, TensorInfo]     # shapes carry batch = 1; executors substitute the batch size
    layers: List[Layer]

    def info(self, name: str, batch: int) -> TensorInfo:
        t = self.tensors[name]
        return TensorInfo((batch,) + tuple(t.shape[1:]), t.dtype, t.scales, t.offset, t.quant_dim)

    def macs_per_image(self, ops=("conv", "depthwise", "fc")) -> int:
        return sum(l.macs_per_image for l in self.layers if l.op in ops)

    def min_bytes_per_image(self, ops=("depthwise",)) -> int:
        """input + output + weights + bias(4 B) + per-channel scale(4 B) of the selected layers, each tensor once."""
        total = 0
        for l in self.layers:
            if l.op not in ops:
                continue
            total += sum(self.tensors[i].num_elements for i in l.inputs) + self.tensors[l.output].num_elements
            if l.weights is not None:
                co = self.tensors[l.output].shape[-1]
                total += l.weights.info.num_elements + 8 * co
        return total


class _Builder:
    def __init__(self, name, seed, act_dtype, weights="per_channel_s8"):
        if weights not in ("per_channel_s8", "per_tensor_u8"):
            raise ValueError(f"unknown weight quantization {weights!r}")
        self.name, self.seed, self.act_dtype, self.weights = name, seed, act_dtype, weights
        self.tensors: Dict[str, TensorInfo] = {}
        self.layers: List[Layer] = []
        self._n = 0

    def _next_seed(self):
        self._n += 1
        return self.seed * 1000 + self._n * 17

    def _weights(self, s, wshape, ws, qdim):
        """Synthetic weights and the scales the bias uses.  "per_channel_s8": QSymmS8, one scale per output channel.
        "per_tensor_u8": QAsymmU8 with one scale and a zero point somewhere in 90..170, the quantization of older
        uint8 models; the same draws, twice as wide, so that codes reach both ends of the range."""
        if self.weights == "per_channel_s8":
            return QTensor(TensorInfo(wshape, DataType.QSymmS8, tuple(ws), 0, qdim), synth.int8_weights(s + 1, wshape)), ws
        zp = 90 + int(synth.uniform01(s + 4, 1, stream=5)[0] * 80.0)
        one = np.asarray([np.float32(np.mean(ws) / 2.0)], np.float32)
        codes = np.clip(2 * synth.int8_weights(s + 1, wshape).astype(np.int32) + zp, 0, 255).astype(np.uint8)
        return QTensor(TensorInfo(wshape, DataType.QAsymmU8, tuple(one), zp, None), codes), one

    def tensor(self, name, shape, scale, offset, dtype=None):
        self.tensors[name] = TensorInfo(tuple(shape), dtype or self.act_dtype, (scale,), offset)
        return name

    def conv(self, name, x, co, k, stride, out_scale, out_offset, act, r_in, depthwise=False, pad="same"):
        xi = self.tensors[x]
        _, h, w, ci = xi.shape
        if pad == "same":
            ho, pt, _ = same_padding(h, k, stride)
            wo, pl, _ = same_padding(w, k, stride)
        else:
            pt = pl = 0
            ho, wo = (h - k) // stride + 1, (w - k) // stride + 1
        if depthwise:
            co = ci
            wshape, taps, qdim = (1, k, k, co), k * k, 3
        else:
            wshape, taps, qdim = (co, k, k, ci), k * k * ci, 0
        s = self._next_seed()
        u = 0.5 + synth.uniform01(s + 3, co, stream=3)
        ws = (u * G_TARGET / (30.0 * np.sqrt(taps) * r_in)).astype(np.float32)
        wt, ws = self._weights(s, wshape, ws, qdim)
        bs = (np.float32(xi.scale) * ws).astype(np.float32)
        bt = QTensor(TensorInfo((co,), DataType.Signed32, tuple(bs), 0, 0 if len(bs) > 1 else None), synth.int32_bias(s + 2, co))
        out = self.tensor(name + ":out", (1, ho, wo, co), out_scale, out_offset)
        params = dict(pad_top=pt, pad_left=pl, stride_x=stride, stride_y=stride, dilation_x=1, dilation_y=1,
                      depthwise=depthwise, _macs=ho * wo * co * taps)
        self.layers.append(Layer("depthwise" if depthwise else "conv", name, (x,), out, wt, bt, params, act))
        return out

    def fc(self, name, x, o, out_scale, out_offset, r_in):
        xi = self.tensors[x]
        k = xi.num_elements // xi.shape[0]
        s = self._next_seed()
        u = 0.5 + synth.uniform01(s + 3, o, stream=3)
        ws = (u * G_TARGET / (30.0 * np.sqrt(k) * r_in)).astype(np.float32)
        wt, ws = self._weights(s, (o, k), ws, 0)
        bs = (np.float32(xi.scale) * ws).astype(np.float32)
        bt = QTensor(TensorInfo((o,), DataType.Signed32, tuple(bs), 0, 0 if len(bs) > 1 else None), synth.int32_bias(s + 2, o))
        out = self.tensor(name + ":out", (1, o), out_scale, out_offset)
        self.layers.append(Layer("fc", name, (x,), out, wt, bt, dict(transpose_weights=True, _macs=k * o)))
        return out

    def pool(self, name, x, pool_type, k, stride, pads=(0, 0, 0, 0), out_scale=None, out_offset=None):
        xi = self.tensors[x]
        _, h, w, c = xi.shape
        pl, pr, pt, pb = pads
        ho, wo = (h + pt + pb - k) // stride + 1, (w + pl + pr - k) // stride + 1
        out = self.tensor(name + ":out", (1, ho, wo, c), xi.scale if out_scale is None else out_scale,
                          xi.offset if out_offset is None else out_offset)
        params = dict(pool_type=pool_type, pool_w=k, pool_h=k, stride_x=stride, stride_y=stride, pad_left=pl,
                      pad_right=pr, pad_top=pt, pad_bottom=pb, padding_method=1)
        self.layers.append(Layer("pool", name, (x,), out, params=params))
        return out

    def reshape(self, name, x, shape):
        xi = self.tensors[x]
        out = self.tensor(name + ":out", shape, xi.scale, xi.offset)
        self.layers.append(Layer("reshape", name, (x,), out))
        return out

    def add(self, name, a, b, out_scale, out_offset, act):
        ai = self.tensors[a]
        out = self.tensor(name + ":out", ai.shape, out_scale, out_offset)
        self.layers.append(Layer("add", name, (a, b), out, act=act))
        return out

    def softmax(self, name, x):
        xi = self.tensors[x]
        off = 0 if self.act_dtype == DataType.QAsymmU8 else -128
        out = self.tensor(name + ":out", xi.shape, float(np.float32(1.0 / 256.0)), off)
        self.layers.append(Layer("softmax", name, (x,), out, params=dict(beta=1.0)))
        return out

    def build(self, inp, out):
        return Network(self.name, inp, out, self.tensors, self.layers)


RELU6 = (2, 6.0, 0.0)
RELU = (1, 0.0, 0.0)
R_IMAGE = 0.58      # rms of uniform codes on [-1, 1]
R_RELU = 1.4        # rms assumed for a ReLU/ReLU6 output whose pre-activation has std 2


def mobilenet_v1(seed: int = 2025, resolution: int = 224, classes: int = 1001, width: float = 1.0,
                 weights: str = "per_channel_s8") -> Network:
    """MobileNetV1-1.0-224-style: stem 3x3/2 -> 32, 13 depthwise-separable blocks, avgpool, FC, softmax."""
    b = _Builder(f"mobilenet_v1_{width}_{resolution}", seed, DataType.QAsymmU8, weights)
    x = b.tensor("input", (1, resolution, resolution, 3), float(np.float32(2.0 / 255.0)), 128)
    ch = lambda c: max(8, int(c * width))
    t = b.conv("stem", x, ch(32), 3, 2, RELU6_SCALE, 0, RELU6, R_IMAGE)
    cfg = [(64, 1), (128, 2), (128, 1), (256, 2), (256, 1), (512, 2), (512, 1), (512, 1), (512, 1), (512, 1), (512, 1),
           (1024, 2), (1024, 1)]
    for i, (co, stride) in enumerate(cfg, start=1):
        t = b.conv(f"dw{i}", t, 0, 3, stride, RELU6_SCALE, 0, RELU6, R_RELU, depthwise=True)
        t = b.conv(f"pw{i}", t, ch(co), 1, 1, RELU6_SCALE, 0, RELU6, R_RELU)
    hw = b.tensors[t].shape[1]
    t = b.pool("avgpool", t, 1, hw, 1)
    t = b.reshape("flatten", t, (1, b.tensors[t].shape[3]))
    t = b.fc("logits", t, classes, 0.1, 128, 1.0)
    t = b.softmax("softmax", t)
    return b.build("input", t)


def resnet50(seed: int = 2026, resolution: int = 224, classes: int = 1001) -> Network:
    """ResNet-50-style: 7x7/2 stem, 3x3/2 maxpool, bottleneck stages [3,4,6,3], requantized residual adds, ReLU."""
    b = _Builder(f"resnet50_{resolution}", seed, DataType.QAsymmS8)
    RS, RO = 0.05, -128            # ReLU outputs inside a block
    AS, AO = 0.1, -128             # ReLU outputs of the residual adds (sum of two branches: wider range)
    LS, LO = 0.1, 0                # linear outputs feeding an add
    R_ADD = 2.8                    # rms assumed for an add output
    x = b.tensor("input", (1, resolution, resolution, 3), float(np.float32(2.0 / 255.0)), 0)
    t = b.conv("stem", x, 64, 7, 2, RS, RO, RELU, R_IMAGE)
    t = b.pool("maxpool", t, 0, 3, 2, pads=(0, 1, 0, 1))
    widths, blocks = [64, 128, 256, 512], [3, 4, 6, 3]
    for s, (wd, nb) in enumerate(zip(widths, blocks)):
        for i in range(nb):
            stride = 2 if (i == 0 and s > 0) else 1
            n = f"s{s + 1}b{i + 1}"
            r_t = R_RELU if (s == 0 and i == 0) else R_ADD
            a = b.conv(n + "_c1", t, wd, 1, 1, RS, RO, RELU, r_t)
            a = b.conv(n + "_c2", a, wd, 3, stride, RS, RO, RELU, R_RELU)
            a = b.conv(n + "_c3", a, wd * 4, 1, 1, LS, LO, (0, 0.0, 0.0), R_RELU)
            if i == 0:
                sc = b.conv(n + "_proj", t, wd * 4, 1, stride, LS, LO, (0, 0.0, 0.0), r_t)
                t = b.add(n + "_add", a, sc, AS, AO, RELU)
            else:
                t = b.add(n + "_add", a, t, AS, AO, RELU)
    hw = b.tensors[t].shape[1]
    t = b.pool("avgpool", t, 1, hw, 1)
    t = b.reshape("flatten", t, (1, b.tensors[t].shape[3]))
    t = b.fc("logits", t, classes, 0.1, 0, 2.0)
    t = b.softmax("softmax", t)
    return b.build("input", t)


def synthetic_input(net: Network, batch: int, seed: int = 7) -> QTensor:
    info = net.info(net.input, batch)
    lo, hi = (0, 255) if info.dtype == DataType.QAsymmU8 else (-128, 127)
    return QTensor(info, synth.uniform_int(seed, info.shape, lo, hi, np.int64))
