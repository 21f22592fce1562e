"""Reads a quantized .tflite model into a nets.Network, with the conventions of Arm NN's TfLite parser.

Only what the device path runs is accepted: 8-bit quantized CONV_2D, DEPTHWISE_CONV_2D, FULLY_CONNECTED,
AVERAGE_POOL_2D, MAX_POOL_2D, ADD, PAD, MEAN (over height and width), RELU, RELU_N1_TO_1, RELU6, RESHAPE, SQUEEZE, QUANTIZE (between 8-bit quantizations) and SOFTMAX, one subgraph, one input, one output.  Anything else raises
``UnsupportedModel`` naming the operator -- nothing is approximated or skipped.

What is taken from the reference parser (src/armnnTfLiteParser/TfLiteParser.cpp):
  * SAME padding, front = total // 2 (CalcPadding, :406-427); VALID = none;
  * pooling excludes padding from the divisor and rounds output sizes down (ParsePool: PaddingMethod::Exclude, Floor);
  * a fused activation becomes ReLu, BoundedReLu(6, 0) or BoundedReLu(1, -1) behind the layer, in the layer's own
    output quantization (AddFusedActivationLayer, :5405-5464);
  * FULLY_CONNECTED flattens an input of more than two dimensions to [elements / K, K] first (ParseFullyConnected);
    TfLite keeps FC weights as [outputs, K], i.e. m_TransposeWeightMatrix = true;
  * convolution weights are [O, H, W, I] and depthwise weights [1, H, W, I * multiplier], as the reference keeps them;
  * MEAN over the height and width of an NHWC tensor runs as an average pooling over the whole feature map: the
    reference's Reduce (workloads/Reduce.cpp:69-173) adds the window up in the same order and divides by the same
    count, and the two give the same bytes;
  * per-channel weights carry their scales along quantized_dimension; the int32 bias keeps the scale the file states.

The file format is FlatBuffers; the few accessors needed are written out here (the schema is tensorflow/lite/schema/
schema.fbs, version 3: field numbers are cited where they are used).
"""
from __future__ import annotations

import struct
from typing import Dict, List, Optional, Tuple

import numpy as np

from .nets import Layer, Network, same_padding
from .tensor import DataType, QTensor, TensorInfo


class UnsupportedModel(ValueError):
    pass


# ---- FlatBuffers ---------------------------------------------------------------------------------------------------------
class _Table:
    """A FlatBuffers table: fields are looked up through the vtable the table points back to."""

    def __init__(self, buf: bytes, pos: int):
        self.buf, self.pos = buf, pos
        self.vt = pos - struct.unpack_from("<i", buf, pos)[0]
        self.vt_size = struct.unpack_from("<H", buf, self.vt)[0]

    def _field(self, k: int) -> int:
        off = 4 + 2 * k
        if off >= self.vt_size:
            return 0
        rel = struct.unpack_from("<H", self.buf, self.vt + off)[0]
        return self.pos + rel if rel else 0

    def scalar(self, k: int, fmt: str, default=0):
        p = self._field(k)
        return struct.unpack_from("<" + fmt, self.buf, p)[0] if p else default

    def table(self, k: int) -> Optional["_Table"]:
        p = self._field(k)
        return _Table(self.buf, p + struct.unpack_from("<I", self.buf, p)[0]) if p else None

    def _vector(self, k: int) -> Tuple[int, int]:
        p = self._field(k)
        if not p:
            return 0, 0
        v = p + struct.unpack_from("<I", self.buf, p)[0]
        return v + 4, struct.unpack_from("<I", self.buf, v)[0]

    def string(self, k: int) -> str:
        start, n = self._vector(k)
        return self.buf[start:start + n].decode("utf-8", "replace") if start else ""

    def numbers(self, k: int, dtype) -> np.ndarray:
        start, n = self._vector(k)
        return np.frombuffer(self.buf, dtype=dtype, count=n, offset=start).copy() if start else np.zeros(0, dtype)

    def tables(self, k: int) -> List["_Table"]:
        start, n = self._vector(k)
        out = []
        for i in range(n):
            p = start + 4 * i
            out.append(_Table(self.buf, p + struct.unpack_from("<I", self.buf, p)[0]))
        return out


# ---- schema constants ------------------------------------------------------------------------------------------------------
_UINT8, _INT32, _INT8 = 3, 2, 9                                   # TensorType
_OPS = {0: "ADD", 1: "AVERAGE_POOL_2D", 3: "CONV_2D", 4: "DEPTHWISE_CONV_2D", 9: "FULLY_CONNECTED", 17: "MAX_POOL_2D",
        19: "RELU", 20: "RELU_N1_TO_1", 21: "RELU6", 22: "RESHAPE", 25: "SOFTMAX", 34: "PAD", 40: "MEAN", 43: "SQUEEZE",
        114: "QUANTIZE"}                  # BuiltinOperator
_ACT = {0: (0, 0.0, 0.0), 1: (1, 0.0, 0.0), 2: (2, 1.0, -1.0), 3: (2, 6.0, 0.0)}    # NONE, RELU, RELU_N1_TO_1, RELU6
_SAME, _VALID = 0, 1


def _fused(code: int):
    if code not in _ACT:
        raise UnsupportedModel(f"fused activation {code} (NONE, RELU, RELU_N1_TO_1 and RELU6 are supported)")
    return _ACT[code]


def _pad(padding: int, size: int, k: int, stride: int, dilation: int = 1) -> Tuple[int, int]:
    if padding == _VALID:
        return 0, 0
    _, front, back = same_padding(size, k, stride, dilation)
    return front, back


class _Model:
    def __init__(self, data: bytes):
        if len(data) < 8 or data[4:8] != b"TFL3":
            raise UnsupportedModel("not a TfLite flatbuffer (file identifier TFL3 missing)")
        self.buf = data
        root = _Table(data, struct.unpack_from("<I", data, 0)[0])
        self.opcodes = root.tables(1)                              # Model.operator_codes
        graphs = root.tables(2)                                    # Model.subgraphs
        if len(graphs) != 1:
            raise UnsupportedModel(f"{len(graphs)} subgraphs (one is supported)")
        self.graph = graphs[0]
        self.buffers = root.tables(4)                              # Model.buffers
        self.tensors = self.graph.tables(0)                        # SubGraph.tensors
        self.description = root.string(3)

    def opcode(self, op: _Table) -> int:
        oc = self.opcodes[op.scalar(0, "I")]                      # Operator.opcode_index
        # OperatorCode.builtin_code (3) superseded deprecated_builtin_code (0, a byte) for codes above 127
        return max(oc.scalar(3, "i"), oc.scalar(0, "b"))

    def info(self, index: int, constant: bool = False) -> TensorInfo:
        t = self.tensors[index]
        shape = tuple(int(v) for v in t.numbers(0, np.int32))     # Tensor.shape
        ttype = t.scalar(1, "b")                                   # Tensor.type
        q = t.table(4)                                             # Tensor.quantization
        scales = q.numbers(2, np.float32) if q else np.zeros(0, np.float32)       # QuantizationParameters.scale
        zeros = q.numbers(3, np.int64) if q else np.zeros(0, np.int64)            # .zero_point
        qdim = q.scalar(6, "i") if q else 0                        # .quantized_dimension
        name = t.string(3)
        if ttype == _INT32:
            dtype = DataType.Signed32
        elif ttype == _UINT8:
            dtype = DataType.QAsymmU8
        elif ttype == _INT8:
            # the reference maps per-channel int8 constants to QSymmS8 and everything else to QAsymmS8
            dtype = DataType.QSymmS8 if (constant and len(scales) > 1) else DataType.QAsymmS8
        else:
            raise UnsupportedModel(f"tensor '{name}' has TensorType {ttype}; only UINT8, INT8 and INT32 run on the device")
        if len(scales) == 0:
            if dtype != DataType.Signed32:
                raise UnsupportedModel(f"tensor '{name}' carries no quantization")
            scales = np.ones(1, np.float32)
        if len(scales) > 1:
            if np.any(zeros != 0):
                raise UnsupportedModel(f"tensor '{name}': per-channel quantization with non-zero zero points")
            return TensorInfo(shape, dtype, tuple(float(s) for s in scales), 0, int(qdim))
        return TensorInfo(shape, dtype, (float(scales[0]),), int(zeros[0]) if len(zeros) else 0)

    def constant(self, index: int) -> Optional[QTensor]:
        t = self.tensors[index]
        b = self.buffers[t.scalar(2, "I")]                         # Tensor.buffer -> Buffer.data
        info = self.info(index, constant=True)
        np_dtype = {DataType.Signed32: np.int32, DataType.QAsymmU8: np.uint8}.get(info.dtype, np.int8)
        raw = b.numbers(0, np.uint8)
        if raw.size == 0:
            return None
        data = raw.view(np_dtype).reshape(info.shape)
        return QTensor(info, data.astype(np.int64))


def load(path: str) -> Network:
    with open(path, "rb") as f:
        return parse(f.read(), name=path.rsplit("/", 1)[-1])


def parse(data: bytes, name: str = "tflite") -> Network:
    try:
        return _parse(data, name)
    except (struct.error, IndexError, OverflowError, KeyError, TypeError, AttributeError) as e:
        # offsets that lead outside the buffer, vectors longer than the file, operator or tensor indices out of range
        raise UnsupportedModel(f"malformed flatbuffer: {e}") from e
    except ValueError as e:
        if isinstance(e, UnsupportedModel):
            raise
        raise UnsupportedModel(f"malformed flatbuffer: {e}") from e


def _parse(data: bytes, name: str) -> Network:
    m = _Model(data)
    inputs = m.graph.numbers(1, np.int32)                          # SubGraph.inputs
    outputs = m.graph.numbers(2, np.int32)                         # SubGraph.outputs
    if len(inputs) != 1 or len(outputs) != 1:
        raise UnsupportedModel(f"{len(inputs)} inputs and {len(outputs)} outputs (one of each is supported)")
    tname = lambda i: f"t{i}:{m.tensors[i].string(3)}"
    tensors: Dict[str, TensorInfo] = {}
    layers: List[Layer] = []

    def activation_tensor(i: int) -> str:
        n = tname(i)
        if n not in tensors:
            tensors[n] = m.info(i)
        return n

    def need_constant(i: int, what: str, op: str) -> QTensor:
        c = m.constant(i) if i >= 0 else None
        if c is None:
            raise UnsupportedModel(f"{op}: {what} must be a constant tensor")
        return c

    activation_tensor(int(inputs[0]))
    for k, op in enumerate(m.graph.tables(3)):                     # SubGraph.operators
        code = m.opcode(op)
        kind = _OPS.get(code)
        ins = [int(v) for v in op.numbers(1, np.int32)]            # Operator.inputs
        outs = [int(v) for v in op.numbers(2, np.int32)]           # Operator.outputs
        o = op.table(4)                                            # Operator.builtin_options
        lname = f"op{k}:{kind}"
        if kind is None:
            raise UnsupportedModel(f"operator {k} has builtin code {code}, which the device path does not run")
        x = activation_tensor(ins[0])
        xi = tensors[x]
        y = activation_tensor(outs[0])
        yi = tensors[y]

        def expect(shape, what=kind):
            # buffers are sized from the file's shapes and kernels from the operator's arithmetic: they have to agree
            if tuple(yi.shape) != tuple(shape):
                raise UnsupportedModel(f"{what}: the file gives the output shape {yi.shape}, the operator produces {tuple(shape)}")

        if kind in ("CONV_2D", "DEPTHWISE_CONV_2D"):
            dw = kind == "DEPTHWISE_CONV_2D"
            w = need_constant(ins[1], "weights", kind)
            b = need_constant(ins[2], "bias", kind) if len(ins) > 2 and ins[2] >= 0 else None
            padding, sw, sh = o.scalar(0, "b"), o.scalar(1, "i"), o.scalar(2, "i")
            act = _fused(o.scalar(4 if dw else 3, "b"))
            dwf, dhf = o.scalar(5 if dw else 4, "i", 1), o.scalar(6 if dw else 5, "i", 1)
            _, h, wd, ci = xi.shape
            kh, kw = w.info.shape[1], w.info.shape[2]
            pt, _ = _pad(padding, h, kh, sh, dhf)
            pl, _ = _pad(padding, wd, kw, sw, dwf)
            if len(xi.shape) != 4 or len(w.info.shape) != 4 or min(sw, sh, dwf, dhf) < 1:
                raise UnsupportedModel(f"{kind}: needs 4-D tensors and positive strides and dilations")
            if dw and (w.info.shape[0] != 1 or w.info.shape[3] % ci != 0):
                raise UnsupportedModel("DEPTHWISE_CONV_2D weights must be [1, H, W, I * multiplier]")
            if not dw and w.info.shape[3] != ci:
                raise UnsupportedModel("CONV_2D weights must be [O, H, W, I]")
            _, pb = _pad(padding, h, kh, sh, dhf)
            _, pr = _pad(padding, wd, kw, sw, dwf)
            expect((xi.shape[0], (h + pt + pb - (dhf * (kh - 1) + 1)) // sh + 1, (wd + pl + pr - (dwf * (kw - 1) + 1)) // sw + 1,
                    w.info.shape[3] if dw else w.info.shape[0]))
            if b is not None:
                b = _bias_like_reference(b, xi, w.info)
            taps = kh * kw if dw else kh * kw * ci
            params = dict(pad_top=pt, pad_left=pl, stride_x=sw, stride_y=sh, dilation_x=dwf, dilation_y=dhf, depthwise=dw,
                          _macs=yi.shape[1] * yi.shape[2] * yi.shape[3] * taps)
            layers.append(Layer("depthwise" if dw else "conv", lname, (x,), y, w, b, params, act))
        elif kind == "FULLY_CONNECTED":
            w = need_constant(ins[1], "weights", kind)
            b = need_constant(ins[2], "bias", kind) if len(ins) > 2 and ins[2] >= 0 else None
            kdim = w.info.shape[1]
            if len(xi.shape) > 2 or xi.shape[-1] != kdim:
                flat = f"{x}:flat"
                tensors[flat] = TensorInfo((xi.num_elements // kdim, kdim), xi.dtype, xi.scales, xi.offset)
                layers.append(Layer("reshape", lname + ":flatten", (x,), flat))
                x, xi = flat, tensors[flat]
            if b is not None:
                b = _bias_like_reference(b, xi, w.info)
            if len(w.info.shape) != 2 or xi.num_elements % kdim != 0:
                raise UnsupportedModel("FULLY_CONNECTED: weights must be [outputs, K] with K dividing the input")
            if yi.num_elements != xi.shape[0] * w.info.shape[0]:
                expect((xi.shape[0], w.info.shape[0]))
            if len(yi.shape) != 2:
                tensors[y] = yi = TensorInfo((xi.shape[0], w.info.shape[0]), yi.dtype, yi.scales, yi.offset)
            layers.append(Layer("fc", lname, (x,), y, w, b, dict(transpose_weights=True, _macs=kdim * w.info.shape[0]),
                                _fused(o.scalar(0, "b")) if o else _fused(0)))
        elif kind in ("AVERAGE_POOL_2D", "MAX_POOL_2D"):
            padding, sw, sh, fw, fh = o.scalar(0, "b"), o.scalar(1, "i"), o.scalar(2, "i"), o.scalar(3, "i"), o.scalar(4, "i")
            if len(xi.shape) != 4 or min(sw, sh, fw, fh) < 1:
                raise UnsupportedModel(f"{kind}: needs a 4-D tensor and positive window and strides")
            _, h, wd, _ = xi.shape
            pt, pb = _pad(padding, h, fh, sh)
            pl, pr = _pad(padding, wd, fw, sw)
            expect((xi.shape[0], (h + pt + pb - fh) // sh + 1, (wd + pl + pr - fw) // sw + 1, xi.shape[3]))
            params = dict(pool_type=0 if kind == "MAX_POOL_2D" else 1, pool_w=fw, pool_h=fh, stride_x=sw, stride_y=sh,
                          pad_left=pl, pad_right=pr, pad_top=pt, pad_bottom=pb, padding_method=1)
            layers.append(Layer("pool", lname, (x,), y, params=params, act=_fused(o.scalar(5, "b"))))
        elif kind == "ADD":
            x1 = activation_tensor(ins[1])
            if tensors[x1].shape != xi.shape:
                raise UnsupportedModel("ADD with broadcasting")
            expect(xi.shape)
            layers.append(Layer("add", lname, (x, x1), y, act=_fused(o.scalar(0, "b")) if o else _fused(0)))
        elif kind == "PAD":
            p = need_constant(ins[1], "paddings", kind)
            pads = tuple((int(a), int(b)) for a, b in p.data.reshape(-1, 2))
            if len(pads) != len(xi.shape) or len(pads) > 4 or any(a < 0 or b < 0 for a, b in pads):
                raise UnsupportedModel("PAD: one non-negative (before, after) pair per dimension, at most 4 dimensions")
            expect(tuple(d + a + b for d, (a, b) in zip(xi.shape, pads)))
            # TfLite pads with the real number 0, which is the zero point in the tensor's own code
            layers.append(Layer("pad", lname, (x,), y, params=dict(pad_list=pads, pad_value=float(xi.offset))))
        elif kind == "MEAN":
            axes = sorted(int(v) % 4 for v in need_constant(ins[1], "axes", kind).data.ravel())
            if len(xi.shape) != 4 or axes != [1, 2]:
                raise UnsupportedModel("MEAN: only the mean over height and width of a 4-D tensor runs on the device")
            n_, h, wd, c_ = xi.shape
            keep = bool(o.scalar(0, "b")) if o else False                     # ReducerOptions.keep_dims
            expect((n_, 1, 1, c_) if keep else (n_, c_))
            pooled = y
            if not keep:
                pooled = f"{y}:pooled"
                tensors[pooled] = TensorInfo((n_, 1, 1, c_), yi.dtype, yi.scales, yi.offset)
            params = dict(pool_type=1, pool_w=wd, pool_h=h, stride_x=1, stride_y=1, pad_left=0, pad_right=0, pad_top=0, pad_bottom=0,
                          padding_method=1)
            layers.append(Layer("pool", lname, (x,), pooled, params=params))
            if not keep:
                layers.append(Layer("reshape", lname + ":squeeze", (pooled,), y))
        elif kind in ("RELU", "RELU_N1_TO_1", "RELU6"):
            # an Activation layer of its own (ParseRelu / ParseReluN1To1 / ParseRelu6); it re-quantizes when the output
            # tensor's quantization differs from the input's
            expect(xi.shape)
            layers.append(Layer("activation", lname, (x,), y, act=_fused({"RELU": 1, "RELU_N1_TO_1": 2, "RELU6": 3}[kind])))
        elif kind == "QUANTIZE":
            # a Quantize layer (ParseQuantize); between two 8-bit quantizations it decodes and encodes every value
            # (RefQuantizeWorkload.cpp), which is what an Activation layer without a function does
            expect(xi.shape)
            layers.append(Layer("activation", lname, (x,), y, act=(0, 0.0, 0.0)))
        elif kind == "RESHAPE":
            if yi.num_elements != xi.num_elements:
                raise UnsupportedModel("RESHAPE: input and output differ in their number of elements")
            layers.append(Layer("reshape", lname, (x,), y))
        elif kind == "SQUEEZE":
            # a Reshape layer (ParseSqueeze); the output keeps the input's dimensions except some of extent 1
            kept = iter(yi.shape)
            nxt = next(kept, None)
            for extent in xi.shape:
                if nxt is not None and extent == nxt:
                    nxt = next(kept, None)
                elif extent != 1:
                    nxt = -1
                    break
            if nxt is not None:
                raise UnsupportedModel(f"SQUEEZE: {tuple(yi.shape)} is not {tuple(xi.shape)} without some of its dimensions of extent 1")
            layers.append(Layer("reshape", lname, (x,), y))
        elif kind == "SOFTMAX":
            expect(xi.shape)
            if len(xi.shape) != 2:
                raise UnsupportedModel("SOFTMAX: runs over the columns of a 2-D tensor")
            layers.append(Layer("softmax", lname, (x,), y, params=dict(beta=float(o.scalar(0, "f", 1.0)) if o else 1.0)))
    return Network(name, tname(int(inputs[0])), tname(int(outputs[0])), tensors, layers)


def _bias_like_reference(b: QTensor, x: TensorInfo, w: TensorInfo) -> QTensor:
    """The bias keeps the scale(s) the file gives it, as the reference's decoder reads them; what the reference checks
    (ValidateBiasTensorQuantization, src/backends/backendsCommon/WorkloadData.cpp) is checked here as well: Signed32,
    zero point 0, as many scales as the weights have."""
    if b.info.dtype != DataType.Signed32:
        raise UnsupportedModel("bias is not INT32")
    if b.info.offset != 0:
        raise UnsupportedModel("bias zero point is not 0")
    if len(b.info.scales) != len(w.scales):
        raise UnsupportedModel("bias and weights differ in their number of quantization scales")
    return b


def main(argv=None) -> int:
    """python -m armnn_amd.tflite model.tflite [--batch N] [--iterations K]: loads the model, runs it on the device on
    seeded synthetic input and prints the layer list, the class distribution of the first image and the throughput
    (what tests/ExecuteNetwork reports for a model in the reference: inference time over a number of iterations)."""
    import argparse
    import json
    import time

    from . import nets
    from .executor import DeviceNetwork

    ap = argparse.ArgumentParser()
    ap.add_argument("model")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--iterations", type=int, default=50)
    ap.add_argument("--lanes", type=int, default=1)
    a = ap.parse_args(argv)
    net = load(a.model)
    for l in net.layers:
        print(f"{l.op:>9s} {l.name:<28s} {' '.join(str(net.tensors[i].shape) for i in l.inputs)} -> {net.tensors[l.output].shape}")
    dn = DeviceNetwork(net, a.batch, lanes=a.lanes)
    x = nets.synthetic_input(net, a.batch)
    y = dn.run(x)
    t0 = time.perf_counter()
    for _ in range(a.iterations):
        dn.enqueue()
    dn.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / a.iterations
    dn.close()
    print(json.dumps({"model": net.name, "batch": a.batch, "ms_per_inference": ms, "images_per_sec": a.batch / ms * 1e3,
                      "first_image_output": [int(v) for v in y.data[0].ravel()[:16]]}))
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())
