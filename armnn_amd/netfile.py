"""Writes a benchmark network (armnn_amd.nets.Network) to one binary file that the C++ side reads back into an
INetwork (armnn_amd/backend/test/NetFile.hpp), so that the backend runs exactly the constants the device executor and
the CPU checker run.

Layout (little endian): magic "MI355XNT", u32 version = 1, u32 batch, u32 tensor count, u32 layer count, the names of
the network's input and output tensors, then the tensors (name, u32 rank, u32 extents with the batch substituted, u32
data type, f32 scale, i32 offset) and the layers in execution order (operation, name, u32 input count, input names,
output name, i32 activation function, f32 a, f32 b, 16 x i32 parameters, f32 beta, weights record, bias record).
A string is u32 length + bytes.  A constant record is u32 present; if present: u32 data type, u32 rank, u32 extents,
u32 scale count, f32 scales, i32 offset, i32 quantization dimension (-1: none), u64 byte count, bytes.
Data type codes are those of armnn_amd.tensor.DataType.
"""
from __future__ import annotations

import struct

import numpy as np

from .nets import Network
from .tensor import QTensor

MAGIC = b"MI355XNT"
PARAMS = ("pad_top", "pad_left", "pad_bottom", "pad_right", "stride_x", "stride_y", "dilation_x", "dilation_y", "depthwise",
          "pool_type", "pool_w", "pool_h", "padding_method", "transpose_weights", "_reserved0", "_reserved1")


def _s(b: bytearray, text: str):
    raw = text.encode()
    b += struct.pack("<I", len(raw)) + raw


def _const(b: bytearray, t: QTensor | None):
    if t is None:
        b += struct.pack("<I", 0)
        return
    info = t.info
    data = np.ascontiguousarray(t.data)
    b += struct.pack("<III", 1, int(info.dtype), len(info.shape))
    b += struct.pack(f"<{len(info.shape)}I", *info.shape)
    b += struct.pack("<I", len(info.scales))
    b += np.asarray(info.scales, np.float32).tobytes()
    b += struct.pack("<iiQ", info.offset, -1 if info.quant_dim is None else info.quant_dim, data.nbytes)
    b += data.tobytes()


def write_net(net: Network, batch: int, path: str) -> None:
    b = bytearray()
    b += MAGIC + struct.pack("<IIII", 1, batch, len(net.tensors), len(net.layers))
    _s(b, net.input)
    _s(b, net.output)
    for name in net.tensors:
        t = net.info(name, batch)
        _s(b, name)
        b += struct.pack("<I", len(t.shape)) + struct.pack(f"<{len(t.shape)}I", *t.shape)
        b += struct.pack("<Ifi", int(t.dtype), t.scales[0], t.offset)
    for l in net.layers:
        _s(b, l.op)
        _s(b, l.name)
        b += struct.pack("<I", len(l.inputs))
        for i in l.inputs:
            _s(b, i)
        _s(b, l.output)
        b += struct.pack("<iff", int(l.act[0]), float(l.act[1]), float(l.act[2]))
        b += struct.pack("<16i", *[int(l.params.get(k, 0)) for k in PARAMS])
        b += struct.pack("<f", float(l.params.get("beta", 1.0)))
        _const(b, l.weights)
        _const(b, l.bias)
    with open(path, "wb") as f:
        f.write(bytes(b))
