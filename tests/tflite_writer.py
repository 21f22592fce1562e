"""Writes small .tflite flatbuffers for the parser tests (the schema's field numbers, nothing generated).

Objects are laid out front to back: a table's vtable, then the table with its inline fields, then whatever the table
refers to -- FlatBuffers offsets to strings, vectors and tables are unsigned and point forwards, so children follow
their parent.  A table is described as {field number: value}; a value is ("i"|"b"|"B"|"f"|"I", number) for a scalar,
a str, a dict (sub-table), a list of dicts (vector of tables) or a numpy array (vector of numbers).
"""
from __future__ import annotations

import struct

import numpy as np

_SIZES = {"b": 1, "B": 1, "i": 4, "I": 4, "f": 4}


class _Out:
    def __init__(self):
        self.b = bytearray()

    def align(self, n):
        while len(self.b) % n:
            self.b.append(0)

    def patch_u32(self, at, value):
        struct.pack_into("<I", self.b, at, value)


def _place(out: _Out, value) -> int:
    """Writes `value` at the end of the buffer and returns the position offsets to it must point at."""
    if isinstance(value, dict):
        return _place_table(out, value)
    if isinstance(value, str):
        raw = value.encode()
        out.align(4)
        pos = len(out.b)
        out.b += struct.pack("<I", len(raw)) + raw + b"\0"
        return pos
    if isinstance(value, list):                       # vector of tables
        out.align(4)
        pos = len(out.b)
        out.b += struct.pack("<I", len(value)) + bytes(4 * len(value))
        for k, child in enumerate(value):
            slot = pos + 4 + 4 * k
            out.patch_u32(slot, _place(out, child) - slot)
        return pos
    arr = np.ascontiguousarray(value)
    item = arr.dtype.itemsize
    out.align(4)
    while (len(out.b) + 4) % max(item, 4):            # the elements, not the length word, carry the alignment
        out.b.append(0)
    pos = len(out.b)
    out.b += struct.pack("<I", arr.size) + arr.tobytes()
    return pos


def _place_table(out: _Out, fields: dict) -> int:
    n = (max(fields) + 1) if fields else 0
    # inline layout: soffset, then every field at its natural alignment
    layout, size = {}, 4
    for k in sorted(fields):
        v = fields[k]
        width = _SIZES[v[0]] if isinstance(v, tuple) else 4
        size = (size + width - 1) // width * width
        layout[k] = size
        size += width
    out.align(2)
    vt = len(out.b)
    out.b += struct.pack("<HH", 4 + 2 * n, size) + b"".join(struct.pack("<H", layout.get(k, 0)) for k in range(n))
    out.align(4)
    pos = len(out.b)
    out.b += bytes(size)
    struct.pack_into("<i", out.b, pos, pos - vt)
    pending = []
    for k, v in fields.items():
        at = pos + layout[k]
        if isinstance(v, tuple):
            struct.pack_into("<" + v[0], out.b, at, v[1])
        else:
            pending.append((at, v))
    for at, v in pending:
        out.patch_u32(at, _place(out, v) - at)
    return pos


def build(root: dict) -> bytes:
    out = _Out()
    out.b += bytes(4) + b"TFL3"
    out.patch_u32(0, _place_table(out, root))
    return bytes(out.b)


# ---- the TfLite schema, as far as the tests need it ----------------------------------------------------------------------
FLOAT32, INT32, UINT8, INT8 = 0, 2, 3, 9
ADD, AVERAGE_POOL_2D, CONV_2D, DEPTHWISE_CONV_2D, FULLY_CONNECTED, MAX_POOL_2D, RESHAPE, SOFTMAX, PAD, TANH, MEAN = 0, 1, 3, 4, 9, 17, 22, 25, 34, 28, 40
RELU, RELU_N1_TO_1, RELU6, SQUEEZE, QUANTIZE = 19, 20, 21, 43, 114
SAME, VALID = 0, 1
ACT_NONE, ACT_RELU, ACT_RELU_N1_TO_1, ACT_RELU6 = 0, 1, 2, 3
# BuiltinOptions union tags
OPT_CONV, OPT_DEPTHWISE, OPT_POOL, OPT_FC, OPT_SOFTMAX, OPT_ADD, OPT_PAD, OPT_RESHAPE, OPT_REDUCER = 1, 2, 5, 8, 9, 11, 22, 17, 27


class ModelBuilder:
    def __init__(self):
        self.buffers = [{}]                            # buffer 0 is the empty one by convention
        self.tensors = []
        self.operators = []
        self.opcodes = []

    def tensor(self, name, shape, ttype, scale=None, zero_point=0, data=None, quantized_dimension=0):
        fields = {0: np.asarray(shape, np.int32), 1: ("b", ttype), 3: name}
        if data is not None:
            self.buffers.append({0: np.ascontiguousarray(data).view(np.uint8).reshape(-1)})
            fields[2] = ("I", len(self.buffers) - 1)
        if scale is not None:
            scales = np.atleast_1d(np.asarray(scale, np.float32))
            zeros = np.zeros(scales.size, np.int64) + np.asarray(zero_point, np.int64)
            fields[4] = {2: scales, 3: zeros, 6: ("i", quantized_dimension)}
        self.tensors.append(fields)
        return len(self.tensors) - 1

    def op(self, code, inputs, outputs, options_type=0, options=None):
        if code not in self.opcodes:
            self.opcodes.append(code)
        fields = {0: ("I", self.opcodes.index(code)), 1: np.asarray(inputs, np.int32), 2: np.asarray(outputs, np.int32)}
        if options is not None:
            fields[3] = ("B", options_type)
            fields[4] = options
        self.operators.append(fields)

    def finish(self, inputs, outputs, description="written by the parser tests"):
        graph = {0: self.tensors, 1: np.asarray(inputs, np.int32), 2: np.asarray(outputs, np.int32), 3: self.operators, 4: "main"}
        codes = [{0: ("b", min(c, 127)), 2: ("i", 1), 3: ("i", c)} for c in self.opcodes]
        return build({0: ("I", 3), 1: codes, 2: [graph], 3: description, 4: self.buffers})
