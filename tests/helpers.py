"""Shared helpers for the parity tests."""
from __future__ import annotations

import json
import os

import numpy as np

from armnn_amd.tensor import DataType, QTensor, TensorInfo, numpy_dtype

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_json(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def tensor_from_json(d) -> QTensor:
    if d is None:
        return None
    info = TensorInfo(tuple(d["shape"]), DataType[d["dtype"]], tuple(d["scales"]), d["offset"], d["quant_dim"])
    data = np.asarray(d["data"], dtype=np.int64).astype(numpy_dtype(info.dtype)).reshape(info.shape)
    return QTensor(info, data)


def lsb_diff(a: np.ndarray, b: np.ndarray):
    """(max |a-b|, fraction of exactly equal elements) for quantized tensors."""
    d = np.abs(a.astype(np.int32) - b.astype(np.int32))
    return int(d.max()) if d.size else 0, float((d == 0).mean()) if d.size else 1.0
