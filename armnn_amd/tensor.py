"""Tensor records mirroring armnn::TensorInfo (include/armnn/Tensor.hpp:152-274) for the quantized path."""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import numpy as np


class DataType(enum.IntEnum):
    """Codes shared by the device library and the CPU checker (armnn::DataType, include/armnn/Types.hpp:48-64)."""
    QAsymmS8 = 0
    QAsymmU8 = 1
    QSymmS8 = 2
    Signed32 = 3
    Float32 = 4


_NP = {
    DataType.QAsymmS8: np.int8,
    DataType.QAsymmU8: np.uint8,
    DataType.QSymmS8: np.int8,
    DataType.Signed32: np.int32,
    DataType.Float32: np.float32,
}


def numpy_dtype(dt: DataType):
    return _NP[DataType(dt)]


@dataclass
class TensorInfo:
    """Shape + data type + quantization (per-tensor: one scale; per-axis: one scale per slice of quant_dim)."""
    shape: Tuple[int, ...]
    dtype: DataType
    scales: Tuple[float, ...] = (1.0,)
    offset: int = 0
    quant_dim: Optional[int] = None

    def __post_init__(self):
        self.shape = tuple(int(s) for s in self.shape)
        self.dtype = DataType(self.dtype)
        if np.isscalar(self.scales):
            self.scales = (float(self.scales),)
        # keep scales as exact float32 values
        self.scales = tuple(float(np.float32(s)) for s in self.scales)

    @property
    def num_elements(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n

    def has_per_axis_quantization(self) -> bool:
        return len(self.scales) > 1 or self.quant_dim is not None

    @property
    def scale(self) -> float:
        if len(self.scales) > 1:
            raise ValueError("GetQuantizationScale on a tensor with multiple scales")
        return self.scales[0] if self.scales else 1.0

    def scales_f32(self) -> np.ndarray:
        return np.asarray(self.scales, dtype=np.float32)


@dataclass
class QTensor:
    """A TensorInfo plus host data."""
    info: TensorInfo
    data: np.ndarray = field(default=None)

    def __post_init__(self):
        want = numpy_dtype(self.info.dtype)
        if self.data is None:
            self.data = np.zeros(self.info.shape, dtype=want)
        self.data = np.ascontiguousarray(self.data, dtype=want).reshape(self.info.shape)

    @classmethod
    def empty(cls, shape: Sequence[int], dtype: DataType, scale=1.0, offset=0) -> "QTensor":
        return cls(TensorInfo(tuple(shape), dtype, (scale,), offset))
