"""ctypes access to the CPU checker libraries -- TEST INFRASTRUCTURE ONLY.

Two libraries expose the same calls:
  * ``Oracle("port")``       oracle/libcpuref_oracle.so            the C restatement (prefix ``orc_``)
  * ``Oracle("reference")``  oracle/_ref/libarmnn_cpuref_hotpath.so  the reference's own sources (prefix ``ref_``)

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from typing import Optional

import numpy as np

from armnn_amd.tensor import DataType, QTensor, TensorInfo, numpy_dtype

_HERE = os.path.dirname(os.path.abspath(__file__))
PORT_LIB = os.path.join(_HERE, "libcpuref_oracle.so")
REF_LIB = os.path.join(_HERE, "_ref", "libarmnn_cpuref_hotpath.so")

ACT_NONE, ACT_RELU, ACT_BOUNDED_RELU = 0, 1, 2
POOL_MAX, POOL_AVERAGE = 0, 1
PAD_IGNORE_VALUE, PAD_EXCLUDE = 0, 1
NHWC, NCHW = 0, 1


class _Tensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int32), ("ndim", C.c_uint32), ("shape", C.c_uint32 * 6),
                ("scales", C.POINTER(C.c_float)), ("n_scales", C.c_uint32), ("quant_dim", C.c_int32),
                ("offset", C.c_int32)]


class _ConvParams(C.Structure):
    _fields_ = [("pad_top", C.c_uint32), ("pad_left", C.c_uint32), ("stride_x", C.c_uint32),
                ("stride_y", C.c_uint32), ("dilation_x", C.c_uint32), ("dilation_y", C.c_uint32),
                ("bias_enabled", C.c_int32), ("data_layout", C.c_int32), ("depthwise", C.c_int32)]


class _PoolParams(C.Structure):
    _fields_ = [("pool_type", C.c_int32), ("padding_method", C.c_int32), ("pad_left", C.c_uint32),
                ("pad_right", C.c_uint32), ("pad_top", C.c_uint32), ("pad_bottom", C.c_uint32),
                ("pool_w", C.c_uint32), ("pool_h", C.c_uint32), ("stride_x", C.c_uint32), ("stride_y", C.c_uint32)]


def build(reference: bool = True, quiet: bool = True) -> None:
    """Compile the checker libraries (the reference one only where the reference tree is mounted)."""
    out = subprocess.DEVNULL if quiet else None
    subprocess.run(["make", "-C", _HERE, "all"], check=True, stdout=out)
    if reference and os.path.isdir("/root/reference/src/backends/reference"):
        subprocess.run(["make", "-C", _HERE, "_ref"], check=True, stdout=out)


def have(kind: str) -> bool:
    return os.path.exists(PORT_LIB if kind == "port" else REF_LIB)


class Oracle:
    def __init__(self, kind: str = "port"):
        assert kind in ("port", "reference")
        self.kind = kind
        path = PORT_LIB if kind == "port" else REF_LIB
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} is not built (make -C oracle {'all' if kind == 'port' else '_ref'})")
        self.lib = C.CDLL(path)
        self.p = "orc_" if kind == "port" else "ref_"
        f = self._fn
        f("dequantize_s8", C.c_float, [C.c_int8, C.c_float, C.c_int32])
        f("dequantize_u8", C.c_float, [C.c_uint8, C.c_float, C.c_int32])
        f("dequantize_s32", C.c_float, [C.c_int32, C.c_float, C.c_int32])
        f("quantize_s8", C.c_int8, [C.c_float, C.c_float, C.c_int32])
        f("quantize_u8", C.c_uint8, [C.c_float, C.c_float, C.c_int32])
        TP = C.POINTER(_Tensor)
        f("decode_tensor", C.c_int, [TP, C.c_int, C.c_void_p])
        f("conv2d", C.c_int, [TP, TP, TP, TP, C.POINTER(_ConvParams), C.c_int])
        f("fully_connected", C.c_int, [TP, TP, TP, TP, C.c_int, C.c_int, C.c_int])
        f("activation", C.c_int, [TP, TP, C.c_int, C.c_float, C.c_float])
        f("pooling2d", C.c_int, [TP, TP, C.POINTER(_PoolParams), C.c_int])
        f("softmax", C.c_int, [TP, TP, C.c_float, C.c_int])
        f("add", C.c_int, [TP, TP, TP])
        f("pad", C.c_int, [TP, TP, C.POINTER(C.c_uint32), C.c_float])
        if kind == "reference":
            f("mean", C.c_int, [TP, TP, C.POINTER(C.c_uint32), C.c_uint32])
        f("last_error", C.c_char_p, [])

    def _fn(self, name, restype, argtypes):
        fn = getattr(self.lib, self.p + name)
        fn.restype, fn.argtypes = restype, argtypes
        setattr(self, "_" + name, fn)

    # ---- helpers -------------------------------------------------------------------------------
    @staticmethod
    def _t(t: QTensor, keep: list) -> _Tensor:
        info = t.info
        if len(info.shape) > 6:
            raise ValueError("rank > 6")
        sc = np.ascontiguousarray(info.scales_f32())
        keep.append(sc)
        keep.append(t.data)
        s = _Tensor()
        s.data = t.data.ctypes.data
        s.dtype = int(info.dtype)
        s.ndim = len(info.shape)
        for i, d in enumerate(info.shape):
            s.shape[i] = d
        s.scales = sc.ctypes.data_as(C.POINTER(C.c_float))
        s.n_scales = sc.size
        s.quant_dim = -1 if info.quant_dim is None else int(info.quant_dim)
        s.offset = int(info.offset)
        return s

    def _check(self, rc):
        if rc != 0:
            raise RuntimeError(f"{self.kind} oracle: {self._last_error().decode()}")

    # ---- scalar ----------------------------------------------------------------------------------
    def quantize(self, value: float, scale: float, offset: int, dtype: DataType) -> int:
        fn = self._quantize_u8 if DataType(dtype) == DataType.QAsymmU8 else self._quantize_s8
        return int(fn(float(np.float32(value)), float(np.float32(scale)), int(offset)))

    def dequantize(self, value: int, scale: float, offset: int, dtype: DataType) -> float:
        dt = DataType(dtype)
        fn = {DataType.QAsymmU8: self._dequantize_u8, DataType.Signed32: self._dequantize_s32}.get(dt, self._dequantize_s8)
        return float(fn(int(value), float(np.float32(scale)), int(offset)))

    # ---- tensors ---------------------------------------------------------------------------------
    def decode(self, t: QTensor, is_depthwise: bool = False) -> np.ndarray:
        keep = []
        st = self._t(t, keep)
        out = np.empty(t.info.num_elements, dtype=np.float32)
        self._check(self._decode_tensor(C.byref(st), int(is_depthwise), out.ctypes.data))
        return out.reshape(t.info.shape)

    def conv2d(self, x: QTensor, w: QTensor, b: Optional[QTensor], out_info: TensorInfo, *, pad_top=0, pad_left=0,
               stride_x=1, stride_y=1, dilation_x=1, dilation_y=1, depthwise=False, data_layout=NHWC,
               fast=True) -> QTensor:
        y = QTensor(out_info)
        keep = []
        p = _ConvParams(pad_top, pad_left, stride_x, stride_y, dilation_x, dilation_y, int(b is not None),
                        data_layout, int(depthwise))
        sx, sw, sy = self._t(x, keep), self._t(w, keep), self._t(y, keep)
        sb = self._t(b, keep) if b is not None else None
        use_fast = int(fast and data_layout == NHWC)
        self._check(self._conv2d(C.byref(sx), C.byref(sw), C.byref(sb) if sb is not None else None,
                                 C.byref(sy), C.byref(p), use_fast))
        return y

    def fully_connected(self, x: QTensor, w: QTensor, b: Optional[QTensor], out_info: TensorInfo, *,
                        transpose_weights=True, fast=True) -> QTensor:
        y = QTensor(out_info)
        keep = []
        sx, sw, sy = self._t(x, keep), self._t(w, keep), self._t(y, keep)
        sb = self._t(b, keep) if b is not None else None
        self._check(self._fully_connected(C.byref(sx), C.byref(sw), C.byref(sb) if sb is not None else None,
                                          C.byref(sy), int(b is not None), int(transpose_weights), int(fast)))
        return y

    def activation(self, x: QTensor, out_info: TensorInfo, function: int, a: float = 0.0, b: float = 0.0) -> QTensor:
        y = QTensor(out_info)
        keep = []
        sx, sy = self._t(x, keep), self._t(y, keep)
        self._check(self._activation(C.byref(sx), C.byref(sy), int(function), float(a), float(b)))
        return y

    def pooling2d(self, x: QTensor, out_info: TensorInfo, *, pool_type, pool_w, pool_h, stride_x, stride_y,
                  pad_left=0, pad_right=0, pad_top=0, pad_bottom=0, padding_method=PAD_EXCLUDE,
                  data_layout=NHWC) -> QTensor:
        y = QTensor(out_info)
        keep = []
        p = _PoolParams(pool_type, padding_method, pad_left, pad_right, pad_top, pad_bottom, pool_w, pool_h,
                        stride_x, stride_y)
        sx, sy = self._t(x, keep), self._t(y, keep)
        self._check(self._pooling2d(C.byref(sx), C.byref(sy), C.byref(p), data_layout))
        return y

    def softmax(self, x: QTensor, out_info: TensorInfo, beta: float = 1.0, axis: int = -1) -> QTensor:
        y = QTensor(out_info)
        keep = []
        sx, sy = self._t(x, keep), self._t(y, keep)
        self._check(self._softmax(C.byref(sx), C.byref(sy), float(beta), int(axis)))
        return y

    def pad(self, x: QTensor, out_info: TensorInfo, pad_before, pad_value: float = 0.0) -> QTensor:
        """Constant padding; what is added behind each dimension follows from out_info.shape."""
        y = QTensor(out_info)
        keep = []
        sx, sy = self._t(x, keep), self._t(y, keep)
        before = (C.c_uint32 * len(pad_before))(*[int(v) for v in pad_before])
        self._check(self._pad(C.byref(sx), C.byref(sy), before, float(pad_value)))
        return y

    def mean(self, x: QTensor, out_info: TensorInfo, axes) -> QTensor:
        """Mean over `axes` as the reference's Reduce computes it (reference build only; the restatement expresses the
        spatial mean of an NHWC tensor as a global average pooling, which tests show to be the same bytes)."""
        y = QTensor(out_info)
        keep = []
        sx, sy = self._t(x, keep), self._t(y, keep)
        ax = (C.c_uint32 * len(axes))(*[int(a) for a in axes])
        self._check(self._mean(C.byref(sx), C.byref(sy), ax, len(axes)))
        return y

    def add(self, a: QTensor, b: QTensor, out_info: TensorInfo) -> QTensor:
        y = QTensor(out_info)
        keep = []
        sa, sb, sy = self._t(a, keep), self._t(b, keep), self._t(y, keep)
        self._check(self._add(C.byref(sa), C.byref(sb), C.byref(sy)))
        return y
