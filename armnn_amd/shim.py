"""ctypes binding of the device library's C ABI (include/armnn_mi355x.h).

Loads the prebuilt ``armnn_amd/lib/libarmnn_mi355x.so`` and fails loudly when it is missing or when a call
returns an error: there is no CPU fallback anywhere in this package.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

from .tensor import DataType, QTensor, TensorInfo, numpy_dtype

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libarmnn_mi355x.so")

ALGO_AUTO, ALGO_DIRECT, ALGO_MFMA, ALGO_DEPTHWISE, ALGO_DOT4 = 0, 1, 2, 3, 4
ACT_NONE, ACT_RELU, ACT_BOUNDED_RELU = 0, 1, 2

#: every symbol include/armnn_mi355x.h declares
EXPORTS = [
    "mi355x_last_error", "mi355x_last_kernel", "mi355x_abi_version", "mi355x_set_option", "mi355x_device_count", "mi355x_init", "mi355x_device_name",
    "mi355x_device_props", "mi355x_malloc", "mi355x_free", "mi355x_host_alloc", "mi355x_host_device_pointer", "mi355x_host_free",
    "mi355x_memcpy_h2d", "mi355x_memcpy_d2h", "mi355x_memcpy_d2d", "mi355x_memcpy_h2d_async", "mi355x_memcpy_d2h_async", "mi355x_fill_u8", "mi355x_stream_create",
    "mi355x_stream_destroy", "mi355x_stream_synchronize", "mi355x_device_synchronize", "mi355x_event_create",
    "mi355x_event_destroy", "mi355x_event_record", "mi355x_stream_wait_event", "mi355x_event_synchronize", "mi355x_event_elapsed_ms",
    "mi355x_graph_capture_begin", "mi355x_graph_capture_end", "mi355x_graph_launch", "mi355x_graph_destroy",
    "mi355x_conv2d_create", "mi355x_conv2d_run", "mi355x_conv2d_destroy", "mi355x_conv2d_algo",
    "mi355x_conv2d_fusable", "mi355x_conv2d_fusion_pays", "mi355x_conv2d_run_fused", "mi355x_conv2d_pool_fusable",
    "mi355x_conv2d_pool_fusion_pays", "mi355x_conv2d_run_pooled", "mi355x_conv2d_run_add", "mi355x_conv2d_set_concurrency",
    "mi355x_chain_accepts", "mi355x_chain_create", "mi355x_chain_run", "mi355x_chain_status", "mi355x_chain_info", "mi355x_chain_run_stamped", "mi355x_chain_run_noalloc", "mi355x_chain_destroy",
    "mi355x_fc_create", "mi355x_fc_run", "mi355x_fc_destroy", "mi355x_fc_algo",
    "mi355x_activation_run", "mi355x_pool2d_run", "mi355x_add_run", "mi355x_softmax_run", "mi355x_pad_run",
    "mi355x_tail_create", "mi355x_tail_run", "mi355x_tail_status", "mi355x_tail_set_wait_limit", "mi355x_tail_destroy",
]


class Quant(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("scale", C.c_float), ("offset", C.c_int32)]


class ConstQuant(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("offset", C.c_int32), ("n_scales", C.c_uint32), ("scales", C.POINTER(C.c_float))]


class Conv2dDesc(C.Structure):
    _fields_ = [("in_h", C.c_uint32), ("in_w", C.c_uint32), ("in_c", C.c_uint32),
                ("out_h", C.c_uint32), ("out_w", C.c_uint32), ("out_c", C.c_uint32),
                ("kernel_h", C.c_uint32), ("kernel_w", C.c_uint32),
                ("pad_top", C.c_uint32), ("pad_left", C.c_uint32),
                ("stride_x", C.c_uint32), ("stride_y", C.c_uint32),
                ("dilation_x", C.c_uint32), ("dilation_y", C.c_uint32),
                ("depthwise", C.c_uint32), ("bias_enabled", C.c_uint32),
                ("input", Quant), ("output", Quant),
                ("activation", C.c_int32), ("activation_a", C.c_float), ("activation_b", C.c_float),
                ("algo", C.c_int32)]


class FcDesc(C.Structure):
    _fields_ = [("k", C.c_uint32), ("out_features", C.c_uint32), ("transpose_weights", C.c_uint32),
                ("bias_enabled", C.c_uint32), ("input", Quant), ("output", Quant),
                ("activation", C.c_int32), ("activation_a", C.c_float), ("activation_b", C.c_float),
                ("algo", C.c_int32)]


class Pool2dDesc(C.Structure):
    _fields_ = [("in_h", C.c_uint32), ("in_w", C.c_uint32), ("channels", C.c_uint32), ("out_h", C.c_uint32),
                ("out_w", C.c_uint32), ("pool_w", C.c_uint32), ("pool_h", C.c_uint32), ("stride_x", C.c_uint32),
                ("stride_y", C.c_uint32), ("pad_left", C.c_uint32), ("pad_right", C.c_uint32),
                ("pad_top", C.c_uint32), ("pad_bottom", C.c_uint32), ("pool_type", C.c_int32),
                ("padding_method", C.c_int32), ("input", Quant), ("output", Quant)]


class PadDesc(C.Structure):
    _fields_ = [("rank", C.c_uint32), ("in_shape", C.c_uint32 * 4), ("pad_before", C.c_uint32 * 4),
                ("pad_after", C.c_uint32 * 4), ("pad_value", C.c_float), ("input", Quant), ("output", Quant)]


class ShimError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"mi355x error {code}: {msg}")
        self.code = code


_lib = None


def load_library(path: str = LIB_PATH) -> C.CDLL:
    """dlopen the device library (no GPU needed for loading)."""
    global _lib
    if _lib is None:
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} not found: build it with `make -C armnn_amd/csrc` "
                                    f"(or __graft_entry__.build()); there is no fallback path")
        _lib = C.CDLL(path)
        _lib.mi355x_last_error.restype = C.c_char_p
        _lib.mi355x_last_kernel.restype = C.c_char_p
        V = C.c_void_p
        sig = {
            "mi355x_malloc": [C.POINTER(V), C.c_size_t], "mi355x_free": [V],
            "mi355x_host_alloc": [C.POINTER(V), C.c_size_t], "mi355x_host_free": [V],
            "mi355x_host_device_pointer": [V, C.POINTER(V), C.POINTER(C.c_int)],
            "mi355x_memcpy_h2d": [V, V, C.c_size_t, V], "mi355x_memcpy_d2h": [V, V, C.c_size_t, V],
            "mi355x_memcpy_d2d": [V, V, C.c_size_t, V], "mi355x_memcpy_h2d_async": [V, V, C.c_size_t, V],
            "mi355x_memcpy_d2h_async": [V, V, C.c_size_t, V], "mi355x_fill_u8": [V, C.c_uint8, C.c_size_t, V],
            "mi355x_stream_create": [C.POINTER(V)], "mi355x_stream_destroy": [V], "mi355x_stream_synchronize": [V],
            "mi355x_event_create": [C.POINTER(V)], "mi355x_event_destroy": [V], "mi355x_event_record": [V, V],
            "mi355x_stream_wait_event": [V, V],
            "mi355x_event_synchronize": [V], "mi355x_event_elapsed_ms": [V, V, C.POINTER(C.c_float)],
            "mi355x_graph_capture_begin": [V], "mi355x_graph_capture_end": [V, C.POINTER(V)],
            "mi355x_graph_launch": [V, V], "mi355x_graph_destroy": [V],
            "mi355x_conv2d_create": [C.POINTER(Conv2dDesc), V, C.POINTER(ConstQuant), V, C.POINTER(ConstQuant), C.POINTER(V)],
            "mi355x_conv2d_run": [V, C.c_uint32, V, V, V], "mi355x_conv2d_destroy": [V],
            "mi355x_conv2d_algo": [V, C.POINTER(C.c_int32), C.c_char_p, C.c_size_t],
            "mi355x_conv2d_fusable": [V, V], "mi355x_conv2d_fusion_pays": [V, V, C.c_uint32], "mi355x_conv2d_run_fused": [V, V, C.c_uint32, V, V, V],
            "mi355x_conv2d_run_add": [V, C.c_uint32, V, V, C.POINTER(Quant), C.POINTER(Quant), C.c_int32, C.c_float, C.c_float, V, V],
            "mi355x_conv2d_set_concurrency": [V, C.c_uint32],
            "mi355x_chain_accepts": [V, C.c_uint32],
            "mi355x_chain_create": [C.c_uint32, C.POINTER(V), C.c_uint32, V, C.POINTER(V), C.POINTER(V)],
            "mi355x_chain_run": [V, V], "mi355x_chain_status": [V, C.POINTER(C.c_uint32)],
            "mi355x_chain_info": [V, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)], "mi355x_chain_destroy": [V],
            "mi355x_chain_run_stamped": [V, V, C.POINTER(C.c_uint64)],
            "mi355x_chain_run_noalloc": [C.c_uint32, C.POINTER(V), C.c_uint32, V, C.POINTER(V), V],
            "mi355x_fc_create": [C.POINTER(FcDesc), V, C.POINTER(ConstQuant), V, C.POINTER(ConstQuant), C.POINTER(V)],
            "mi355x_fc_run": [V, C.c_uint32, V, V, V], "mi355x_fc_destroy": [V],
            "mi355x_fc_algo": [V, C.POINTER(C.c_int32), C.c_char_p, C.c_size_t],
            "mi355x_activation_run": [C.c_size_t, C.POINTER(Quant), C.POINTER(Quant), C.c_int32, C.c_float, C.c_float, V, V, V],
            "mi355x_pool2d_run": [C.POINTER(Pool2dDesc), C.c_uint32, V, V, V],
            "mi355x_conv2d_pool_fusable": [V, C.POINTER(Pool2dDesc)], "mi355x_conv2d_pool_fusion_pays": [V, C.POINTER(Pool2dDesc), C.c_uint32],
            "mi355x_conv2d_run_pooled": [V, C.POINTER(Pool2dDesc), C.c_uint32, V, V, V],
            "mi355x_add_run": [C.c_size_t, C.POINTER(Quant), C.POINTER(Quant), C.POINTER(Quant), C.c_int32, C.c_float,
                               C.c_float, V, V, V, V],
            "mi355x_softmax_run": [C.c_uint32, C.c_uint32, C.c_float, C.POINTER(Quant), C.POINTER(Quant), V, V, V],
            "mi355x_pad_run": [C.POINTER(PadDesc), V, V, V],
            "mi355x_tail_create": [C.POINTER(Pool2dDesc), V, C.c_float, C.POINTER(Quant), C.POINTER(V)],
            "mi355x_tail_run": [V, C.c_uint32, V, V, V, V, V], "mi355x_tail_status": [V, C.POINTER(C.c_uint32)],
            "mi355x_tail_set_wait_limit": [V, C.c_uint64], "mi355x_tail_destroy": [V],
            "mi355x_device_count": [C.POINTER(C.c_int)], "mi355x_init": [C.c_int],
            "mi355x_set_option": [C.c_char_p, C.c_int],
            "mi355x_device_name": [C.c_char_p, C.c_size_t],
            "mi355x_device_props": [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
        }
        for name, args in sig.items():
            fn = getattr(_lib, name)
            fn.argtypes = args
            fn.restype = C.c_int
    return _lib


def _chk(rc):
    if rc != 0:
        raise ShimError(rc, load_library().mi355x_last_error().decode(errors="replace"))


def _quant(info: TensorInfo) -> Quant:
    return Quant(int(info.dtype), float(np.float32(info.scale)), int(info.offset))


def last_kernel() -> str:
    """Name of the device kernel the calling thread's last launch through the library used (mi355x_last_kernel)."""
    return (load_library().mi355x_last_kernel() or b"").decode()


def set_option(name: str, value: int):
    _chk(load_library().mi355x_set_option(name.encode(), int(value)))


class DeviceBuffer:
    """Device memory from mi355x_malloc."""

    def __init__(self, nbytes: int):
        self.lib = load_library()
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        _chk(self.lib.mi355x_malloc(C.byref(p), max(self.nbytes, 1)))
        self.ptr = p.value

    def upload(self, arr: np.ndarray, stream=None):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        _chk(self.lib.mi355x_memcpy_h2d(self.ptr, arr.ctypes.data, arr.nbytes, stream))
        return self

    def download(self, shape, dtype, stream=None) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        _chk(self.lib.mi355x_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes, stream))
        return out

    def free(self):
        if self.ptr:
            _chk(self.lib.mi355x_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Device:
    """Process-wide device context."""

    _inited = False

    def __init__(self, index: int = 0):
        self.lib = load_library()
        if not Device._inited:
            _chk(self.lib.mi355x_init(index))
            Device._inited = True

    @staticmethod
    def count() -> int:
        n = C.c_int(0)
        _chk(load_library().mi355x_device_count(C.byref(n)))
        return n.value

    def name(self) -> str:
        buf = C.create_string_buffer(128)
        _chk(self.lib.mi355x_device_name(buf, 128))
        return buf.value.decode()

    def props(self):
        cu, clk, mem, lds = C.c_int(), C.c_int(), C.c_size_t(), C.c_size_t()
        _chk(self.lib.mi355x_device_props(C.byref(cu), C.byref(clk), C.byref(mem), C.byref(lds)))
        return {"compute_units": cu.value, "clock_khz": clk.value, "total_mem": mem.value, "lds_per_cu": lds.value}

    def synchronize(self):
        _chk(self.lib.mi355x_device_synchronize())

    def stream(self):
        s = C.c_void_p()
        _chk(self.lib.mi355x_stream_create(C.byref(s)))
        return s.value

    def stream_sync(self, s):
        _chk(self.lib.mi355x_stream_synchronize(s))

    def stream_destroy(self, s):
        _chk(self.lib.mi355x_stream_destroy(s))

    def event(self):
        e = C.c_void_p()
        _chk(self.lib.mi355x_event_create(C.byref(e)))
        return e.value

    def event_record(self, e, stream=None):
        _chk(self.lib.mi355x_event_record(e, stream))

    def stream_wait_event(self, stream, e):
        _chk(self.lib.mi355x_stream_wait_event(stream, e))

    def event_sync(self, e):
        _chk(self.lib.mi355x_event_synchronize(e))

    def elapsed_ms(self, e0, e1) -> float:
        ms = C.c_float()
        _chk(self.lib.mi355x_event_elapsed_ms(e0, e1, C.byref(ms)))
        return ms.value

    def graph_begin(self, stream):
        _chk(self.lib.mi355x_graph_capture_begin(stream))

    def graph_end(self, stream):
        g = C.c_void_p()
        _chk(self.lib.mi355x_graph_capture_end(stream, C.byref(g)))
        return g.value

    def graph_launch(self, g, stream):
        _chk(self.lib.mi355x_graph_launch(g, stream))

    def graph_destroy(self, g):
        _chk(self.lib.mi355x_graph_destroy(g))


def _const_quant(info: TensorInfo, keep: list) -> ConstQuant:
    sc = np.ascontiguousarray(info.scales_f32())
    keep.append(sc)
    return ConstQuant(int(info.dtype), int(info.offset), sc.size, sc.ctypes.data_as(C.POINTER(C.c_float)))


class Conv2dPlan:
    """mi355x_conv2d_create / run / destroy.  Argument names follow armnn::Convolution2dDescriptor."""

    def __init__(self, in_info: TensorInfo, w: QTensor, b: Optional[QTensor], out_info: TensorInfo, *, pad_top=0,
                 pad_left=0, stride_x=1, stride_y=1, dilation_x=1, dilation_y=1, depthwise=False, activation=ACT_NONE,
                 act_a=0.0, act_b=0.0, algo=ALGO_AUTO):
        self.lib = load_library()
        self.in_info, self.out_info = in_info, out_info
        _, h, wd, ci = in_info.shape
        _, ho, wo, co = out_info.shape
        kh, kw = w.info.shape[1], w.info.shape[2]
        d = Conv2dDesc(h, wd, ci, ho, wo, co, kh, kw, pad_top, pad_left, stride_x, stride_y, dilation_x, dilation_y,
                       int(depthwise), int(b is not None), _quant(in_info), _quant(out_info), activation, act_a, act_b, algo)
        keep = []
        wq = _const_quant(w.info, keep)
        bq = _const_quant(b.info, keep) if b is not None else None
        plan = C.c_void_p()
        _chk(self.lib.mi355x_conv2d_create(C.byref(d), w.data.ctypes.data, C.byref(wq),
                                           b.data.ctypes.data if b is not None else None,
                                           C.byref(bq) if bq is not None else None, C.byref(plan)))
        self.plan = plan.value

    def algo(self):
        a = C.c_int32()
        buf = C.create_string_buffer(128)
        _chk(self.lib.mi355x_conv2d_algo(self.plan, C.byref(a), buf, 128))
        return a.value, buf.value.decode()

    def run(self, batch: int, x_dev: int, y_dev: int, stream=None):
        _chk(self.lib.mi355x_conv2d_run(self.plan, batch, x_dev, y_dev, stream))

    def fusable_with(self, second: "Conv2dPlan") -> bool:
        """True when this plan and `second`, the layer consuming its output, can run as one kernel: 3x3 depthwise + 1x1
        convolution, or 1x1 convolution + 3x3 depthwise over images of at most 224 pixels."""
        return self.lib.mi355x_conv2d_fusable(self.plan, second.plan) == 0

    def fusion_pays(self, second: "Conv2dPlan", batch: int) -> bool:
        """True when the library recommends running this plan and `second` as one launch at this batch."""
        return self.lib.mi355x_conv2d_fusion_pays(self.plan, second.plan, batch) == 1

    def run_fused(self, second: "Conv2dPlan", batch: int, x_dev: int, y_dev: int, stream=None):
        """Both layers without the intermediate tensor; bytes equal run() + second.run()."""
        _chk(self.lib.mi355x_conv2d_run_fused(self.plan, second.plan, batch, x_dev, y_dev, stream))

    def pool_fusable(self, pool: "Pool2dDesc") -> bool:
        """True when this plan (an unpadded 1x1 convolution) and the pooling over its whole output image can run as one kernel."""
        return self.lib.mi355x_conv2d_pool_fusable(self.plan, C.byref(pool)) == 0

    def pool_fusion_pays(self, pool: "Pool2dDesc", batch: int) -> bool:
        """True when the library recommends that one launch at this batch."""
        return self.lib.mi355x_conv2d_pool_fusion_pays(self.plan, C.byref(pool), batch) == 1

    def run_pooled(self, pool: "Pool2dDesc", batch: int, x_dev: int, y_dev: int, stream=None):
        """The convolution and the pooling behind it; only the pooled tensor [batch][channels] is written, with the bytes
        of run() followed by mi355x_pool2d_run."""
        _chk(self.lib.mi355x_conv2d_run_pooled(self.plan, C.byref(pool), batch, x_dev, y_dev, stream))

    def set_concurrency(self, lanes: int):
        """Tell the plan that `lanes` launches of its network run side by side (kernels with small blocks are preferred then)."""
        _chk(self.lib.mi355x_conv2d_set_concurrency(self.plan, int(lanes)))

    def run_add(self, batch: int, x_dev: int, other_dev: int, other_info: TensorInfo, sum_info: TensorInfo, y_dev: int,
                activation=ACT_NONE, act_a=0.0, act_b=0.0, stream=None):
        """This convolution and the Addition consuming it in one launch where the kernel can; bytes equal run() followed
        by the Addition (the other input in `other_dev`, the sum quantized as `sum_info`, then the activation)."""
        qo, qs = _quant(other_info), _quant(sum_info)
        _chk(self.lib.mi355x_conv2d_run_add(self.plan, batch, x_dev, other_dev, C.byref(qo), C.byref(qs), activation, act_a, act_b,
                                            y_dev, stream))

    def destroy(self):
        if self.plan:
            self.lib.mi355x_conv2d_destroy(self.plan)
            self.plan = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class LayerChain:
    """mi355x_chain_*: consecutive convolution plans (plans[k] reads plans[k - 1]'s output) as one persistent launch.
    Addresses are bound here; the bytes written to every output equal those of running the plans one by one."""

    def __init__(self, plans: Sequence["Conv2dPlan"], batch: int, x_dev: int, outputs_dev: Sequence[int]):
        self.lib = load_library()
        self.plans = list(plans)                  # the chain refers to them: keep them alive
        n = len(self.plans)
        pa = (C.c_void_p * n)(*[p.plan for p in self.plans])
        oa = (C.c_void_p * n)(*outputs_dev)
        chain = C.c_void_p()
        _chk(self.lib.mi355x_chain_create(n, pa, batch, x_dev, oa, C.byref(chain)))
        self.chain = chain.value

    @staticmethod
    def run_noalloc(plans: Sequence["Conv2dPlan"], batch: int, x_dev: int, outputs_dev: Sequence[int], stream=None):
        """mi355x_chain_run_noalloc: the same run without a chain object and without any device allocation (at most 32
        layers and 64 images); calls on one GPU share one device array and must not overlap."""
        n = len(plans)
        pa = (C.c_void_p * n)(*[p.plan for p in plans])
        oa = (C.c_void_p * n)(*outputs_dev)
        _chk(load_library().mi355x_chain_run_noalloc(n, pa, batch, x_dev, oa, stream))

    @staticmethod
    def accepts(plan: "Conv2dPlan", batch: int) -> bool:
        return load_library().mi355x_chain_accepts(plan.plan, batch) == 0

    def run(self, stream=None):
        _chk(self.lib.mi355x_chain_run(self.chain, stream))

    def gave_up(self) -> int:
        """Blocks whose bounded wait ran out in a launch since the last call (0 in normal operation); call after synchronizing."""
        n = C.c_uint32()
        _chk(self.lib.mi355x_chain_status(self.chain, C.byref(n)))
        return n.value

    def run_stamped(self, stream=None):
        """One launch with per-phase cycle sums over all blocks: dict of cycles per phase and tile counts."""
        sums = (C.c_uint64 * 8)()
        _chk(self.lib.mi355x_chain_run_stamped(self.chain, stream, sums))
        names = ("pop", "wait", "mfma_tiles", "dw_tiles", "drain", "n_mfma_tiles", "n_dw_tiles", "n_waited")
        return dict(zip(names, [int(v) for v in sums]))

    def info(self):
        items, blocks = C.c_uint32(), C.c_uint32()
        _chk(self.lib.mi355x_chain_info(self.chain, C.byref(items), C.byref(blocks)))
        return items.value, blocks.value

    def destroy(self):
        if self.chain:
            self.lib.mi355x_chain_destroy(self.chain)
            self.chain = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class FullyConnectedPlan:
    """mi355x_fc_create / run / destroy.  Argument names follow armnn::FullyConnectedDescriptor."""

    def __init__(self, in_info: TensorInfo, w: QTensor, b: Optional[QTensor], out_info: TensorInfo, *,
                 transpose_weights=True, activation=ACT_NONE, act_a=0.0, act_b=0.0, algo=ALGO_AUTO):
        self.lib = load_library()
        k = 1
        for s in in_info.shape[1:]:
            k *= s
        o = out_info.shape[1]
        d = FcDesc(k, o, int(transpose_weights), int(b is not None), _quant(in_info), _quant(out_info), activation,
                   act_a, act_b, algo)
        keep = []
        wq = _const_quant(w.info, keep)
        bq = _const_quant(b.info, keep) if b is not None else None
        plan = C.c_void_p()
        _chk(self.lib.mi355x_fc_create(C.byref(d), w.data.ctypes.data, C.byref(wq),
                                       b.data.ctypes.data if b is not None else None,
                                       C.byref(bq) if bq is not None else None, C.byref(plan)))
        self.plan = plan.value

    def algo(self):
        a = C.c_int32()
        buf = C.create_string_buffer(128)
        _chk(self.lib.mi355x_fc_algo(self.plan, C.byref(a), buf, 128))
        return a.value, buf.value.decode()

    def run(self, batch: int, x_dev: int, y_dev: int, stream=None):
        _chk(self.lib.mi355x_fc_run(self.plan, batch, x_dev, y_dev, stream))

    def destroy(self):
        if self.plan:
            self.lib.mi355x_fc_destroy(self.plan)
            self.plan = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class ClassifierTail:
    """mi355x_tail_create / run / status / destroy: global pooling -> FullyConnected -> Softmax as one launch.  Raises
    ShimError (unsupported) for what the library runs as three calls only."""

    def __init__(self, pool_desc: "Pool2dDesc", fc: FullyConnectedPlan, beta: float, out_info: TensorInfo):
        self.lib = load_library()
        self.fc = fc                      # must outlive the object
        self._desc = pool_desc
        qo = _quant(out_info)
        tail = C.c_void_p()
        _chk(self.lib.mi355x_tail_create(C.byref(pool_desc), fc.plan, beta, C.byref(qo), C.byref(tail)))
        self.tail = tail.value

    def run(self, batch: int, x_dev: int, pooled_dev: int, logits_dev: int, y_dev: int, stream=None):
        _chk(self.lib.mi355x_tail_run(self.tail, batch, x_dev, pooled_dev, logits_dev, y_dev, stream))

    def gave_up(self) -> int:
        """waits that ran out in runs since the last call (after the stream has been synchronized)"""
        n = C.c_uint32()
        _chk(self.lib.mi355x_tail_status(self.tail, C.byref(n)))
        return n.value

    def set_wait_limit(self, microseconds: int):
        _chk(self.lib.mi355x_tail_set_wait_limit(self.tail, microseconds))

    def destroy(self):
        if self.tail:
            self.lib.mi355x_tail_destroy(self.tail)
            self.tail = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


# ---- one-call helpers: upload, run, download (tests and the smoke check) -------------------------------------
def conv2d(x: QTensor, w: QTensor, b: Optional[QTensor], out_info: TensorInfo, concurrency: int = 1, **kw) -> QTensor:
    Device()
    plan = Conv2dPlan(x.info, w, b, out_info, **kw)
    if concurrency != 1:
        plan.set_concurrency(concurrency)
    xd = DeviceBuffer(x.data.nbytes).upload(x.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(y.data.nbytes)
    plan.run(x.info.shape[0], xd.ptr, yd.ptr)
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    plan.destroy()
    return y


def fully_connected(x: QTensor, w: QTensor, b: Optional[QTensor], out_info: TensorInfo, **kw) -> QTensor:
    Device()
    plan = FullyConnectedPlan(x.info, w, b, out_info, **kw)
    xd = DeviceBuffer(x.data.nbytes).upload(x.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(y.data.nbytes)
    plan.run(x.info.shape[0], xd.ptr, yd.ptr)
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    plan.destroy()
    return y


def activation(x: QTensor, out_info: TensorInfo, function: int, a=0.0, b=0.0) -> QTensor:
    Device()
    lib = load_library()
    xd = DeviceBuffer(x.data.nbytes).upload(x.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(y.data.nbytes)
    qi, qo = _quant(x.info), _quant(out_info)
    _chk(lib.mi355x_activation_run(x.info.num_elements, C.byref(qi), C.byref(qo), function, a, b, xd.ptr, yd.ptr, None))
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    return y


def pooling2d(x: QTensor, out_info: TensorInfo, *, pool_type, pool_w, pool_h, stride_x, stride_y, pad_left=0,
              pad_right=0, pad_top=0, pad_bottom=0, padding_method=1) -> QTensor:
    Device()
    lib = load_library()
    n, h, w, c = x.info.shape
    _, ho, wo, _ = out_info.shape
    d = Pool2dDesc(h, w, c, ho, wo, pool_w, pool_h, stride_x, stride_y, pad_left, pad_right, pad_top, pad_bottom,
                   pool_type, padding_method, _quant(x.info), _quant(out_info))
    xd = DeviceBuffer(x.data.nbytes).upload(x.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(y.data.nbytes)
    _chk(lib.mi355x_pool2d_run(C.byref(d), n, xd.ptr, yd.ptr, None))
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    return y


def add(a: QTensor, b: QTensor, out_info: TensorInfo, activation=ACT_NONE, act_a=0.0, act_b=0.0) -> QTensor:
    Device()
    lib = load_library()
    ad = DeviceBuffer(a.data.nbytes).upload(a.data)
    bd = DeviceBuffer(b.data.nbytes).upload(b.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(y.data.nbytes)
    q0, q1, qo = _quant(a.info), _quant(b.info), _quant(out_info)
    _chk(lib.mi355x_add_run(a.info.num_elements, C.byref(q0), C.byref(q1), C.byref(qo), activation, act_a, act_b,
                            ad.ptr, bd.ptr, yd.ptr, None))
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    return y


def softmax(x: QTensor, out_info: TensorInfo, beta=1.0) -> QTensor:
    Device()
    lib = load_library()
    rows, cols = x.info.shape
    xd = DeviceBuffer(x.data.nbytes).upload(x.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(y.data.nbytes)
    qi, qo = _quant(x.info), _quant(out_info)
    _chk(lib.mi355x_softmax_run(rows, cols, beta, C.byref(qi), C.byref(qo), xd.ptr, yd.ptr, None))
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    return y


def pad_desc(in_shape, pad_list, pad_value, in_info: TensorInfo, out_info: TensorInfo) -> PadDesc:
    """pad_list holds one (before, after) pair per dimension, as armnn::PadDescriptor::m_PadList does."""
    d = PadDesc()
    d.rank = len(in_shape)
    for k, (extent, (before, after)) in enumerate(zip(in_shape, pad_list)):
        d.in_shape[k], d.pad_before[k], d.pad_after[k] = extent, before, after
    d.pad_value = float(pad_value)
    d.input, d.output = _quant(in_info), _quant(out_info)
    return d


def pad(x: QTensor, out_info: TensorInfo, pad_list, pad_value=0.0) -> QTensor:
    Device()
    lib = load_library()
    d = pad_desc(x.info.shape, pad_list, pad_value, x.info, out_info)
    xd = DeviceBuffer(max(x.data.nbytes, 1)).upload(x.data)
    y = QTensor(out_info)
    yd = DeviceBuffer(max(y.data.nbytes, 1))
    _chk(lib.mi355x_pad_run(C.byref(d), xd.ptr, yd.ptr, None))
    y.data = yd.download(out_info.shape, numpy_dtype(out_info.dtype))
    return y
