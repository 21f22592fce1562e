"""Global pooling -> FullyConnected -> Softmax as one launch (mi355x_tail_*): the same bytes as mi355x_pool2d_run,
mi355x_fc_run and mi355x_softmax_run one behind the other (which the layer tests hold to the CPU checker), launch after
launch on one object, inside replayed graphs, and in lanes."""
import ctypes as C

import numpy as np
import pytest

from armnn_amd import nets, shim, synth
from armnn_amd.executor import DeviceNetwork
from armnn_amd.tensor import DataType, QTensor, TensorInfo
from oracle import cpuref
from tests.cases import make_fc_case
from tests.helpers import lsb_diff

pytestmark = pytest.mark.gpu

S8, U8 = DataType.QAsymmS8, DataType.QAsymmU8


class _Tail:
    """the three layers of a classifier's tail over `batch` images of hw x hw x chans, on the device"""

    def __init__(self, seed, batch, hw, chans, classes, dtype=S8, pool_type=cpuref.POOL_AVERAGE, w_dtype=DataType.QSymmS8, per_axis=True):
        lo, hi = (0, 255) if dtype == U8 else (-128, 127)
        self.batch, self.chans, self.classes = batch, chans, classes
        self.x = QTensor(TensorInfo((batch, hw, hw, chans), dtype, (0.0235,), lo + 3), synth.uniform_int(seed, (batch, hw, hw, chans), lo, lo + 140, np.int64))
        self.pool_info = TensorInfo((batch, 1, 1, chans), dtype, (0.0235,), lo + 3)
        self.pool_kw = dict(pool_type=pool_type, pool_w=hw, pool_h=hw, stride_x=1, stride_y=1, padding_method=cpuref.PAD_EXCLUDE)
        case = make_fc_case("tail", seed + 10, m=batch, k=chans, o=classes, in_dtype=dtype, in_scale=0.0235, in_offset=lo + 3,
                            w_dtype=w_dtype, per_axis=per_axis, w_offset=0 if w_dtype == DataType.QSymmS8 else 131, out_offset=lo + 70)
        self.case = case
        self.out_info = TensorInfo((batch, classes), dtype, (1.0 / 256,), lo)
        self.desc = shim.Pool2dDesc(hw, hw, chans, 1, 1, hw, hw, 1, 1, 0, 0, 0, 0, pool_type, cpuref.PAD_EXCLUDE,
                                    shim._quant(self.x.info), shim._quant(self.pool_info))
        shim.Device()
        self.lib = shim.load_library()
        self.fc = shim.FullyConnectedPlan(TensorInfo((batch, chans), dtype, (0.0235,), lo + 3), case.w, case.b, case.out_info,
                                          transpose_weights=case.transpose_weights)
        self.xd = shim.DeviceBuffer(self.x.data.nbytes).upload(self.x.data)
        self.bufs = [[shim.DeviceBuffer(batch * chans), shim.DeviceBuffer(batch * classes), shim.DeviceBuffer(batch * classes)] for _ in range(2)]

    def three_calls(self, batch=None):
        b = batch or self.batch
        pooled, logits, out = self.bufs[0]
        qi, qo = shim._quant(self.case.out_info), shim._quant(self.out_info)
        shim._chk(self.lib.mi355x_pool2d_run(C.byref(self.desc), b, self.xd.ptr, pooled.ptr, None))
        self.fc.run(b, pooled.ptr, logits.ptr)
        shim._chk(self.lib.mi355x_softmax_run(b, self.classes, 1.0, C.byref(qi), C.byref(qo), logits.ptr, out.ptr, None))
        return self._download(0, b)

    def _download(self, which, b):
        pooled, logits, out = self.bufs[which]
        return (pooled.download((self.batch, self.chans), np.uint8)[:b], logits.download((self.batch, self.classes), np.uint8)[:b],
                out.download((self.batch, self.classes), np.uint8)[:b])

    def tail(self):
        return shim.ClassifierTail(self.desc, self.fc, 1.0, self.out_info)

    def one_launch(self, tail, batch=None):
        b = batch or self.batch
        pooled, logits, out = self.bufs[1]
        for buf in self.bufs[1]:
            shim._chk(self.lib.mi355x_fill_u8(buf.ptr, 0x5a, buf.nbytes, None))
        tail.run(b, self.xd.ptr, pooled.ptr, logits.ptr, out.ptr)
        shim.Device().synchronize()
        return self._download(1, b)


TAILS = [
    # (name, batch, hw, channels, classes, dtype, pool type)
    ("mobilenet_b64", 64, 7, 1024, 1001, S8, cpuref.POOL_AVERAGE),
    ("resnet_lane_b16", 16, 7, 2048, 1001, S8, cpuref.POOL_AVERAGE),
    ("one_image_u8", 1, 7, 1024, 1001, U8, cpuref.POOL_AVERAGE),
    ("two_row_tiles_b33", 33, 7, 1280, 1000, S8, cpuref.POOL_AVERAGE),
    ("small_everything", 5, 3, 256, 37, U8, cpuref.POOL_MAX),
    ("wide_rows_196_taps", 3, 14, 128, 1500, S8, cpuref.POOL_AVERAGE),
    ("many_rows_b300", 300, 2, 512, 64, S8, cpuref.POOL_AVERAGE),
    ("partial_channel_group", 9, 4, 272, 100, S8, cpuref.POOL_AVERAGE),
]


@pytest.mark.parametrize("cfg", TAILS, ids=[c[0] for c in TAILS])
def test_one_launch_gives_the_bytes_of_the_three_calls(cfg):
    name, batch, hw, chans, classes, dtype, ptype = cfg
    print("tail", name, flush=True)
    t = _Tail(71, batch, hw, chans, classes, dtype, ptype)
    want = t.three_calls()
    tail = t.tail()
    for launch in range(3):                      # the object's counters are back at zero after every launch
        got = t.one_launch(tail)
        assert shim.last_kernel().startswith("TailKernel")
        for g, w, what in zip(got, want, ("pooled", "logits", "softmax")):
            np.testing.assert_array_equal(g, w, err_msg=f"{name} launch {launch} {what}")
    assert tail.gave_up() == 0
    if batch > 2:                                 # a smaller run on the same object and buffers
        want = t.three_calls(batch - 2)
        got = t.one_launch(tail, batch - 2)
        for g, w in zip(got, want):
            np.testing.assert_array_equal(g, w)
    tail.destroy()


def test_one_launch_against_the_cpu_checker(port):
    t = _Tail(83, 6, 7, 1024, 1001, S8, cpuref.POOL_AVERAGE)
    pooled = port.pooling2d(t.x, t.pool_info, **t.pool_kw)
    flat = QTensor(TensorInfo((6, 1024), S8, t.pool_info.scales, t.pool_info.offset), pooled.data.reshape(6, 1024))
    logits = port.fully_connected(flat, t.case.w, t.case.b, t.case.out_info, transpose_weights=t.case.transpose_weights)
    want = port.softmax(logits, t.out_info)
    tail = t.tail()
    got = t.one_launch(tail)
    np.testing.assert_array_equal(got[0].view(np.int8).reshape(pooled.data.shape), pooled.data)
    mx, exact = lsb_diff(got[1].view(np.int8), logits.data)
    assert mx <= 1 and exact >= 0.99
    # Softmax of the device's own logits, so that a 1-LSB logit does not count against the Softmax
    mine = QTensor(t.case.out_info, got[1].view(np.int8).astype(np.int64))
    mx, exact = lsb_diff(got[2].view(np.int8), port.softmax(mine, t.out_info).data)
    assert mx <= 1 and exact >= 0.99
    del want
    tail.destroy()


def test_what_the_tail_does_not_take_is_refused():
    t = _Tail(5, 4, 7, 1024, 1001)
    d = shim.Pool2dDesc(7, 7, 1024, 3, 3, 3, 3, 2, 2, 0, 0, 0, 0, 1, 1, shim._quant(t.x.info), shim._quant(t.pool_info))
    with pytest.raises(shim.ShimError, match="whole unpadded image"):
        shim.ClassifierTail(d, t.fc, 1.0, t.out_info)
    other = TensorInfo(t.pool_info.shape, S8, (0.5,), 0)
    d = shim.Pool2dDesc(7, 7, 1024, 1, 1, 7, 7, 1, 1, 0, 0, 0, 0, 1, 1, shim._quant(t.x.info), shim._quant(other))
    with pytest.raises(shim.ShimError, match="quantization"):
        shim.ClassifierTail(d, t.fc, 1.0, t.out_info)
    d = shim.Pool2dDesc(7, 7, 512, 1, 1, 7, 7, 1, 1, 0, 0, 0, 0, 1, 1, shim._quant(t.x.info), shim._quant(t.pool_info))
    with pytest.raises(shim.ShimError, match="inputs per row"):
        shim.ClassifierTail(d, t.fc, 1.0, t.out_info)
    tail = t.tail()
    pooled, logits, out = t.bufs[1]
    with pytest.raises(shim.ShimError, match="overlap"):
        tail.run(4, t.xd.ptr, pooled.ptr, logits.ptr, logits.ptr + 8)
    with pytest.raises(shim.ShimError, match="aligned"):
        tail.run(4, t.xd.ptr, pooled.ptr + 4, logits.ptr, out.ptr)
    tail.destroy()


def test_a_wait_that_runs_out_is_reported_and_the_object_works_again():
    """The waits inside the kernel are bounded; with a limit of zero every block that has to wait gives up at once and
    leaves normally.  The report names it, clears it, and the next run with the usual limit is right."""
    t = _Tail(9, 64, 7, 1024, 1001)
    want = t.three_calls()
    tail = t.tail()
    tail.set_wait_limit(0)
    got = t.one_launch(tail)
    gave_up = tail.gave_up()
    print("gave up:", gave_up, flush=True)
    if gave_up == 0:                              # nobody had to wait: then the run is simply right
        for g, w in zip(got, want):
            np.testing.assert_array_equal(g, w)
    assert tail.gave_up() == 0                    # reported once
    tail.set_wait_limit(2_000_000)
    for _ in range(2):
        got = t.one_launch(tail)
        for g, w in zip(got, want):
            np.testing.assert_array_equal(g, w)
    assert tail.gave_up() == 0
    tail.destroy()


@pytest.mark.parametrize("which,batch,lanes", [("mobilenet", 64, 1), ("resnet", 32, 2), ("mobilenet", 8, 2), ("mobilenet", 6, 2), ("resnet", 1, 1)])
def test_networks_end_in_one_launch_and_give_the_same_bytes(which, batch, lanes):
    net = nets.mobilenet_v1() if which == "mobilenet" else nets.resnet50()
    x = nets.synthetic_input(net, batch)
    apart = DeviceNetwork(net, batch, use_graph=False, lanes=1)
    want = apart.run(x).data.copy()
    apart.close()
    dn = DeviceNetwork(net, batch, use_graph=True, lanes=lanes, fuse_tail=True)
    if (batch // lanes * 1001) % 4 == 0:
        assert [l.op for l, _ in dn.steps][-1] == "tail" and len(dn.tails) == lanes
    else:                                          # a lane's logits would not start on a dword: three launches
        assert [l.op for l, _ in dn.steps][-1] == "softmax" and not dn.tails
    for replay in range(3):
        got = dn.run(x).data
        np.testing.assert_array_equal(got, want, err_msg=f"replay {replay}")
    assert all(t.gave_up() == 0 for t in dn.tails)
    dn.close()
