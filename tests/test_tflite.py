"""The .tflite reader: a real quantized model from the reference's own test data (delegate/python/test/test_data/
mock_model.tflite, kept as a fixture) and small models written for the occasion (tests/tflite_writer.py)."""
import os

import numpy as np
import pytest

from armnn_amd import nets, tflite
from armnn_amd.tensor import DataType
from oracle import netref
from tests import tflite_writer as tw
from tests.helpers import GOLDEN


def pool_activation_model(seed=5):
    """MAX_POOL_2D with a fused RELU6 and AVERAGE_POOL_2D with a fused RELU: the clamps must survive on the device."""
    rng = np.random.default_rng(seed)
    b = tw.ModelBuilder()
    x = b.tensor("input", (1, 12, 12, 16), tw.INT8, 0.1, -20)
    m = b.tensor("maxpool/out", (1, 6, 6, 16), tw.INT8, 0.1, -20)
    b.op(tw.MAX_POOL_2D, [x], [m], tw.OPT_POOL, {0: ("b", tw.SAME), 1: ("i", 2), 2: ("i", 2), 3: ("i", 2), 4: ("i", 2), 5: ("b", tw.ACT_RELU6)})
    a = b.tensor("avgpool/out", (1, 3, 3, 16), tw.INT8, 0.1, -20)
    b.op(tw.AVERAGE_POOL_2D, [m], [a], tw.OPT_POOL, {0: ("b", tw.VALID), 1: ("i", 2), 2: ("i", 2), 3: ("i", 2), 4: ("i", 2), 5: ("b", tw.ACT_RELU)})
    return b.finish([x], [a])


def mock_model():
    return tflite.load(os.path.join(GOLDEN, "mock_model.tflite"))


def written_model(seed=3):
    """int8 with per-channel weights: PAD -> CONV_2D (VALID, stride 2, RELU6) -> DEPTHWISE_CONV_2D (SAME, RELU) ->
    AVERAGE_POOL_2D (SAME, stride 2) -> ADD (x + x) -> FULLY_CONNECTED (RELU_N1_TO_1) -> SOFTMAX."""
    rng = np.random.default_rng(seed)
    b = tw.ModelBuilder()
    w8 = lambda shape: np.clip(np.rint(rng.normal(0, 30, shape)), -127, 127).astype(np.int8)
    x = b.tensor("input", (1, 9, 9, 8), tw.INT8, 0.02, -5)
    pads = b.tensor("paddings", (4, 2), tw.INT32, data=np.array([[0, 0], [1, 1], [1, 1], [0, 0]], np.int32))
    padded = b.tensor("padded", (1, 11, 11, 8), tw.INT8, 0.02, -5)
    b.op(tw.PAD, [x, pads], [padded], tw.OPT_PAD, {})
    ws = rng.uniform(0.001, 0.003, 16).astype(np.float32)
    w1 = b.tensor("conv/w", (16, 3, 3, 8), tw.INT8, ws, 0, w8((16, 3, 3, 8)), quantized_dimension=0)
    b1 = b.tensor("conv/b", (16,), tw.INT32, np.float32(0.02) * ws, 0, rng.integers(-300, 300, 16).astype(np.int32))
    c1 = b.tensor("conv/out", (1, 5, 5, 16), tw.INT8, 0.0235, -128)
    b.op(tw.CONV_2D, [padded, w1, b1], [c1], tw.OPT_CONV, {0: ("b", tw.VALID), 1: ("i", 2), 2: ("i", 2), 3: ("b", tw.ACT_RELU6)})
    wd = rng.uniform(0.004, 0.01, 16).astype(np.float32)
    w2 = b.tensor("dw/w", (1, 3, 3, 16), tw.INT8, wd, 0, w8((1, 3, 3, 16)), quantized_dimension=3)
    b2 = b.tensor("dw/b", (16,), tw.INT32, np.float32(0.0235) * wd, 0, rng.integers(-100, 100, 16).astype(np.int32))
    c2 = b.tensor("dw/out", (1, 5, 5, 16), tw.INT8, 0.03, -128)
    b.op(tw.DEPTHWISE_CONV_2D, [c1, w2, b2], [c2], tw.OPT_DEPTHWISE,
         {0: ("b", tw.SAME), 1: ("i", 1), 2: ("i", 1), 3: ("i", 1), 4: ("b", tw.ACT_RELU)})
    p = b.tensor("pool/out", (1, 3, 3, 16), tw.INT8, 0.03, -128)
    b.op(tw.AVERAGE_POOL_2D, [c2], [p], tw.OPT_POOL, {0: ("b", tw.SAME), 1: ("i", 2), 2: ("i", 2), 3: ("i", 2), 4: ("i", 2)})
    s = b.tensor("sum", (1, 3, 3, 16), tw.INT8, 0.06, -128)
    b.op(tw.ADD, [p, p], [s], tw.OPT_ADD, {})
    wf = b.tensor("fc/w", (10, 144), tw.INT8, 0.004, 0, w8((10, 144)))
    bf = b.tensor("fc/b", (10,), tw.INT32, np.float32(0.06) * np.float32(0.004), 0, rng.integers(-50, 50, 10).astype(np.int32))
    f = b.tensor("fc/out", (1, 10), tw.INT8, 0.01, 0)
    b.op(tw.FULLY_CONNECTED, [s, wf, bf], [f], tw.OPT_FC, {0: ("b", tw.ACT_RELU_N1_TO_1)})
    y = b.tensor("probabilities", (1, 10), tw.INT8, 1.0 / 256.0, -128)
    b.op(tw.SOFTMAX, [f], [y], tw.OPT_SOFTMAX, {0: ("f", 2.0)})
    return b.finish([x], [y])


def test_mock_model_is_read_as_the_file_states():
    net = mock_model()
    assert [l.op for l in net.layers] == ["depthwise", "conv", "pool", "conv", "pool", "reshape", "fc", "softmax"]
    assert net.tensors[net.input].shape == (1, 28, 28, 1) and net.tensors[net.input].dtype == DataType.QAsymmU8
    dw, conv = net.layers[0], net.layers[1]
    assert dw.weights.info.shape == (1, 3, 3, 32) and dw.weights.info.dtype == DataType.QAsymmU8      # depth multiplier 32
    assert dw.weights.info.offset == 115 and conv.weights.info.offset == 125
    assert dw.params["pad_top"] == 1 and dw.params["pad_left"] == 1                                   # SAME
    assert conv.bias.info.dtype == DataType.Signed32 and conv.bias.data.shape == (32,)
    # TOCO wrote the bias scale as input scale * weight scale
    want = np.float32(net.tensors[conv.inputs[0]].scale) * np.float32(conv.weights.info.scale)
    assert abs(conv.bias.info.scale - want) <= 1e-6 * want
    pool = net.layers[2]
    assert pool.params["pool_type"] == 0 and pool.params["pool_w"] == 2 and pool.params["pad_top"] == 0   # MAX, VALID
    assert net.tensors[net.layers[5].output].shape == (1, 1568)                                       # flattened for the FC
    fc = net.layers[6]
    assert fc.weights.info.shape == (10, 1568) and fc.params["transpose_weights"]
    out = net.tensors[net.output]
    assert out.shape == (1, 10) and out.scale == 1.0 / 256.0 and out.offset == 0
    assert all(l.act == (0, 0.0, 0.0) for l in net.layers)


def test_written_model_maps_padding_strides_and_activations():
    net = tflite.parse(written_model(), "written")
    assert [l.op for l in net.layers] == ["pad", "conv", "depthwise", "pool", "add", "reshape", "fc", "softmax"]
    pad, conv, dw, pool, add, _, fc, sm = net.layers
    assert pad.params["pad_list"] == ((0, 0), (1, 1), (1, 1), (0, 0)) and pad.params["pad_value"] == -5.0
    assert conv.params["stride_x"] == 2 and conv.params["pad_top"] == 0 and conv.act == (2, 6.0, 0.0)
    assert conv.weights.info.dtype == DataType.QSymmS8 and len(conv.weights.info.scales) == 16 and conv.weights.info.quant_dim == 0
    assert dw.params["pad_top"] == 1 and dw.params["depthwise"] and dw.act == (1, 0.0, 0.0) and dw.weights.info.quant_dim == 3
    # 5 -> 3 with a 2x2 window at stride 2: one row and column of padding, behind (front = total // 2 = 0)
    assert (pool.params["pad_top"], pool.params["pad_bottom"], pool.params["pad_left"], pool.params["pad_right"]) == (0, 1, 0, 1)
    assert pool.params["pool_type"] == 1 and pool.params["padding_method"] == 1
    assert add.inputs[0] == add.inputs[1]
    assert fc.act == (2, 1.0, -1.0) and fc.weights.info.dtype == DataType.QAsymmS8      # per-tensor int8 stays asymmetric
    assert sm.params["beta"] == 2.0


def test_what_cannot_run_is_refused_by_name():
    with pytest.raises(tflite.UnsupportedModel, match="TFL3"):
        tflite.parse(b"\x10\0\0\0ABCD" + bytes(64))
    with pytest.raises(tflite.UnsupportedModel, match="3 inputs"):
        tflite.load(os.path.join(GOLDEN, "conv2d_float32.tflite"))          # the reference's float model, weights as inputs
    b = tw.ModelBuilder()
    x = b.tensor("x", (1, 4), tw.FLOAT32)
    y = b.tensor("y", (1, 4), tw.FLOAT32)
    b.op(tw.SOFTMAX, [x], [y], tw.OPT_SOFTMAX, {0: ("f", 1.0)})
    with pytest.raises(tflite.UnsupportedModel, match="TensorType 0"):
        tflite.parse(b.finish([x], [y]))
    b = tw.ModelBuilder()
    x = b.tensor("x", (1, 4), tw.UINT8, 0.1, 0)
    y = b.tensor("y", (1, 4), tw.UINT8, 0.1, 0)
    b.op(tw.TANH, [x], [y])
    with pytest.raises(tflite.UnsupportedModel, match="builtin code 28"):
        tflite.parse(b.finish([x], [y]))


@pytest.mark.parametrize("which", ["mock", "written"])
def test_port_and_reference_build_agree_on_the_models(port, reference, which):
    net = mock_model() if which == "mock" else tflite.parse(written_model(), "written")
    x = nets.synthetic_input(net, 3, seed=11)
    a = netref.run_network(port, net, x, keep=True, fast=False)
    b = netref.run_network(reference, net, x, keep=True)
    for name in a:
        np.testing.assert_array_equal(a[name].data, b[name].data, err_msg=name)
    probs = a[net.output].data.astype(np.int64) - net.tensors[net.output].offset
    assert np.all(np.abs(probs.sum(axis=-1) - 256) <= 8)                     # a distribution over the 10 classes
    assert len(np.unique(a[net.output].data)) > 2


def test_damaged_files_are_refused_not_misread():
    """Truncations and overwritten offsets end in UnsupportedModel, never in another exception or a silently wrong net."""
    data = open(os.path.join(GOLDEN, "mock_model.tflite"), "rb").read()
    good = tflite.parse(data)
    rng = np.random.default_rng(99)
    refused = 0
    for trial in range(300):
        damaged = bytearray(data)
        if trial % 3 == 0:
            damaged = damaged[:int(rng.integers(8, len(data)))]
        else:
            at = int(rng.integers(8, 2200))            # tables, vtables and offsets live at the front of this file
            damaged[at:at + 4] = rng.integers(0, 256, 4, dtype=np.uint8).tobytes()
        try:
            net = tflite.parse(bytes(damaged))
        except tflite.UnsupportedModel:
            refused += 1
            continue
        assert len(net.layers) <= len(good.layers) + 1            # still a network the reader understands
    assert refused > 50


def test_shapes_the_operator_cannot_produce_are_refused():
    """Buffers are sized from the file, kernels from the operator: a PAD whose output tensor is smaller than input plus
    padding, or a pooling output larger than the window arithmetic gives, must not reach the device."""
    b = tw.ModelBuilder()
    x = b.tensor("x", (1, 4, 4, 8), tw.UINT8, 0.1, 3)
    pads = b.tensor("paddings", (4, 2), tw.INT32, data=np.array([[0, 0], [2, 2], [2, 2], [0, 0]], np.int32))
    y = b.tensor("y", (1, 6, 6, 8), tw.UINT8, 0.1, 3)               # should be 8 x 8
    b.op(tw.PAD, [x, pads], [y], tw.OPT_PAD, {})
    with pytest.raises(tflite.UnsupportedModel, match="output shape"):
        tflite.parse(b.finish([x], [y]))
    b = tw.ModelBuilder()
    x = b.tensor("x", (1, 8, 8, 4), tw.INT8, 0.1, 0)
    y = b.tensor("y", (1, 5, 5, 4), tw.INT8, 0.1, 0)                # 2x2 stride 2 VALID gives 4 x 4
    b.op(tw.MAX_POOL_2D, [x], [y], tw.OPT_POOL, {0: ("b", tw.VALID), 1: ("i", 2), 2: ("i", 2), 3: ("i", 2), 4: ("i", 2)})
    with pytest.raises(tflite.UnsupportedModel, match="output shape"):
        tflite.parse(b.finish([x], [y]))


def mean_model(keep_dims):
    """uint8: CONV_2D 1x1 (RELU6) -> MEAN over height and width -> FULLY_CONNECTED -> SOFTMAX, the tail of a ResNet."""
    rng = np.random.default_rng(5)
    b = tw.ModelBuilder()
    x = b.tensor("input", (1, 7, 6, 16), tw.UINT8, 0.02, 120)
    w = b.tensor("conv/w", (32, 1, 1, 16), tw.UINT8, 0.01, 128, rng.integers(60, 200, (32, 1, 1, 16)).astype(np.uint8))
    bias = b.tensor("conv/b", (32,), tw.INT32, np.float32(0.02) * np.float32(0.01), 0, rng.integers(-200, 200, 32).astype(np.int32))
    c = b.tensor("conv/out", (1, 7, 6, 32), tw.UINT8, 0.0235, 0)
    b.op(tw.CONV_2D, [x, w, bias], [c], tw.OPT_CONV, {0: ("b", tw.VALID), 1: ("i", 1), 2: ("i", 1), 3: ("b", tw.ACT_RELU6)})
    axes = b.tensor("axes", (2,), tw.INT32, data=np.array([1, 2], np.int32))
    m = b.tensor("mean", (1, 1, 1, 32) if keep_dims else (1, 32), tw.UINT8, 0.02, 2)
    b.op(tw.MEAN, [c, axes], [m], tw.OPT_REDUCER, {0: ("b", 1 if keep_dims else 0)})
    wf = b.tensor("fc/w", (10, 32), tw.UINT8, 0.02, 128, rng.integers(60, 200, (10, 32)).astype(np.uint8))
    bf = b.tensor("fc/b", (10,), tw.INT32, np.float32(0.02) * np.float32(0.02), 0, rng.integers(-50, 50, 10).astype(np.int32))
    f = b.tensor("fc/out", (1, 10), tw.UINT8, 0.05, 100)
    b.op(tw.FULLY_CONNECTED, [m, wf, bf], [f], tw.OPT_FC, {0: ("b", tw.ACT_NONE)})
    y = b.tensor("probabilities", (1, 10), tw.UINT8, 1.0 / 256.0, 0)
    b.op(tw.SOFTMAX, [f], [y], tw.OPT_SOFTMAX, {0: ("f", 1.0)})
    return b.finish([x], [y])


@pytest.mark.parametrize("keep_dims", [True, False])
def test_mean_over_height_and_width_is_read_as_a_global_average_pooling(reference, port, keep_dims):
    net = tflite.parse(mean_model(keep_dims), "mean")
    ops = [l.op for l in net.layers]
    assert ops == (["conv", "pool", "reshape", "fc", "softmax"] if keep_dims else ["conv", "pool", "reshape", "fc", "softmax"])
    pool = net.layers[1]
    assert pool.params["pool_type"] == 1 and (pool.params["pool_h"], pool.params["pool_w"]) == (7, 6)
    # the pooling the reader substitutes gives the bytes of the reference's own Reduce
    x = nets.synthetic_input(net, 3, seed=4)
    vals = netref.run_network(port, net, x, keep=True)
    conv_out = vals[net.layers[0].output]
    pooled = vals[pool.output]
    want = reference.mean(conv_out, pooled.info, [1, 2])
    np.testing.assert_array_equal(pooled.data, want.data)


def test_mean_over_other_axes_is_refused():
    b = tw.ModelBuilder()
    x = b.tensor("x", (1, 4, 4, 8), tw.UINT8, 0.1, 0)
    axes = b.tensor("axes", (1,), tw.INT32, data=np.array([3], np.int32))
    y = b.tensor("y", (1, 4, 4, 1), tw.UINT8, 0.1, 0)
    b.op(tw.MEAN, [x, axes], [y], tw.OPT_REDUCER, {0: ("b", 1)})
    with pytest.raises(tflite.UnsupportedModel, match="height and width"):
        tflite.parse(b.finish([x], [y]))


def relu_model():
    """int8: standalone RELU6 that re-quantizes, RELU_N1_TO_1 and RELU that keep the quantization, then SOFTMAX."""
    b = tw.ModelBuilder()
    x = b.tensor("input", (1, 48), tw.INT8, 0.1, -10)
    a = b.tensor("relu6", (1, 48), tw.INT8, 6.0 / 255.0, -128)
    b.op(tw.RELU6, [x], [a])
    c = b.tensor("relu_n1_to_1", (1, 48), tw.INT8, 6.0 / 255.0, -128)
    b.op(tw.RELU_N1_TO_1, [a], [c])
    d = b.tensor("relu", (1, 48), tw.INT8, 0.01, -100)
    b.op(tw.RELU, [c], [d])
    y = b.tensor("probabilities", (1, 48), tw.INT8, 1.0 / 256.0, -128)
    b.op(tw.SOFTMAX, [d], [y], tw.OPT_SOFTMAX, {0: ("f", 1.0)})
    return b.finish([x], [y])


def test_standalone_activations_become_layers_of_their_own(port, reference):
    net = tflite.parse(relu_model(), "relu")
    assert [l.op for l in net.layers] == ["activation", "activation", "activation", "softmax"]
    assert [l.act for l in net.layers[:3]] == [(2, 6.0, 0.0), (2, 1.0, -1.0), (1, 0.0, 0.0)]
    x = nets.synthetic_input(net, 5, seed=8)
    a = netref.run_network(port, net, x, keep=True)
    b = netref.run_network(reference, net, x, keep=True)
    for name in a:
        np.testing.assert_array_equal(a[name].data, b[name].data, err_msg=name)
    first = a[net.layers[0].output].data
    assert first.min() == -128 and first.max() == 127            # [0, 6] fills the re-quantized range


def quantize_squeeze_model(squeezed=(2, 24)):
    """uint8 input re-quantized to int8 (QUANTIZE), pooled to 1x1, squeezed to two dimensions, softmax."""
    b = tw.ModelBuilder()
    x = b.tensor("input", (2, 4, 4, 24), tw.UINT8, 0.05, 120)
    q = b.tensor("as_int8", (2, 4, 4, 24), tw.INT8, 0.05, -8)
    b.op(tw.QUANTIZE, [x], [q])
    p = b.tensor("pooled", (2, 1, 1, 24), tw.INT8, 0.05, -8)
    b.op(tw.AVERAGE_POOL_2D, [q], [p], tw.OPT_POOL, {0: ("b", tw.VALID), 1: ("i", 4), 2: ("i", 4), 3: ("i", 4), 4: ("i", 4)})
    s = b.tensor("squeezed", squeezed, tw.INT8, 0.05, -8)
    b.op(tw.SQUEEZE, [p], [s])
    y = b.tensor("probabilities", squeezed, tw.INT8, 1.0 / 256.0, -128)
    b.op(tw.SOFTMAX, [s], [y], tw.OPT_SOFTMAX, {0: ("f", 1.0)})
    return b.finish([x], [y])


def test_quantize_between_8_bit_types_and_squeeze(port, reference):
    net = tflite.parse(quantize_squeeze_model(), "qs")
    assert [l.op for l in net.layers] == ["activation", "pool", "reshape", "softmax"]
    assert net.layers[0].act == (0, 0.0, 0.0)
    x = nets.synthetic_input(net, 2, seed=9)
    a = netref.run_network(port, net, x, keep=True)
    b = netref.run_network(reference, net, x, keep=True)
    for name in a:
        np.testing.assert_array_equal(a[name].data, b[name].data, err_msg=name)
    # same scale, zero points 128 apart: the int8 codes are the uint8 codes shifted
    np.testing.assert_array_equal(a[net.layers[0].output].data.astype(np.int32), x.data.astype(np.int32) - 128)
    with pytest.raises(tflite.UnsupportedModel, match="SQUEEZE"):
        tflite.parse(quantize_squeeze_model(squeezed=(4, 12)), "bad")
