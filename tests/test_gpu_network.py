"""Whole networks on the device vs the CPU checker (needs an MI355X)."""
import numpy as np
import pytest

from armnn_amd import nets, shim
from armnn_amd.executor import DeviceNetwork
from armnn_amd.tensor import QTensor, numpy_dtype
from oracle import netref
from tests.helpers import lsb_diff

pytestmark = pytest.mark.gpu


def _layerwise(port, net, batch):
    """Each device layer is fed the checker's own input for that layer, so every layer is judged at <= 1 LSB
    independently of drift upstream.  Returns the end-to-end device output as well."""
    x = nets.synthetic_input(net, batch)
    ref = netref.run_network(port, net, x, keep=True)
    dn = DeviceNetwork(net, batch, use_graph=False, fuse=False, fuse_add=False)
    worst = 0
    for l, fn in dn.steps:
        for name in l.inputs:
            dn.buffers[name].upload(ref[name].data, dn.stream)
        fn(dn.stream)
        got = dn.download(l.output)
        mx, exact = lsb_diff(got.data, ref[l.output].data)
        print(f"{net.name} b{batch} {l.name:>10s} {l.op:>9s}: max|d|={mx} exact={exact:.6f}", flush=True)
        assert mx <= 1, l.name
        if l.op != "softmax":
            assert exact >= 0.995, l.name
        worst = max(worst, mx)
    # end to end (drift allowed to accumulate): graph replay must equal eager launches bit for bit
    eager = dn.run(x)
    dn.close()
    # depthwise + pointwise pairs as one kernel: same bytes, fewer launches
    df = DeviceNetwork(net, batch, use_graph=False, fuse=True)
    n_fused = sum(1 for l, _ in df.steps if l.op == "dwpw")
    fused = df.run(x)
    df.close()
    print(f"{net.name} b{batch}: {n_fused} fused depthwise+pointwise pairs", flush=True)
    np.testing.assert_array_equal(fused.data, eager.data)
    # pointwise + the depthwise after it as one kernel, where whole images fit a block (graph replay with two lanes too)
    for kw in ({"use_graph": False}, {"use_graph": True, "lanes": 2 if batch % 2 == 0 else 1}):
        df = DeviceNetwork(net, batch, fuse="pwdw", **kw)
        n_fused = sum(1 for l, _ in df.steps if l.op == "dwpw")
        fused = df.run(x)
        df.close()
        print(f"{net.name} b{batch}: {n_fused} fused pointwise+depthwise pairs {kw}", flush=True)
        np.testing.assert_array_equal(fused.data, eager.data)
    # residual Additions inside the write-out of the convolution that feeds them (the default): same bytes
    da = DeviceNetwork(net, batch, use_graph=False, fuse_add=True)
    n_add = sum(1 for l, _ in da.steps if l.op == "convadd")
    with_add = da.run(x)
    da.close()
    print(f"{net.name} b{batch}: {n_add} Additions fused into convolutions", flush=True)
    n_layers = sum(1 for l in net.layers if l.op == "add")
    assert n_add <= n_layers and (n_add == n_layers or not net.name.startswith("resnet"))     # every residual block of ResNet fuses
    np.testing.assert_array_equal(with_add.data, eager.data)
    dg = DeviceNetwork(net, batch, use_graph=True, fuse=False)
    g1 = dg.run(x)
    dg.enqueue()
    g2 = dg.download()
    dg.close()
    np.testing.assert_array_equal(g1.data, eager.data)
    np.testing.assert_array_equal(g2.data, eager.data)
    # the batch split into slices that run side by side on forked streams (eager, then as a replayed graph)
    for lanes in sorted({n for n in (2, 3, 4) if batch % n == 0}):
        for use_graph in (False, True):
            dl = DeviceNetwork(net, batch, use_graph=use_graph, lanes=lanes)
            l1 = dl.run(x)
            dl.enqueue()
            l2 = dl.download()
            dl.close()
            np.testing.assert_array_equal(l1.data, eager.data)
            np.testing.assert_array_equal(l2.data, eager.data)
    mx, exact = lsb_diff(eager.data, ref[net.output].data)
    top1 = float((eager.data.argmax(-1) == ref[net.output].data.argmax(-1)).mean())
    print(f"{net.name} b{batch} end-to-end: max|d|={mx} exact={exact:.6f} top1-agree={top1:.3f}", flush=True)
    return worst


def test_mobilenet_v1_batch2(port):
    _layerwise(port, nets.mobilenet_v1(), 2)


def test_mobilenet_v1_batch1(port):
    # batch 1 selects the matrix-vector classifier and the few-block tilings everywhere
    _layerwise(port, nets.mobilenet_v1(), 1)


def test_resnet50_224_batch2(port):
    # what the batch-32 property test compares its rows with
    _layerwise(port, nets.resnet50(), 2)


def test_resnet50_224_batch1(port):
    # full resolution against the CPU checker: what the batch-32 row-equality test below chains to
    _layerwise(port, nets.resnet50(), 1)


def test_mobilenet_v1_small_odd_resolution(port):
    # odd spatial sizes exercise the SAME-padding edges of every stride-2 layer
    _layerwise(port, nets.mobilenet_v1(resolution=97, classes=37), 3)


def test_resnet50_batch1(port):
    _layerwise(port, nets.resnet50(resolution=96), 1)


def test_resnet50_batch4_in_lanes(port):
    # the residual adds and the pooling layers split by image like the convolutions
    _layerwise(port, nets.resnet50(resolution=64), 4)


def _rows_equal_small_batch_runs(net, batch, picks, lanes):
    """Full-size property: image i of a large batch gives the bytes it gives in a batch of two (images are independent,
    whatever tiles, lanes or kernels the batch size selects); the batch of two is what the layerwise tests tie to the
    CPU checker."""
    x = nets.synthetic_input(net, batch)
    big = DeviceNetwork(net, batch, use_graph=True, lanes=lanes)
    y = big.run(x)
    big.close()
    small = DeviceNetwork(net, 2, use_graph=False)
    for i in picks:
        xi = QTensor(net.info(net.input, 2), np.ascontiguousarray(x.data[i:i + 2]))
        yi = small.run(xi)
        np.testing.assert_array_equal(yi.data, y.data[i:i + 2], err_msg=f"{net.name} images {i},{i + 1} of {batch}")
    small.close()
    assert y.data.max() > y.data.min()                    # not one constant value


def test_mobilenet_v1_batch64_rows_equal_batch2_runs():
    _rows_equal_small_batch_runs(nets.mobilenet_v1(), 64, (0, 31, 62), lanes=2)


def test_mobilenet_v1_batch64_as_the_benchmark_runs_it_rows_equal_batch2_runs():
    """bench.py's configuration: one lane, the pairs the library recommends as one launch each (eleven depthwise + pointwise
    pairs on the fused kernels, pw12 + dw13 in the other order, and pw13 with the global pooling behind it), replayed as a
    graph."""
    net = nets.mobilenet_v1()
    x = nets.synthetic_input(net, 64)
    big = DeviceNetwork(net, 64, use_graph=True, lanes=1, fuse="auto")
    names = [l.name for l, _ in big.steps]
    assert names == (["stem"] + [f"dw{i}+pw{i}" for i in range(1, 12)] + ["dw12", "pw12+dw13", "pw13+avgpool", "logits", "softmax"]), names
    y = big.run(x)
    for _ in range(2):                                    # replays give the same bytes
        big.enqueue()
        np.testing.assert_array_equal(big.download().data, y.data)
    big.close()
    small = DeviceNetwork(net, 2, use_graph=False)
    for i in (0, 17, 40, 62):
        yi = small.run(QTensor(net.info(net.input, 2), np.ascontiguousarray(x.data[i:i + 2])))
        np.testing.assert_array_equal(yi.data, y.data[i:i + 2], err_msg=f"images {i},{i + 1} of 64")
    small.close()


@pytest.mark.parametrize("batch,lanes,forced", [(64, 2, None), (8, 1, None), (6, 2, True), (1, 1, True), (2, 1, None)])
def test_mobilenet_v1_last_convolution_with_the_pooling_behind_it_gives_the_bytes_of_the_layers_run_apart(batch, lanes, forced):
    """fuse_pool None: where the library recommends it (from 32 blocks of four 7 x 7 images x 64 channels per launch on);
    True: wherever it takes the pair.  Both the pooled tensor and the network's output must be those of the unfused run."""
    net = nets.mobilenet_v1()
    x = nets.synthetic_input(net, batch, seed=5)
    apart = DeviceNetwork(net, batch, use_graph=False, lanes=1)
    want = apart.run(x).data.copy()
    want_pooled = apart.download("avgpool:out").data.copy()
    apart.close()
    dn = DeviceNetwork(net, batch, use_graph=True, lanes=lanes, fuse="auto", fuse_pool=forced)
    names = [l.name for l, _ in dn.steps]
    if forced or batch // lanes >= 8:
        assert "pw13+avgpool" in names and "avgpool" not in names, names
    else:
        assert "pw13+avgpool" not in names and "avgpool" in names, names
    for replay in range(2):
        np.testing.assert_array_equal(dn.run(x).data, want, err_msg=f"replay {replay}")
    np.testing.assert_array_equal(dn.download("avgpool:out").data, want_pooled)
    dn.close()


@pytest.mark.parametrize("which,batch,lanes", [("mobilenet", 8, 1), ("resnet", 4, 2)])
def test_the_measured_choice_between_launching_and_replaying_changes_no_byte(which, batch, lanes):
    net = nets.mobilenet_v1(resolution=96, classes=50) if which == "mobilenet" else nets.resnet50(resolution=64)
    x = nets.synthetic_input(net, batch, seed=9)
    dn = DeviceNetwork(net, batch, use_graph=False, lanes=lanes, fuse="auto")
    want = dn.run(x).data.copy()
    trial = dn.choose_submission(passes=10, rounds=2)
    assert set(trial) == {"eager_ms", "graph_ms"} and all(0.0 < v < 50.0 for v in trial.values()), trial
    assert dn.use_graph == (trial["graph_ms"] < trial["eager_ms"])
    np.testing.assert_array_equal(dn.run(x).data, want)
    dn.use_graph = not dn.use_graph                      # the other way gives the same bytes
    np.testing.assert_array_equal(dn.run(x).data, want)
    dn.close()


def test_mobilenet_v1_batch64_in_one_lane_rows_equal_batch2_runs():
    # 64 images per launch: the largest launches of the benchmark (persistent blocks walk the most tiles here)
    _rows_equal_small_batch_runs(nets.mobilenet_v1(), 64, (0, 20, 42, 62), lanes=1)


def test_resnet50_batch32_rows_equal_batch2_runs():
    _rows_equal_small_batch_runs(nets.resnet50(), 32, (0, 15, 30), lanes=2)


def test_two_threads_run_two_networks_at_once():
    """The library is re-entrant per stream: two host threads, each with its own network, plans, buffers and stream,
    give the bytes they give when run one after the other."""
    import threading

    nets_and_batches = [(nets.mobilenet_v1(resolution=96, classes=50), 4), (nets.resnet50(resolution=64), 2)]
    inputs = [nets.synthetic_input(n, b, seed=21 + i) for i, (n, b) in enumerate(nets_and_batches)]
    want = []
    for (n, b), x in zip(nets_and_batches, inputs):
        dn = DeviceNetwork(n, b, use_graph=False)
        want.append(dn.run(x).data.copy())
        dn.close()
    got, errors = [None, None], []

    def worker(k):
        try:
            n, b = nets_and_batches[k]
            dn = DeviceNetwork(n, b, use_graph=(k == 0), lanes=2)
            for _ in range(5):
                out = dn.run(inputs[k]).data.copy()
                np.testing.assert_array_equal(out, want[k])
            got[k] = out
            dn.close()
        except Exception as e:      # reported by the main thread
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=240)
    assert not errors, errors
    assert all(not t.is_alive() for t in threads)
    for k in range(2):
        np.testing.assert_array_equal(got[k], want[k])


def test_tflite_model_from_the_reference_test_data(port):
    """delegate/python/test/test_data/mock_model.tflite (kept under tests/golden): uint8 with asymmetric per-tensor
    weights, a depthwise layer of multiplier 32, max pooling, dense and softmax layers."""
    import os
    from armnn_amd import tflite
    from tests.helpers import GOLDEN
    net = tflite.load(os.path.join(GOLDEN, "mock_model.tflite"))
    _layerwise(port, net, 1)
    _layerwise(port, net, 8)


def test_tflite_model_with_pad_per_channel_weights_and_fused_activations(port):
    from armnn_amd import tflite
    from tests.test_tflite import written_model
    net = tflite.parse(written_model(), "written")
    _layerwise(port, net, 1)
    _layerwise(port, net, 6)


@pytest.mark.parametrize("keep_dims", [True, False])
def test_tflite_model_with_mean_over_height_and_width(port, keep_dims):
    from armnn_amd import tflite
    from tests.test_tflite import mean_model
    net = tflite.parse(mean_model(keep_dims), "mean")
    _layerwise(port, net, 1)
    _layerwise(port, net, 16)


def test_tflite_model_with_standalone_activations(port):
    from armnn_amd import tflite
    from tests.test_tflite import relu_model
    net = tflite.parse(relu_model(), "relu")
    _layerwise(port, net, 1)
    _layerwise(port, net, 32)


def test_tflite_pooling_with_fused_activations(port):
    """The clamp of a fused RELU6 / RELU behind MAX_POOL_2D / AVERAGE_POOL_2D: with input scale 0.1 and offset -20 the
    codes span -10.8 .. 14.7, so both bounds bite and a dropped activation changes most outputs."""
    from armnn_amd import tflite
    from tests.test_tflite import pool_activation_model
    net = tflite.parse(pool_activation_model(), "poolact")
    assert [l.act[0] for l in net.layers if l.op == "pool"] == [2, 1]
    x = nets.synthetic_input(net, 4)
    ref = netref.run_network(port, net, x, keep=True)
    pooled = [l.output for l in net.layers if l.op == "pool"]
    assert ref[pooled[0]].data.max() == -20 + 60 and ref[pooled[0]].data.min() == -20      # 6.0 and 0.0 in codes: both bounds bite
    _layerwise(port, net, 4)


def test_tflite_model_with_quantize_and_squeeze(port):
    from armnn_amd import tflite
    from tests.test_tflite import quantize_squeeze_model
    net = tflite.parse(quantize_squeeze_model(), "qs")
    _layerwise(port, net, 2)


def test_mobilenet_with_per_tensor_uint8_weights(port):
    """Every layer's weights QAsymmU8 with one scale and a zero point: the stem and the depthwise layers multiply with the
    weights minus their zero point in two int8 halves, the pointwise layers and the classifier sum their rows' activations."""
    net = nets.mobilenet_v1(resolution=96, classes=50, weights="per_tensor_u8")
    assert all(l.weights.info.dtype.name == "QAsymmU8" and l.weights.info.offset != 128 for l in net.layers if l.weights is not None)
    _layerwise(port, net, 3)
    dn = DeviceNetwork(net, 3, use_graph=False, fuse=False)
    kinds = {l.name: p.algo()[1] for (l, _), p in zip(dn.steps, dn._step_plans) if p is not None}
    dn.close()
    print(kinds, flush=True)
    assert "two int8 halves" in kinds["stem"] and "smallci_dot4" in kinds["stem"]
    assert all("depthwise3x3_mfma" in k for n, k in kinds.items() if n.startswith("dw"))
    assert all("weight zero point by row sums" in k for n, k in kinds.items() if n.startswith("pw") or n == "logits")
