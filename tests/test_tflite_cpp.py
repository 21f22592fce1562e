"""The C++ TfLite front end (ITfLiteParser of the host core): a .tflite file becomes an INetwork and runs through
Optimize / LoadNetwork / EnqueueWorkload in armnn_amd/backend/test/TfLiteRun.cpp.

  * on the reference's own runtime (the same sources built against an Arm NN tree and its libarmnn.so,
    armnn_amd/backend/test/bin/real/tflite_run): the network the parser builds, computed by the reference's CpuRef
    backend, gives the bytes the Python reader + CPU checker give -- the two front ends agree, and the checker's whole
    network evaluation agrees with the reference's;
  * on the device, on the host core and on the reference's runtime: every layer is placed on Mi355x and the output is
    the Python executor's, byte for byte.
"""
import json
import os
import subprocess

import numpy as np
import pytest

from armnn_amd import tflite
from armnn_amd.tensor import QTensor
from tests import test_tflite as models
from tests.helpers import GOLDEN

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "armnn_amd", "backend", "test", "bin")


def _model_bytes(which):
    if which == "mock":
        with open(os.path.join(GOLDEN, "mock_model.tflite"), "rb") as f:
            return f.read()
    return {"written": models.written_model, "pool_activation": models.pool_activation_model, "mean_keep": lambda: models.mean_model(True),
            "mean_squeeze": lambda: models.mean_model(False), "relu": models.relu_model}[which]()


MODELS = ["mock", "written", "pool_activation", "mean_keep", "mean_squeeze", "relu"]


def _seeded_input(info):
    """the bytes TfLiteRun.cpp draws for the input file '-' (xorshift64)"""
    n = int(np.prod(info.shape))
    s, mask = 88172645463325252, (1 << 64) - 1
    out = np.empty(n, dtype=np.uint8)
    for i in range(n):
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        out[i] = s & 0xFF
    signed = "U8" not in str(info.dtype)
    return QTensor(info, (out.view(np.int8) if signed else out).astype(np.int64).reshape(info.shape))


def _run(exe, data, tmp_path, backends):
    path = str(tmp_path / "model.tflite")
    with open(path, "wb") as f:
        f.write(data)
    out = str(tmp_path / "out.bin")
    env = dict(os.environ)
    proc = subprocess.run([exe, path, "-", out, backends], capture_output=True, text=True, timeout=300, env=env)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    fig = json.loads(proc.stdout.strip().splitlines()[-1])
    return fig, np.fromfile(out, dtype=np.uint8)


def _codes(t):
    return (t.data.astype(np.int64) & 0xFF).astype(np.uint8).ravel()


def _real(name):
    exe = os.path.join(BIN, "real", name)
    if not os.path.exists(exe):
        pytest.skip("not built against an Arm NN source tree (make -C armnn_amd/backend real-armnn real-runtime)")
    return exe


@pytest.mark.parametrize("which", MODELS)
def test_cpp_parser_on_the_reference_runtime_gives_the_checkers_bytes(tmp_path, port, which):
    from oracle import netref
    data = _model_bytes(which)
    fig, got = _run(_real("tflite_run"), data, tmp_path, "CpuRef")
    net = tflite.parse(data, which)
    x = _seeded_input(net.tensors[net.input])
    want = netref.run_network(port, net, x)
    assert fig["input_shape"] == list(net.tensors[net.input].shape) and fig["output_shape"] == list(want.info.shape)
    assert all(layer[2] == "CpuRef" for layer in fig["layers"])
    kinds = [layer[0] for layer in fig["layers"]]
    print(which, kinds)
    np.testing.assert_array_equal(got, _codes(want))


def test_cpp_parser_names_and_bindings_follow_the_reference(tmp_path):
    fig, _ = _run(_real("tflite_run"), _model_bytes("mock"), tmp_path, "CpuRef")
    # binding id = (tensor index << 8) + subgraph index; layer names "<Kind>:<subgraph>:<operator>"
    assert fig["input"] == "input_1" and fig["input_binding"] == 13 << 8
    assert fig["output"] == "dense/Softmax" and fig["output_binding"] == 11 << 8
    names = [layer[1] for layer in fig["layers"]]
    # (the flattening Reshape in front of FULLY_CONNECTED is folded away by the reference's optimizer)
    for want in ("DepthwiseConv2D:0:0", "Conv2D:0:1", "MaxPool2D:0:2", "Conv2D:0:3", "MaxPool2D:0:4",
                 "FullyConnected:0:5", "Softmax:0:6", "Conv2D:0:1:weights", "FullyConnected:0:5:bias"):
        assert want in names, (want, names)


def test_cpp_parser_refuses_damaged_and_unsupported_files(tmp_path):
    exe = os.path.join(BIN, "tflite_run")
    if not os.path.exists(exe):
        import __graft_entry__
        __graft_entry__.build()
    good = _model_bytes("written")

    def fails(data, needle):
        path = str(tmp_path / "bad.tflite")
        with open(path, "wb") as f:
            f.write(data)
        proc = subprocess.run([exe, path, "-", str(tmp_path / "o.bin"), "Mi355x"], capture_output=True, text=True, timeout=60)
        assert proc.returncode == 1 and needle in proc.stderr, (proc.returncode, proc.stderr[-500:])

    fails(b"not a model", "TFL3")
    fails(good[:len(good) // 2], "malformed flatbuffer")
    fails(good[:8] + b"\xff" * 64 + good[72:], "malformed flatbuffer")
    # an operator outside the list: ADD's builtin code rewritten to 18 (MUL)
    from tests import tflite_writer as tw
    b = tw.ModelBuilder()
    x = b.tensor("x", (1, 4, 4, 8), tw.INT8, 0.1, 0)
    y = b.tensor("y", (1, 4, 4, 8), tw.INT8, 0.1, 0)
    b.op(18, [x, x], [y], tw.OPT_ADD, {})
    fails(b.finish([x], [y]), "builtin code 18")
    proc = subprocess.run([exe, str(tmp_path / "missing.tflite"), "-", str(tmp_path / "o.bin"), "Mi355x"], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 1 and "Cannot find the file" in proc.stderr


@pytest.mark.gpu
@pytest.mark.parametrize("runtime", ["host_core", "reference_runtime"])
@pytest.mark.parametrize("which", MODELS)
def test_cpp_parser_to_the_backend_gives_the_executors_bytes(tmp_path, which, runtime):
    from armnn_amd.executor import DeviceNetwork
    exe = os.path.join(BIN, "tflite_run") if runtime == "host_core" else _real("tflite_run")
    assert os.path.exists(exe), "tflite_run is not built"
    data = _model_bytes(which)
    fig, got = _run(exe, data, tmp_path, "Mi355x" if runtime == "host_core" else "Mi355x,CpuRef")
    placed = {layer[2] for layer in fig["layers"]}
    assert placed == {"Mi355x"}, fig["layers"]
    # the fused activations of convolutions, fully connected layers and additions went back into those layers
    assert not any(layer[0] == "Activation" and layer[1].split(":")[0] in ("Conv2D", "DepthwiseConv2D", "FullyConnected", "Add") for layer in fig["layers"]), fig["layers"]
    net = tflite.parse(data, which)
    x = _seeded_input(net.tensors[net.input])
    dn = DeviceNetwork(net, 1, use_graph=False)
    want = dn.run(x)
    dn.close()
    print(f"{which} on {runtime}: {len(fig['layers'])} layers, {fig['ms_per_inference']:.3f} ms")
    np.testing.assert_array_equal(got, _codes(want))
