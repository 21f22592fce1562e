"""The reference's own parser tests for per-channel quantized convolutions (src/armnnTfLiteParser/test/Conv2D.cpp:379-688,
DepthwiseConvolution2D.cpp:406-723), as data: tests/golden/parser_fixtures.json holds each test's model parameters,
input and expected output.  RunTest accepts a difference of 1 between quantized values (SelectiveComparer,
include/armnnTestUtils/TensorHelpers.hpp:24-31), and one of the tests needs it: ...PerChannelQuant4 expects 8 where four
taps of 6 * 0.3 give 7.2 -- the checker, the reference's CpuRef and the device all say 7.  The models are written out as
.tflite files by tests/tflite_writer.py and must give those outputs, by that comparison and exactly wherever the
reference itself does,
  * through the Python reader and the CPU checker,
  * through the C++ parser on the reference's runtime with its CpuRef backend (the reference's test, with this parser),
  * through the C++ parser on the device backend."""
import json
import os
import subprocess

import numpy as np
import pytest

from armnn_amd import tflite
from armnn_amd.tensor import QTensor
from tests import tflite_writer as tw
from tests.helpers import GOLDEN

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "armnn_amd", "backend", "test", "bin")

with open(os.path.join(GOLDEN, "parser_fixtures.json")) as _f:
    FIXTURES = json.load(_f)["fixtures"]
IDS = [f["name"] for f in FIXTURES]
#: where the reference's own CpuRef differs from the test's expectation (by 1, which its comparison accepts)
OFF_BY_ONE = {"ParseDepthwiseConv2DFilterWeightsPerChannelQuant4": 9}


def _compare(f, got):
    d = np.abs(np.asarray(got, np.int64).ravel() - np.array(f["expected"], np.int64))
    assert d.max() <= 1, f["name"]
    assert int((d != 0).sum()) == OFF_BY_ONE.get(f["name"], 0), f["name"]


def model_bytes(f) -> bytes:
    b = tw.ModelBuilder()
    x = b.tensor("inputTensor", tuple(f["input_shape"]), tw.INT8, f["input_scale"], f["input_zero_point"])
    w = b.tensor("filterTensor", tuple(f["filter_shape"]), tw.INT8, np.array(f["filter_scales"], np.float32), f["filter_zero_point"],
                 np.array(f["filter_bytes"], np.uint8).view(np.int8).reshape(f["filter_shape"]), quantized_dimension=f["filter_quantized_dimension"])
    inputs = [x, w]
    if f["bias"] is not None:
        bias = f["bias"]
        inputs.append(b.tensor("biasTensor", tuple(bias["shape"]), tw.INT32, np.array(bias["scales"], np.float32), 0,
                               np.array(bias["bytes"], np.uint8).view("<i4").reshape(bias["shape"])))
    y = b.tensor("outputTensor", tuple(f["output_shape"]), tw.INT8, f["output_scale"], f["output_zero_point"])
    pad = tw.SAME if f["padding"] == "SAME" else tw.VALID
    if f["op"] == "CONV_2D":
        b.op(tw.CONV_2D, inputs, [y], tw.OPT_CONV, {0: ("b", pad), 1: ("i", f["stride"]), 2: ("i", f["stride"]), 3: ("b", tw.ACT_NONE)})
    else:
        # the tests write depth_multiplier 1 whatever the shapes say; the parser goes by the shapes
        b.op(tw.DEPTHWISE_CONV_2D, inputs, [y], tw.OPT_DEPTHWISE,
             {0: ("b", pad), 1: ("i", f["stride"]), 2: ("i", f["stride"]), 3: ("i", 1), 4: ("b", tw.ACT_NONE)})
    return b.finish([x], [y])


@pytest.mark.parametrize("f", FIXTURES, ids=IDS)
def test_python_reader_and_checker_give_the_parser_tests_outputs(port, f):
    from oracle import netref
    net = tflite.parse(model_bytes(f), f["name"])
    info = net.tensors[net.input]
    x = QTensor(info, np.array(f["input"], np.int64).reshape(info.shape))
    got = netref.run_network(port, net, x, fast=False)
    _compare(f, got.data)


def _run(exe, f, tmp_path, backends):
    path, inp, out = str(tmp_path / "model.tflite"), str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(path, "wb") as fh:
        fh.write(model_bytes(f))
    np.array(f["input"], np.int8).tofile(inp)
    proc = subprocess.run([exe, path, inp, out, backends], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    fig = json.loads(proc.stdout.strip().splitlines()[-1])
    return fig, np.fromfile(out, dtype=np.int8).astype(np.int64)


@pytest.mark.parametrize("f", FIXTURES, ids=IDS)
def test_cpp_parser_on_the_reference_runtime_gives_the_parser_tests_outputs(tmp_path, f):
    exe = os.path.join(BIN, "real", "tflite_run")
    if not os.path.exists(exe):
        pytest.skip("not built against an Arm NN source tree (make -C armnn_amd/backend real-armnn real-runtime)")
    fig, got = _run(exe, f, tmp_path, "CpuRef")
    assert fig["output_shape"] == f["output_shape"]
    _compare(f, got)


@pytest.mark.gpu
@pytest.mark.parametrize("f", FIXTURES, ids=IDS)
def test_cpp_parser_on_the_device_gives_the_parser_tests_outputs(tmp_path, f):
    fig, got = _run(os.path.join(BIN, "tflite_run"), f, tmp_path, "Mi355x")
    assert all(layer[2] == "Mi355x" for layer in fig["layers"]), fig["layers"]
    d = np.abs(got - np.array(f["expected"], np.int64))
    print(f["name"], "max |d| =", d.max(), "exact =", float((d == 0).mean()), flush=True)
    _compare(f, got)           # also the same values as the reference's own CpuRef, element for element
