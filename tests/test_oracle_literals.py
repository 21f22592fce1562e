"""The CPU checker against the known-answer vectors the reference's own tests hold (no GPU)."""
import numpy as np
import pytest

from oracle import cpuref
from tests.helpers import load_json, tensor_from_json, lsb_diff

LIT = load_json("reference_literals.json")
ACT = {"ReLu": cpuref.ACT_RELU, "BoundedReLu": cpuref.ACT_BOUNDED_RELU}


def run_case(orc, case, fast):
    x, w, b = (tensor_from_json(case[k]) for k in ("input", "weights", "bias"))
    exp = tensor_from_json(case["output"])
    if case["op"] == "conv2d":
        p = dict(case["params"])
        layout = cpuref.NHWC if p.pop("layout") == "NHWC" else cpuref.NCHW
        y = orc.conv2d(x, w, b, exp.info, data_layout=layout, fast=fast, **p)
    else:
        y = orc.fully_connected(x, w, b, exp.info, transpose_weights=case["params"]["transpose_weights"], fast=fast)
    if "activation" in case:
        a = case["activation"]
        y = orc.activation(y, exp.info, ACT[a["function"]], a["a"], a["b"])
    return y, exp


@pytest.mark.parametrize("case", LIT["cases"], ids=[c["name"] for c in LIT["cases"]])
@pytest.mark.parametrize("fast", [False, True], ids=["literal-loops", "fast"])
def test_port_layer_literals(port, case, fast):
    y, exp = run_case(port, case, fast)
    mx, _ = lsb_diff(y.data, exp.data)
    # vectors produced by CpuRef itself must match exactly; TfLite-produced ones carry the reference's tolerance of 1
    assert mx <= (0 if case["exact_on_cpuref"] else case["tolerance"]), (y.data.ravel(), exp.data.ravel())


@pytest.mark.parametrize("case", LIT["cases"], ids=[c["name"] for c in LIT["cases"]])
def test_reference_build_layer_literals(reference, case):
    y, exp = run_case(reference, case, False)
    mx, _ = lsb_diff(y.data, exp.data)
    assert mx <= (0 if case["exact_on_cpuref"] else case["tolerance"])


@pytest.mark.parametrize("case", LIT["decode_cases"], ids=[c["name"] for c in LIT["decode_cases"]])
def test_port_decoder_literals(port, case):
    out = port.decode(tensor_from_json(case["tensor"]), case["is_depthwise"])
    np.testing.assert_array_equal(out.ravel(), np.asarray(case["expected"], dtype=np.float32))


def test_round_half_away_from_zero(port):
    # Convolution2dPerAxisQuantTest channel 0 is -6.5 -> -7; pin the scalar rule directly as well
    from armnn_amd.tensor import DataType
    assert port.quantize(-6.5, 1.0, 128, DataType.QAsymmU8) == 121
    assert port.quantize(6.5, 1.0, 0, DataType.QAsymmS8) == 7
    assert port.quantize(2.5, 1.0, 0, DataType.QAsymmS8) == 3      # not banker's rounding (would give 2)
    assert port.quantize(-2.5, 1.0, 0, DataType.QAsymmS8) == -3
    assert port.quantize(1e9, 1.0, 0, DataType.QAsymmS8) == 127
    assert port.quantize(-1e9, 1.0, 0, DataType.QAsymmU8) == 0


# PadQAsymmTestCommon (src/backends/backendsCommon/test/layerTests/PadTestImpl.cpp:491-565): a 3x3 tensor of raw codes
# padded by 2 on every side; the expected border holds the pad value itself as a code, whatever scale and offset are.
# PadInt8AsymmTest :758-765 (scale 2, offset 2, pad value 0) and PadInt8CustomPaddingAsymmTest :767-775 (scale 2,
# offset 3, pad value 1).
@pytest.mark.parametrize("scale,offset,value", [(2.0, 2, 0.0), (2.0, 3, 1.0)])
@pytest.mark.parametrize("which", ["port", "reference"])
def test_pad_qasymm_literals(request, which, scale, offset, value):
    from armnn_amd.tensor import DataType, QTensor, TensorInfo
    orc = request.getfixturevalue(which)
    codes = np.array([[4, 8, 6], [7, 4, 4], [3, 2, 4]])
    for dtype in (DataType.QAsymmS8, DataType.QAsymmU8):
        x = QTensor(TensorInfo((3, 3), dtype, (scale,), offset), codes)
        want = np.full((7, 7), int(value))
        want[2:5, 2:5] = codes
        got = orc.pad(x, TensorInfo((7, 7), dtype, (scale,), offset), [2, 2], value)
        np.testing.assert_array_equal(got.data.astype(np.int32), want)
