"""HIP kernels vs the CPU checker through the C ABI, on seeded inputs (needs an MI355X).

Bar: every quantized output within 1 LSB of CpuRef's float-accumulated result (the reference's own tolerance for
quantized layer tests, include/armnnTestUtils/TensorHelpers.hpp:24-31); the exact-match fraction is printed and
asserted to stay high.  Kernels that share the integer accumulation (direct / MFMA / depthwise) must agree with
each other bit for bit.
"""
import numpy as np
import pytest

from armnn_amd import shim
from armnn_amd.tensor import DataType
from tests import cases
from tests.helpers import load_json, tensor_from_json, lsb_diff

pytestmark = pytest.mark.gpu

CONV = cases.small_conv_cases()
FC = cases.small_fc_cases()
LIT = load_json("reference_literals.json")


def _oracle_conv(port, c):
    y = port.conv2d(c.x, c.w, c.b, c.out_info, **c.params)
    fn, a, b = c.act
    return port.activation(y, c.out_info, fn, a, b) if fn else y


def _gpu_conv(c, algo):
    fn, a, b = c.act
    return shim.conv2d(c.x, c.w, c.b, c.out_info, activation=fn, act_a=a, act_b=b, algo=algo, **c.params)


@pytest.mark.parametrize("case", CONV, ids=[c.name for c in CONV])
def test_conv_cases(port, case):
    print(f"case={case.name} x={case.x.info.shape} w={case.w.info.shape}", flush=True)
    want = _oracle_conv(port, case)
    direct = _gpu_conv(case, shim.ALGO_DIRECT)
    mx, exact = lsb_diff(direct.data, want.data)
    print(f"  direct: max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    auto = _gpu_conv(case, shim.ALGO_AUTO)
    np.testing.assert_array_equal(auto.data, direct.data)


@pytest.mark.parametrize("case", FC, ids=[c.name for c in FC])
def test_fc_cases(port, case):
    print(f"case={case.name} x={case.x.info.shape} w={case.w.info.shape}", flush=True)
    fn, a, b = case.act
    want = port.fully_connected(case.x, case.w, case.b, case.out_info, transpose_weights=case.transpose_weights)
    if fn:
        want = port.activation(want, case.out_info, fn, a, b)
    kw = dict(transpose_weights=case.transpose_weights, activation=fn, act_a=a, act_b=b)
    direct = shim.fully_connected(case.x, case.w, case.b, case.out_info, algo=shim.ALGO_DIRECT, **kw)
    mx, exact = lsb_diff(direct.data, want.data)
    print(f"  direct: max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    auto = shim.fully_connected(case.x, case.w, case.b, case.out_info, algo=shim.ALGO_AUTO, **kw)
    np.testing.assert_array_equal(auto.data, direct.data)


@pytest.mark.parametrize("case", [c for c in LIT["cases"] if c["params"].get("layout", "NHWC") == "NHWC"],
                         ids=lambda c: c["name"])
def test_reference_literals_on_gpu(case):
    x, w, b = (tensor_from_json(case[k]) for k in ("input", "weights", "bias"))
    exp = tensor_from_json(case["output"])
    act = case.get("activation")
    fn = {"ReLu": 1, "BoundedReLu": 2}[act["function"]] if act else 0
    a, bb = (act["a"], act["b"]) if act else (0.0, 0.0)
    if case["op"] == "conv2d":
        p = {k: v for k, v in case["params"].items() if k != "layout"}
        y = shim.conv2d(x, w, b, exp.info, activation=fn, act_a=a, act_b=bb, **p)
    else:
        y = shim.fully_connected(x, w, b, exp.info, transpose_weights=case["params"]["transpose_weights"])
    mx, _ = lsb_diff(y.data, exp.data)
    assert mx <= case["tolerance"]


def test_algo_selection():
    c = cases.make_conv_case("sel", 1, ci=16, co=16)
    plan = shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, **c.params)
    assert plan.algo()[0] == shim.ALGO_MFMA
    c = cases.make_conv_case("sel", 1, ci=3, co=16)
    assert shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, **c.params).algo()[0] == shim.ALGO_DOT4
    c = cases.make_conv_case("sel", 1, ci=3, co=15)
    assert shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, **c.params).algo()[0] == shim.ALGO_DIRECT
    c = cases.make_conv_case("sel", 1, ci=24, depthwise=True)
    a, info = shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, **c.params).algo()
    assert a == shim.ALGO_DEPTHWISE and "c4" in info
    c = cases.make_conv_case("sel", 1, ci=16, depthwise=True)
    a, info = shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, **c.params).algo()
    assert a == shim.ALGO_DEPTHWISE and "depthwise3x3" in info
    c = cases.make_conv_case("sel", 1, ci=64, depthwise=True)
    a, info = shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, **c.params).algo()
    assert a == shim.ALGO_DEPTHWISE and "depthwise3x3" in info
    with pytest.raises(shim.ShimError):
        c = cases.make_conv_case("sel", 1, ci=3, co=16)
        shim.Conv2dPlan(c.x.info, c.w, c.b, c.out_info, algo=shim.ALGO_MFMA, **c.params)


def test_fast_epilogue_equals_exact_division():
    """The reciprocal fast path (with its fallback near rounding ties) must give the same bytes as dividing every
    output, on tensors large enough to hit many near-tie values."""
    cs = [cases.make_conv_case("epi_conv", 501, n=4, h=56, w=56, ci=32, co=64, kh=1, kw=1, in_dtype=cases.U8, in_scale=0.0235,
                               in_offset=0, out_scale=0.0235, out_offset=0, act=cases.RELU6),
          cases.make_conv_case("epi_conv_s8", 502, n=2, h=40, w=40, ci=16, co=32, out_scale=0.11, out_offset=17),
          cases.make_conv_case("epi_dw", 503, n=4, h=56, w=56, ci=64, depthwise=True, in_dtype=cases.U8, in_scale=0.0235,
                               in_offset=128, out_scale=0.0235, out_offset=0, act=cases.RELU6, w_scale_range=(0.01, 0.05)),
          cases.make_conv_case("epi_stem", 504, n=4, h=64, w=64, ci=3, co=32, stride=(2, 2), in_dtype=cases.U8,
                               in_scale=0.0078, in_offset=128, out_scale=0.0235, out_offset=0, act=cases.RELU6,
                               w_scale_range=(0.005, 0.02))]
    fast = [_gpu_conv(c, shim.ALGO_AUTO) for c in cs]
    shim.set_option("exact_division_epilogue", 1)
    try:
        exact = [_gpu_conv(c, shim.ALGO_AUTO) for c in cs]
    finally:
        shim.set_option("exact_division_epilogue", 0)
    for c, f, e in zip(cs, fast, exact):
        print(f"{c.name}: {f.data.size} outputs, distinct codes {len(np.unique(f.data))}", flush=True)
        np.testing.assert_array_equal(f.data, e.data)


def test_stem_mfma_equals_stem_dot4():
    """Small-Ci convolutions: the matrix-core kernel and the v_dot4 kernel produce the same bytes."""
    for c in CONV:
        if not c.name.startswith("stem_") or c.out_info.shape[-1] not in (32, 64) or c.w.info.shape[1] not in (3, 7):
            continue
        print("case", c.name, flush=True)
        mfma = _gpu_conv(c, shim.ALGO_AUTO)
        shim.set_option("stem_dot4", 1)
        try:
            dot4 = _gpu_conv(c, shim.ALGO_AUTO)
        finally:
            shim.set_option("stem_dot4", 0)
        np.testing.assert_array_equal(mfma.data, dot4.data)


def test_every_igemm_tiling_gives_the_same_bytes():
    """64x64, 128x64 and 128x128 tiles, 64- and 128-byte k-tiles, uniform-tap and per-thread tap walks: the automatic
    choice depends on the problem size, so every variant is forced on each case and compared with the direct kernel."""
    cs = [cases.make_conv_case("tile_3x3_c64", 601, n=2, h=30, w=28, ci=64, co=96, act=cases.RELU6),           # BK 64, uniform taps
          cases.make_conv_case("tile_3x3_c128_s2", 602, n=2, h=29, w=31, ci=128, co=64, stride=(2, 2)),         # BK 128, uniform taps
          cases.make_conv_case("tile_3x3_c48", 603, n=1, h=33, w=17, ci=48, co=40, in_dtype=cases.U8, in_offset=119),   # taps straddle k-tiles
          cases.make_conv_case("tile_1x1_c256", 604, n=3, h=14, w=14, ci=256, co=512, kh=1, kw=1),              # pointwise, K > 128
          cases.make_conv_case("tile_1x1_c32", 605, n=2, h=20, w=20, ci=32, co=64, kh=1, kw=1)]                 # pointwise, K <= 128 (weight-stationary by default)
    cs.append(cases.make_conv_case("tile_3x3_c128_u8_dil2", 606, n=2, h=19, w=23, ci=128, co=192, dilation=(2, 2), in_dtype=cases.U8,
                                   in_offset=131, out_offset=-100))                                            # direct-to-LDS, xor on fragments
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for tile in (0, 64, 96, 128, 256, 512):
            for lds in (0, 2, 3):              # register-staged kernel, direct-to-LDS kernel with 2 / 3 stages
                shim.set_option("igemm_tile", tile)
                shim.set_option("igemm_lds", lds)
                try:
                    got = _gpu_conv(c, shim.ALGO_MFMA)
                finally:
                    shim.set_option("igemm_tile", 0)
                    shim.set_option("igemm_lds", 2)
                print(f"{c.name} tile {tile} lds {lds}: {got.data.size} outputs", flush=True)
                np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} tile {tile} lds {lds}")
    with pytest.raises(shim.ShimError):
        shim.set_option("igemm_tile", 100)


def test_xcd_groups_over_the_output_channels_give_the_same_bytes():
    """The direct-to-LDS implicit GEMM with its tiles dealt to the XCDs by row range only, and by channel half x row quarter:
    forced both ways on ragged problems (odd and even numbers of column tiles, fewer row blocks than XCD groups, 3x3 and 1x1)."""
    cs = [cases.make_conv_case("xcd_1x1_c512_co1024", 851, n=6, h=7, w=7, ci=512, co=1024, kh=1, kw=1, in_dtype=DataType.QAsymmU8, in_offset=9, act=cases.RELU6),
          cases.make_conv_case("xcd_1x1_c256_co200", 852, n=3, h=14, w=14, ci=256, co=200, kh=1, kw=1),
          cases.make_conv_case("xcd_3x3_c128_co192", 853, n=2, h=13, w=11, ci=128, co=192, act=cases.RELU),
          cases.make_conv_case("xcd_1x1_c128_few_rows", 854, n=1, h=9, w=9, ci=128, co=512, kh=1, kw=1),
          cases.make_conv_case("xcd_1x1_c1024_co1024", 855, n=32, h=7, w=7, ci=1024, co=1024, kh=1, kw=1, in_dtype=DataType.QAsymmU8, in_offset=0, act=cases.RELU6)]
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for cols in (1, 2, 0):
            for tile in (64, 128):
                shim.set_option("igemm_xcd_cols", cols)
                shim.set_option("igemm_tile", tile)
                try:
                    got = _gpu_conv(c, shim.ALGO_MFMA)
                    kernel = shim.last_kernel()
                finally:
                    shim.set_option("igemm_xcd_cols", 0)
                    shim.set_option("igemm_tile", 0)
                assert kernel.startswith("IgemmLdsKernel<"), kernel
                np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} xcd_cols {cols} tile {tile}")


def test_k_split_over_wave_groups_gives_the_same_bytes():
    """Launches of at most one 64x64 block per CU with K >= 2048 split K over two or four groups of waves inside the
    block (IgemmKSplitKernel).  Forced on small and ragged problems -- fewer k-tiles than groups, k-tile counts that do not
    divide by the group count, channel counts that are no multiple of 16, uint8 activations, stride 2 -- and taken
    automatically for the shapes it is meant for; every result against the direct kernel."""
    U8 = DataType.QAsymmU8
    cs = [cases.make_conv_case("ks_3x3_c512_7", 821, n=3, h=7, w=7, ci=512, co=128, act=cases.RELU6),                  # 36 k-tiles
          cases.make_conv_case("ks_3x3_c256_14_u8", 822, n=2, h=14, w=14, ci=256, co=192, in_dtype=U8, in_offset=131, out_offset=-100),
          cases.make_conv_case("ks_1x1_c1024", 823, n=5, h=7, w=5, ci=1024, co=100, kh=1, kw=1),                       # Co % 16 != 0
          cases.make_conv_case("ks_3x3_c128_one_tile_per_tap", 824, n=1, h=9, w=9, ci=128, co=64, in_dtype=U8, in_offset=3),   # 9 k-tiles
          cases.make_conv_case("ks_1x1_c384", 825, n=2, h=6, w=6, ci=384, co=64, kh=1, kw=1),                          # 3 k-tiles < 4 groups
          cases.make_conv_case("ks_1x1_c128", 826, n=1, h=5, w=5, ci=128, co=70, kh=1, kw=1, in_dtype=U8, in_offset=200),     # 1 k-tile
          cases.make_conv_case("ks_3x3_c640_s2", 827, n=4, h=13, w=14, ci=640, co=64, stride=(2, 2), act=cases.RELU)]
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for tile in (2064, 4064):
            shim.set_option("igemm_tile", tile)
            try:
                got = _gpu_conv(c, shim.ALGO_MFMA)
                kernel = shim.last_kernel()
            finally:
                shim.set_option("igemm_tile", 0)
            print(f"{c.name} tile {tile}: {got.data.size} outputs, {kernel}", flush=True)
            assert kernel.startswith("IgemmKSplitKernel<%d" % (tile // 1000)), kernel
            np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} tile {tile}")
    # the automatic choice: ResNet-50's 3x3 layers of the last two stages at 16 images, FullyConnected-like 1x1 with K = 2048
    auto = [(cases.make_conv_case("ks_auto_7x7_c512", 831, n=16, h=7, w=7, ci=512, co=512, act=cases.RELU), 4),
            (cases.make_conv_case("ks_auto_14x14_c256", 832, n=16, h=14, w=14, ci=256, co=256, act=cases.RELU), 2),
            (cases.make_conv_case("ks_auto_7x7_c2048_1x1", 833, n=16, h=7, w=7, ci=2048, co=512, kh=1, kw=1, act=cases.RELU), 4)]
    for c, groups in auto:
        got = _gpu_conv(c, shim.ALGO_AUTO)
        kernel = shim.last_kernel()
        print(f"{c.name}: {kernel}", flush=True)
        assert kernel.startswith("IgemmKSplitKernel<%d" % groups), kernel
        np.testing.assert_array_equal(got.data, _gpu_conv(c, shim.ALGO_DIRECT).data, err_msg=c.name)


def test_resident_tile_convolution_gives_the_same_bytes():
    """Small filters at stride 1 over 64, 128 or 256 input channels keep the input tile in LDS for all taps
    (HaloConvKernel).  Against the direct kernel: every channel count, narrow and wide output-channel tiles with ragged
    channel counts, 3x3 / 2x2 / 1x3 / 3x1 filters, SAME, VALID and asymmetric padding, widths that do and do not divide the
    pixel fragments, a last tile with fewer rows, several images, uint8 activations, fused activations."""
    U8 = DataType.QAsymmU8
    cs = [cases.make_conv_case("halo_c64_56", 801, n=16, h=56, w=56, ci=64, co=64, act=cases.RELU6),
          cases.make_conv_case("halo_c64_ragged", 802, n=3, h=23, w=19, ci=64, co=40, act=cases.RELU),
          cases.make_conv_case("halo_c64_wide_co", 803, n=1, h=30, w=60, ci=64, co=200),
          cases.make_conv_case("halo_c64_2x2_valid_u8", 804, n=2, h=17, w=33, ci=64, co=96, kh=2, kw=2, padding="valid", in_dtype=U8, in_offset=131,
                               out_offset=-100),
          cases.make_conv_case("halo_c128_28", 805, n=2, h=28, w=28, ci=128, co=128, act=cases.RELU),
          cases.make_conv_case("halo_c128_1x3_asym", 806, n=1, h=9, w=41, ci=128, co=72, kh=1, kw=3, padding=(0, 0, 2, 0)),
          cases.make_conv_case("halo_c128_3x1_u8", 807, n=2, h=20, w=14, ci=128, co=256, kh=3, kw=1, in_dtype=U8, in_offset=120, out_offset=10),
          cases.make_conv_case("halo_c256_14", 808, n=3, h=14, w=14, ci=256, co=256, act=cases.RELU),
          cases.make_conv_case("halo_c256_7_asym", 809, n=2, h=7, w=7, ci=256, co=48, padding=(2, 1, 0, 1)),
          cases.make_conv_case("halo_c64_w224", 810, n=1, h=5, w=224, ci=64, co=64)]
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for tile in (0, 3000, 3001):               # 3001: half-height tiles where the output has at most 64 channels
            shim.set_option("igemm_tile", tile)
            try:
                got = _gpu_conv(c, shim.ALGO_MFMA)
                kernel = shim.last_kernel()
            finally:
                shim.set_option("igemm_tile", 0)
            # unforced, launches of fewer blocks than three quarters of the CUs stay on the implicit GEMM
            assert tile == 0 or kernel.startswith("HaloConvKernel<"), kernel
            if tile == 3001 and c.w.info.shape[-1] == 64 and c.out_info.shape[-1] <= 64 and c.out_info.shape[2] <= 128:
                assert kernel.startswith("HaloConvKernel<64, 2, 2, 2,"), kernel
            np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} tile {tile} {kernel}")
        print(f"{c.name}: {want.data.size} outputs, {kernel}", flush=True)
    # 16 images of 56 x 56 make 224 blocks: the automatic choice
    shim.conv2d(cs[0].x, cs[0].w, cs[0].b, cs[0].out_info, activation=cs[0].act[0], act_a=cs[0].act[1], act_b=cs[0].act[2], **cs[0].params)
    assert shim.last_kernel().startswith("HaloConvKernel<"), shim.last_kernel()
    # a forced implicit-GEMM tile keeps the same layers on the other kernels, which must agree as well
    c = cs[0]
    shim.set_option("igemm_tile", 128)
    try:
        got = _gpu_conv(c, shim.ALGO_MFMA)
        assert not shim.last_kernel().startswith("HaloConvKernel<")
    finally:
        shim.set_option("igemm_tile", 0)
    np.testing.assert_array_equal(got.data, _gpu_conv(c, shim.ALGO_DIRECT).data)


def test_large_tile_gemm_gives_the_same_bytes():
    """The one-wave-per-SIMD kernel (256x256, 256x128 and 128x256 block tiles, accumulators in AGPRs) is chosen only for
    launches that fill the device; here each tiling is forced on small problems -- ragged rows and channels, padding,
    stride, dilation, uint8 activations, weights with a zero point, K of one to eighteen k-tiles -- against the direct kernel."""
    S8, U8 = DataType.QAsymmS8, DataType.QAsymmU8
    cs = [cases.make_conv_case("big_1x1_c256", 611, n=3, h=14, w=14, ci=256, co=512, kh=1, kw=1),
          cases.make_conv_case("big_1x1_c128_co200", 612, n=2, h=13, w=11, ci=128, co=200, kh=1, kw=1, act=cases.RELU6),
          cases.make_conv_case("big_3x3_c128_s2", 613, n=2, h=29, w=31, ci=128, co=256, stride=(2, 2)),
          cases.make_conv_case("big_3x3_c128_u8_dil2", 614, n=2, h=19, w=23, ci=128, co=192, dilation=(2, 2), in_dtype=U8,
                               in_offset=131, out_offset=-100),
          cases.make_conv_case("big_3x3_c256_asym_pad", 615, n=1, h=17, w=20, ci=256, co=256, padding=(2, 0, 1, 3), act=cases.RELU),
          cases.make_conv_case("big_1x1_c128_wzp_s8", 616, n=2, h=16, w=16, ci=128, co=256, kh=1, kw=1, w_dtype=S8, per_axis=False, w_offset=-7),
          cases.make_conv_case("big_3x3_c128_wzp_u8", 617, n=1, h=15, w=18, ci=128, co=256, in_dtype=U8, in_offset=120, w_dtype=U8,
                               per_axis=False, w_offset=93, out_offset=10)]
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for tile in (2256, 2128, 1256):
            shim.set_option("igemm_tile", tile)
            try:
                got = _gpu_conv(c, shim.ALGO_MFMA)
            finally:
                shim.set_option("igemm_tile", 0)
            print(f"{c.name} tile {tile}: {got.data.size} outputs", flush=True)
            np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} tile {tile}")
    # FullyConnected rows through the same kernels
    f = cases.make_fc_case("big_fc", 618, m=300, k=1024, o=512)
    want = shim.fully_connected(f.x, f.w, f.b, f.out_info, algo=shim.ALGO_DIRECT)
    for tile in (2256, 2128, 1256):
        shim.set_option("igemm_tile", tile)
        try:
            got = shim.fully_connected(f.x, f.w, f.b, f.out_info)
        finally:
            shim.set_option("igemm_tile", 0)
        np.testing.assert_array_equal(got.data, want.data, err_msg=f"fc tile {tile}")


def test_filters_of_more_than_32_taps_stay_off_the_large_tile_kernel():
    """The large-tile kernel walks at most 32 taps; a 7 x 7 or 6 x 6 convolution over a multiple of 128 channels must run
    on the other tiles -- when a test forces the large tile and when a launch that fills the device would choose it."""
    small = cases.make_conv_case("taps49_c128", 641, n=2, h=15, w=17, ci=128, co=256, kh=7, kw=7, act=cases.RELU)
    six = cases.make_conv_case("taps36_c256", 642, n=1, h=12, w=12, ci=256, co=128, kh=6, kw=6, padding=(2, 3, 2, 3))
    for c in (small, six):
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for tile in (2256, 2128, 0):
            shim.set_option("igemm_tile", tile)
            try:
                got = _gpu_conv(c, shim.ALGO_MFMA)
                kernel = shim.last_kernel()
            finally:
                shim.set_option("igemm_tile", 0)
            assert not kernel.startswith("BigGemmKernel"), kernel
            np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} tile {tile} {kernel}")
    # 8 x 60 x 60 rows over 256 channels: 226 tiles of 256 x 128, which a filter of up to 32 taps would run on the large tile
    big = cases.make_conv_case("taps49_c128_fills_device", 643, n=8, h=60, w=60, ci=128, co=256, kh=7, kw=7, act=cases.RELU6)
    got = _gpu_conv(big, shim.ALGO_AUTO)
    kernel = shim.last_kernel()
    print(f"{big.name}: {kernel}", flush=True)
    assert not kernel.startswith("BigGemmKernel"), kernel
    np.testing.assert_array_equal(got.data, _gpu_conv(big, shim.ALGO_DIRECT).data)
    same = cases.make_conv_case("taps9_c128_fills_device", 644, n=8, h=120, w=120, ci=128, co=256, stride=(2, 2), act=cases.RELU6)
    _gpu_conv(same, shim.ALGO_AUTO)
    assert shim.last_kernel().startswith("BigGemmKernel"), shim.last_kernel()


def test_specialised_kernels_equal_the_exact_division():
    """Every specialised kernel is otherwise compared with the direct kernel, which shares the bracket constants.  Here each
    one runs layers whose bias term is hundreds of codes and whose offsets are far from zero -- wide brackets, saturation on
    both sides -- against the same kernel with the fp32 division of armnn::Quantize forced for every output."""
    U8, S8 = DataType.QAsymmU8, DataType.QAsymmS8
    big_bias = dict(in_scale=0.5, w_scale_range=(0.01, 0.03), out_scale=0.04)          # |bias * s_in * s_w / s_out| up to some hundreds
    runs = [
        (cases.make_conv_case("xd_ksplit", 901, n=2, h=7, w=7, ci=512, co=128, out_offset=100, **big_bias), 4064, None),
        (cases.make_conv_case("xd_ksplit2_u8", 902, n=2, h=14, w=14, ci=256, co=192, in_dtype=U8, in_offset=131, out_dtype=U8, out_offset=250, **big_bias), 2064, None),
        (cases.make_conv_case("xd_halo", 903, n=4, h=23, w=19, ci=64, co=64, out_offset=-100, act=cases.RELU, **big_bias), 3000, None),
        (cases.make_conv_case("xd_big", 904, n=2, h=29, w=31, ci=128, co=256, stride=(2, 2), out_offset=60, **big_bias), 2256, None),
        (cases.make_conv_case("xd_big_1x1", 905, n=3, h=14, w=14, ci=256, co=512, kh=1, kw=1, out_offset=-77, act=cases.RELU6, **big_bias), 2128, None),
        (cases.make_conv_case("xd_lds64", 906, n=3, h=14, w=14, ci=512, co=512, kh=1, kw=1, in_dtype=U8, in_offset=3, out_dtype=U8, out_offset=5, **big_bias), 64, None),
        (cases.make_conv_case("xd_dw128", 907, n=3, h=14, w=14, ci=256, depthwise=True, in_dtype=U8, in_offset=128, out_dtype=U8, out_offset=200,
                              in_scale=0.5, w_scale_range=(0.01, 0.05), out_scale=0.05), 0, shim.ALGO_DEPTHWISE),
        (cases.make_conv_case("xd_dw64_s2", 908, n=2, h=29, w=31, ci=192, depthwise=True, stride=(2, 2), out_offset=-120, in_scale=0.5,
                              w_scale_range=(0.01, 0.05), out_scale=0.05, act=cases.RELU), 0, shim.ALGO_DEPTHWISE),
    ]
    for c, tile, algo in runs:
        got = {}
        for exact in (0, 1):
            shim.set_option("igemm_tile", tile)
            shim.set_option("exact_division_epilogue", exact)
            try:
                got[exact] = _gpu_conv(c, algo if algo is not None else shim.ALGO_MFMA)
                kernel = shim.last_kernel()
            finally:
                shim.set_option("igemm_tile", 0)
                shim.set_option("exact_division_epilogue", 0)
        codes = np.unique(got[1].data)
        print(f"{c.name}: {kernel}, {len(codes)} distinct codes from {codes.min()} to {codes.max()}", flush=True)
        assert len(codes) > 20, c.name                       # not saturated to a handful of values
        np.testing.assert_array_equal(got[0].data, got[1].data, err_msg=f"{c.name} {kernel}")


def test_depthwise_rows_per_thread_variants_give_the_same_bytes():
    """The 3x3 depthwise kernel with one and with two output rows per thread (8- and 16-row tiles), forced on feature maps
    of every parity of height, against the plain depthwise kernel."""
    cs = [cases.make_conv_case("dwr_s1_h14", 701, n=2, h=14, w=14, ci=64, depthwise=True, act=cases.RELU6),
          cases.make_conv_case("dwr_s1_h23", 702, n=1, h=23, w=37, ci=32, depthwise=True, in_dtype=cases.U8, in_offset=140, out_offset=5),
          cases.make_conv_case("dwr_s2_h29", 703, n=2, h=29, w=31, ci=96, depthwise=True, stride=(2, 2)),
          cases.make_conv_case("dwr_s2_h7", 704, n=3, h=7, w=7, ci=32, depthwise=True, stride=(2, 2), act=cases.RELU)]
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for rows in (0, 1, 2):
            shim.set_option("dw_rows", rows)
            shim.set_option("dw_mfma", 0)
            try:
                got = _gpu_conv(c, shim.ALGO_DEPTHWISE)
            finally:
                shim.set_option("dw_rows", 0)
                shim.set_option("dw_mfma", 1)
            print(f"{c.name} rows {rows}", flush=True)
            np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} rows {rows}")


def test_pointwise_slab_widths_give_the_same_bytes():
    """The weight-stationary kernel for 1x1 convolutions with at most 128 input channels, forced to 32-, 64- and
    128-channel weight slabs ("pw_slab"): ragged row counts, uint8 activations, an output width that is no multiple of
    the slab; a value wider than the layer allows is ignored; against the direct kernel."""
    U8 = DataType.QAsymmU8
    cs = [cases.make_conv_case("slab_k64_co256", 851, n=2, h=31, w=29, ci=64, co=256, kh=1, kw=1, act=cases.RELU),
          cases.make_conv_case("slab_k32_co64_u8", 852, n=3, h=17, w=19, ci=32, co=64, kh=1, kw=1, in_dtype=U8, in_offset=128, act=cases.RELU6),
          cases.make_conv_case("slab_k128_co200", 853, n=1, h=23, w=23, ci=128, co=200, kh=1, kw=1)]
    for c in cs:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        seen = set()
        for slab in (0, 32, 64, 128):
            shim.set_option("pw_slab", slab)
            try:
                got = _gpu_conv(c, shim.ALGO_AUTO)
                kernel = shim.last_kernel()
            finally:
                shim.set_option("pw_slab", 0)
            print(f"{c.name} slab {slab}: {kernel}", flush=True)
            assert kernel.startswith("PwGemmKernel<"), kernel
            seen.add(kernel)
            np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} slab {slab}")
        assert len(seen) >= 2, seen
    with pytest.raises(shim.ShimError):
        shim.set_option("pw_slab", 48)


def test_plans_told_that_they_share_the_device_pick_small_blocks_and_give_the_same_bytes():
    """mi355x_conv2d_set_concurrency(plan, 2): the 3x3 convolution over 64 channels leaves the kernel that keeps its input
    tile in LDS for the implicit GEMM with 128x64 tiles, and the 3x3 convolution over 256 channels at 14x14 leaves the
    K split over two wave groups for plain 64x64 blocks; the four-group split of the smallest launches stays; a 1x1
    convolution over 128 channels takes 64-channel weight slabs instead of 128-channel ones (over 64 channels it has them
    anyway).  Same bytes as alone, and as the direct kernel."""
    picks = [(cases.make_conv_case("shared_3x3_c64_56", 841, n=16, h=56, w=56, ci=64, co=64, act=cases.RELU), "HaloConvKernel<64", "IgemmKernel<128, 64"),
             (cases.make_conv_case("shared_3x3_c256_14", 842, n=16, h=14, w=14, ci=256, co=256, act=cases.RELU), "IgemmKSplitKernel<2", "IgemmLdsKernel<64, 64"),
             (cases.make_conv_case("shared_3x3_c512_7", 843, n=16, h=7, w=7, ci=512, co=512, act=cases.RELU), "IgemmKSplitKernel<4", "IgemmKSplitKernel<4"),
             (cases.make_conv_case("shared_1x1_k128_co512", 845, n=3, h=28, w=28, ci=128, co=512, kh=1, kw=1, act=cases.RELU), "PwGemmKernel<128, 4", "PwGemmKernel<64, 4"),
             (cases.make_conv_case("shared_1x1_k64_co256", 846, n=2, h=56, w=56, ci=64, co=256, kh=1, kw=1), "PwGemmKernel<64, 2", "PwGemmKernel<64, 2"),
             (cases.make_conv_case("shared_3x3_c64_small", 844, n=1, h=20, w=20, ci=64, co=64, act=cases.RELU6), None, None)]
    for c, alone_kernel, shared_kernel in picks:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        fn, a, b = c.act
        alone = shim.conv2d(c.x, c.w, c.b, c.out_info, activation=fn, act_a=a, act_b=b, **c.params)
        k1 = shim.last_kernel()
        shared = shim.conv2d(c.x, c.w, c.b, c.out_info, concurrency=2, activation=fn, act_a=a, act_b=b, **c.params)
        k2 = shim.last_kernel()
        print(f"{c.name}: alone {k1}; sharing the device {k2}", flush=True)
        if alone_kernel is None:
            assert k1 == k2, (k1, k2)             # where the resident-tile kernel would not run anyway, nothing changes
        else:
            assert k1.startswith(alone_kernel) and k2.startswith(shared_kernel), (k1, k2)
        np.testing.assert_array_equal(alone.data, want.data, err_msg=c.name)
        np.testing.assert_array_equal(shared.data, want.data, err_msg=c.name)
    with pytest.raises(shim.ShimError):
        shim.Conv2dPlan(picks[-1][0].x.info, picks[-1][0].w, picks[-1][0].b, picks[-1][0].out_info, **picks[-1][0].params).set_concurrency(0)


def test_depthwise_64_and_128_channel_blocks_give_the_same_bytes():
    """Channel counts that are multiples of 128 run the 3x3 depthwise kernel with 128 channels per block (whole lines per
    pixel), the other multiples of 64 with 64: large, mid-sized and tiny feature maps of ragged sizes, both strides, one
    and two rows per thread, uint8 activations, weights with a zero point (two int8 halves), against the 32-channel
    blocks and the plain kernel."""
    for c in _depthwise_block_cases():
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        for cb in (0, 32):
            for rows in (0, 1, 2):
                shim.set_option("dw_cb", cb)
                shim.set_option("dw_rows", rows)
                shim.set_option("dw_mfma", 0)
                try:
                    got = _gpu_conv(c, shim.ALGO_DEPTHWISE)
                    kernel = shim.last_kernel()
                finally:
                    shim.set_option("dw_cb", 0)
                    shim.set_option("dw_rows", 0)
                    shim.set_option("dw_mfma", 1)
                print(f"{c.name} blocks {cb or 'auto'} rows {rows}: {kernel}", flush=True)
                channels = c.x.info.shape[3]
                blocks = 32 if cb == 32 else 128 if channels % 128 == 0 else 64
                assert kernel.startswith("Depthwise3x3Kernel<") and kernel.endswith(f", {blocks}>"), kernel
                np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} blocks {cb} rows {rows}")


def test_depthwise_on_the_matrix_cores_gives_the_same_bytes():
    """The 3x3 depthwise kernel that computes on the matrix cores (sixteen channels x sixteen pixels x four taps per
    instruction), with the tile chosen from the feature map and with every tile edge forced, 32-, 64- and 128-channel
    blocks: ragged feature maps of both strides, uint8 activations, weights as two int8 halves; against the VALU kernel
    and the plain kernel."""
    more = [cases.make_conv_case("dwm_s1_112x112x32", 731, n=2, h=112, w=112, ci=32, depthwise=True, act=cases.RELU6),
            cases.make_conv_case("dwm_s1_14x14x512", 732, n=3, h=14, w=14, ci=512, depthwise=True, act=cases.RELU6),
            cases.make_conv_case("dwm_s2_14x14x48_u8", 733, n=2, h=14, w=14, ci=48, depthwise=True, stride=(2, 2), in_dtype=DataType.QAsymmU8, in_offset=77, out_offset=9),
            cases.make_conv_case("dwm_s1_28x28x16", 734, n=2, h=28, w=28, ci=16, depthwise=True, act=cases.RELU),
            cases.make_conv_case("dwm_s1_1x1x32", 735, n=2, h=1, w=1, ci=32, depthwise=True),
            cases.make_conv_case("dwm_s1_33x17x80", 736, n=1, h=33, w=17, ci=80, depthwise=True, act=cases.RELU6)]
    seen = set()
    for c in _depthwise_block_cases() + more:
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        shim.set_option("dw_mfma", 0)
        try:
            valu = _gpu_conv(c, shim.ALGO_DEPTHWISE)
            assert shim.last_kernel().startswith("Depthwise3x3Kernel<"), shim.last_kernel()
        finally:
            shim.set_option("dw_mfma", 1)
        np.testing.assert_array_equal(valu.data, want.data, err_msg=c.name)
        for tile in (1, 7, 8, 14, 16):
            for cb in (0, 32):
                shim.set_option("dw_mfma", tile)
                shim.set_option("dw_cb", cb)
                try:
                    got = _gpu_conv(c, shim.ALGO_DEPTHWISE)
                    kernel = shim.last_kernel()
                finally:
                    shim.set_option("dw_mfma", 1)
                    shim.set_option("dw_cb", 0)
                print(f"{c.name} tile {tile} blocks {cb or 'auto'}: {kernel}", flush=True)
                assert kernel.startswith("DepthwiseMfmaKernel<"), kernel
                seen.add(kernel)
                np.testing.assert_array_equal(got.data, want.data, err_msg=f"{c.name} tile {tile} blocks {cb}: {kernel}")
    assert len(seen) >= 12, sorted(seen)
    with pytest.raises(shim.ShimError):
        shim.set_option("dw_mfma", 9)


def _depthwise_block_cases():
    U8 = DataType.QAsymmU8
    return [cases.make_conv_case("dw128_s1_57x53", 711, n=2, h=57, w=53, ci=128, depthwise=True, act=cases.RELU6),
          cases.make_conv_case("dw128_s2_57x53_u8", 712, n=2, h=57, w=53, ci=256, depthwise=True, stride=(2, 2), in_dtype=U8, in_offset=140, out_offset=5),
          cases.make_conv_case("dw128_s1_7x7", 713, n=3, h=7, w=7, ci=256, depthwise=True, act=cases.RELU),
          cases.make_conv_case("dw128_s2_8x5", 714, n=2, h=8, w=5, ci=128, depthwise=True, stride=(2, 2)),
          cases.make_conv_case("dw128_s1_29x27", 716, n=3, h=29, w=27, ci=256, depthwise=True, act=cases.RELU6),
          cases.make_conv_case("dw128_s2_29x27", 717, n=3, h=29, w=27, ci=128, depthwise=True, stride=(2, 2), act=cases.RELU),
          cases.make_conv_case("dw128_s1_15x13_u8", 718, n=5, h=15, w=13, ci=512, depthwise=True, in_dtype=U8, in_offset=131, out_offset=2),
          cases.make_conv_case("dw64_s2_113x59", 719, n=2, h=113, w=59, ci=64, depthwise=True, stride=(2, 2), act=cases.RELU6),
          cases.make_conv_case("dw64_s1_37x41_u8", 720, n=2, h=37, w=41, ci=192, depthwise=True, in_dtype=U8, in_offset=99, out_offset=-7, act=cases.RELU),
          cases.make_conv_case("dw64_s1_6x9", 721, n=3, h=6, w=9, ci=64, depthwise=True),
          cases.make_conv_case("dw64_s2_30x30_zero_point_weights", 722, n=1, h=30, w=30, ci=320, depthwise=True, stride=(2, 2), per_axis=False, w_std=60.0,
                               w_dtype=U8, w_offset=101, in_dtype=U8, in_offset=120, out_offset=3, act=cases.RELU6),
          cases.make_conv_case("dw128_s1_64x50_zero_point_weights", 715, n=1, h=64, w=50, ci=128, depthwise=True, per_axis=False, w_std=60.0,
                               w_dtype=U8, w_offset=93, in_dtype=U8, in_offset=120, out_offset=3, act=cases.RELU6)]
    with pytest.raises(shim.ShimError):
        shim.set_option("dw_cb", 64)


def test_launches_of_tens_of_megabytes_equal_the_plain_kernel():
    """The benchmark networks' largest launches (64 and 32 images of the early MobileNetV1 / ResNet-50 layers: outputs of
    13 to 51 MB, thousands of blocks, persistent blocks walking many tiles) against the plain one-thread-per-output kernel.
    Small cases cannot show a store that goes wrong once in a million."""
    U8 = DataType.QAsymmU8
    cs = [cases.make_conv_case("big_pw_32_64_n64", 901, n=64, h=112, w=112, ci=32, co=64, kh=1, kw=1, in_dtype=U8, in_offset=0, out_offset=0, act=cases.RELU6),
          cases.make_conv_case("big_pw_64_128_n32", 902, n=32, h=56, w=56, ci=64, co=128, kh=1, kw=1, in_dtype=U8, in_offset=0, out_offset=0, act=cases.RELU6),
          cases.make_conv_case("big_pw_128_128_n64", 903, n=64, h=56, w=56, ci=128, co=128, kh=1, kw=1, act=cases.RELU6),
          cases.make_conv_case("big_pw_256_256_n32", 904, n=32, h=28, w=28, ci=256, co=256, kh=1, kw=1, act=cases.RELU6),
          cases.make_conv_case("big_stem_n32", 905, n=32, h=224, w=224, ci=3, co=32, stride=(2, 2), in_dtype=U8, in_offset=128, out_offset=0, act=cases.RELU6),
          cases.make_conv_case("big_c1_n64", 906, n=64, h=56, w=56, ci=64, co=64, act=cases.RELU6),
          cases.make_conv_case("big_dw_128_n32", 907, n=32, h=56, w=56, ci=128, depthwise=True, in_dtype=U8, in_offset=0, out_offset=0, act=cases.RELU6),
          cases.make_conv_case("big_dw_128_s2_n32", 908, n=32, h=56, w=56, ci=128, depthwise=True, stride=(2, 2), act=cases.RELU6)]
    for c in cs:
        got = _gpu_conv(c, shim.ALGO_AUTO)
        kernel = shim.last_kernel()
        want = _gpu_conv(c, shim.ALGO_DIRECT)
        bad = int((got.data != want.data).sum())
        print(f"{c.name}: {got.data.size} outputs, {kernel}, {bad} differ", flush=True)
        assert bad == 0, f"{c.name} {kernel}: {bad} of {got.data.size} bytes differ"


def test_config_c1_full_size(port):
    """Benchmark configuration C1: 1x56x56x64 -> 64, 3x3 SAME, per-channel, ReLU6; expected code range [-128, -8]."""
    c = cases.make_conv_case("C1", 20250101, h=56, w=56, ci=64, co=64, act=cases.RELU6)
    want = _oracle_conv(port, c)
    got = _gpu_conv(c, shim.ALGO_AUTO)
    mx, exact = lsb_diff(got.data, want.data)
    print(f"C1: max|d|={mx} exact={exact:.6f} range=[{got.data.min()},{got.data.max()}]", flush=True)
    assert mx <= 1 and exact >= 0.999
    assert got.data.min() == -128 and got.data.max() == -8
    np.testing.assert_array_equal(_gpu_conv(c, shim.ALGO_DIRECT).data, got.data)


def test_config_c2_block(port):
    """Benchmark configuration C2: depthwise 3x3 + pointwise 32->64 on 1x112x112x32 QAsymmU8, ReLU6 after each."""
    U8 = DataType.QAsymmU8
    dw = cases.make_conv_case("C2dw", 20250102, h=112, w=112, ci=32, depthwise=True, in_dtype=U8, in_scale=0.0235,
                              in_offset=128, out_scale=0.0235, out_offset=0, act=cases.RELU6, w_scale_range=(0.01, 0.05))
    want1 = _oracle_conv(port, dw)
    got1 = _gpu_conv(dw, shim.ALGO_AUTO)
    mx, exact = lsb_diff(got1.data, want1.data)
    print(f"C2 dw: max|d|={mx} exact={exact:.6f}", flush=True)
    assert mx <= 1 and exact >= 0.999
    pw = cases.make_conv_case("C2pw", 20250103, h=112, w=112, ci=32, co=64, kh=1, kw=1, in_dtype=U8, in_scale=0.0235,
                              in_offset=0, out_scale=0.0235, out_offset=0, act=cases.RELU6)
    pw.x.data = want1.data          # feed the oracle's intermediate so the two stages are judged independently
    want2 = _oracle_conv(port, pw)
    got2 = _gpu_conv(pw, shim.ALGO_AUTO)
    mx, exact = lsb_diff(got2.data, want2.data)
    print(f"C2 pw: max|d|={mx} exact={exact:.6f} max code={got2.data.max()}", flush=True)
    assert mx <= 1 and exact >= 0.999


@pytest.mark.parametrize("m", [1, 256, 2048])
def test_config_c4_fc(port, m):
    """Benchmark configuration C4: [M,4096] x [4096,4096] per-channel, fused requantize (output scale 1.0, zp 0), at the
    three row counts the configuration names; M = 2048 is the size the large GEMM tilings are selected and timed at."""
    c = cases.make_fc_case("C4", 20250104, m=m, k=4096, o=4096, in_offset=0, out_scale=1.0, out_offset=0)
    want = port.fully_connected(c.x, c.w, c.b, c.out_info)
    got = shim.fully_connected(c.x, c.w, c.b, c.out_info)
    mx, exact = lsb_diff(got.data, want.data)
    sat = float(((got.data == 127) | (got.data == -128)).mean())
    print(f"C4 M={m}: max|d|={mx} exact={exact:.6f} saturated={sat:.4f}", flush=True)
    assert mx <= 1 and exact >= 0.995 and sat < 0.05
    if m == 2048:
        direct = shim.fully_connected(c.x, c.w, c.b, c.out_info, algo=shim.ALGO_DIRECT)
        np.testing.assert_array_equal(got.data, direct.data)


def test_c4_fc_8192_rows_equal_direct_kernel():
    """M = 8192 selects the largest GEMM tiling; the rows are independent, so every row must carry the bytes the
    one-thread-per-output kernel gives (which the M = 2048 case ties to the CPU checker)."""
    c = cases.make_fc_case("C4big", 20250105, m=8192, k=4096, o=4096, in_offset=0, out_scale=1.0, out_offset=0)
    got = shim.fully_connected(c.x, c.w, c.b, c.out_info)
    direct = shim.fully_connected(c.x, c.w, c.b, c.out_info, algo=shim.ALGO_DIRECT)
    np.testing.assert_array_equal(got.data, direct.data)
    assert got.data.max() > got.data.min()


def _random_conv_case(k):
    """One seeded draw from the space of convolutions the library accepts: shapes, strides, dilations, paddings, data
    types, per-channel or per-tensor (also asymmetric) weights, output quantizations from coarse to fine, activations."""
    rng = np.random.default_rng(7000 + k)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    depthwise = bool(rng.integers(4) == 0)
    kh, kw = pick([1, 1, 2, 3, 3, 3, 5]), pick([1, 1, 2, 3, 3, 3, 5])
    if rng.integers(3) != 0:
        kw = kh
    dil = (pick([1, 1, 1, 2]), pick([1, 1, 1, 2]))
    h = int(rng.integers(max(1, (kh - 1) * dil[1] - 1), 24))
    w = int(rng.integers(max(1, (kw - 1) * dil[0] - 1), 24))
    ci = pick([1, 3, 4, 8, 16, 20, 32, 48, 64, 128, 256])
    co = pick([1, 5, 8, 16, 32, 40, 64, 128, 256])
    in_u8 = bool(rng.integers(2))
    padding = pick(["same", "valid", (int(rng.integers(0, kh + 1)), int(rng.integers(0, kh + 1)), int(rng.integers(0, kw + 1)), int(rng.integers(0, kw + 1)))])
    if padding == "valid" and (h < (kh - 1) * dil[1] + 1 or w < (kw - 1) * dil[0] + 1):
        padding = "same"
    w_kind = pick(["per_axis", "per_axis", "per_tensor", "asym_s8", "asym_u8"])
    w_dtype = {"asym_s8": DataType.QAsymmS8, "asym_u8": DataType.QAsymmU8}.get(w_kind, DataType.QSymmS8)
    w_offset = {"asym_s8": int(rng.integers(-20, 20)), "asym_u8": int(rng.integers(100, 150))}.get(w_kind, 0)
    out_scale = float(np.exp(rng.uniform(np.log(0.004), np.log(0.5))))
    lo = 0 if in_u8 else -128
    act = pick([(0, 0.0, 0.0), (1, 0.0, 0.0), (2, 6.0, 0.0), (2, 1.0, -1.0)])
    return cases.make_conv_case(
        f"random{k}", 9000 + 11 * k, n=int(rng.integers(1, 4)), h=h, w=w, ci=ci, co=co, kh=kh, kw=kw,
        stride=(pick([1, 1, 2, 3]), pick([1, 1, 2, 3])), dilation=dil, padding=padding, depthwise=depthwise,
        mult=pick([1, 1, 1, 2]) if depthwise else 1, in_dtype=DataType.QAsymmU8 if in_u8 else DataType.QAsymmS8,
        in_scale=float(rng.uniform(0.005, 0.05)), in_offset=lo + int(rng.integers(0, 256)), w_dtype=w_dtype,
        per_axis=w_kind == "per_axis", w_offset=w_offset, bias=bool(rng.integers(4) != 0),
        bias_scale_matches=bool(rng.integers(5) != 0), out_scale=out_scale, out_offset=lo + int(rng.integers(0, 256)), act=act)


@pytest.mark.parametrize("chunk", range(8))
def test_random_convolutions(port, chunk):
    """240 seeded draws, 30 per test: whatever kernel AUTO picks must stay within 1 LSB of the checker and give the
    bytes of the direct kernel."""
    for k in range(30 * chunk, 30 * chunk + 30):
        try:
            case = _random_conv_case(k)
        except ValueError:
            continue                                   # a draw whose output would be empty
        if 0 in case.out_info.shape:
            continue
        print(f"random case {k}: x={case.x.info.shape} w={case.w.info.shape} {case.w.info.dtype.name} params={case.params} "
              f"act={case.act} out={case.out_info.scale:.4f}/{case.out_info.offset}", flush=True)
        want = _oracle_conv(port, case)
        auto = _gpu_conv(case, shim.ALGO_AUTO)
        mx, exact = lsb_diff(auto.data, want.data)
        assert mx <= 1, (k, mx)
        assert exact >= 0.995 or auto.data.size < 200, (k, exact)
        direct = _gpu_conv(case, shim.ALGO_DIRECT)
        np.testing.assert_array_equal(auto.data, direct.data, err_msg=f"random case {k}")


def _fast_path_case(k):
    """A seeded draw from the shapes the specialised kernels take: pointwise and 3x3 convolutions with channel counts in
    multiples of 16, 3x3 depthwise layers with channels in multiples of 32, stems with 1..4 input channels."""
    rng = np.random.default_rng(17000 + k)
    pick = lambda xs: xs[int(rng.integers(len(xs)))]
    family = pick(["pointwise", "pointwise", "conv3x3", "conv3x3", "depthwise", "depthwise", "stem"])
    in_u8 = bool(rng.integers(2))
    lo = 0 if in_u8 else -128
    kw = dict(n=int(rng.integers(1, 6)), h=int(rng.integers(3, 41)), w=int(rng.integers(3, 41)), per_axis=bool(rng.integers(4) != 0),
              in_dtype=DataType.QAsymmU8 if in_u8 else DataType.QAsymmS8, in_scale=float(rng.uniform(0.005, 0.05)),
              in_offset=lo + int(rng.integers(0, 256)), bias=bool(rng.integers(5) != 0),
              out_scale=float(np.exp(rng.uniform(np.log(0.01), np.log(0.3)))), out_offset=lo + int(rng.integers(0, 256)),
              act=pick([(0, 0.0, 0.0), (1, 0.0, 0.0), (2, 6.0, 0.0)]))
    if family == "pointwise":
        kw.update(ci=pick([16, 32, 64, 96, 128, 256, 512]), co=pick([16, 24, 32, 64, 128, 200, 256, 512]), kh=1, kw=1, padding="valid")
    elif family == "conv3x3":
        kw.update(ci=pick([16, 32, 64, 128, 256]), co=pick([16, 32, 64, 128, 256]), kh=3, kw=3, stride=pick([(1, 1), (1, 1), (2, 2)]),
                  padding=pick(["same", "same", "valid", (1, 0, 2, 1)]))
    elif family == "depthwise":
        kw.update(ci=pick([32, 64, 96, 128, 256, 512]), kh=3, kw=3, depthwise=True, stride=pick([(1, 1), (2, 2)]), padding=pick(["same", "same", "valid"]))
    else:
        size = pick([3, 3, 7])
        kw.update(ci=pick([1, 3, 3, 4]), co=pick([32, 64]), kh=size, kw=size, stride=pick([(1, 1), (2, 2), (2, 2)]), padding="same",
                  h=int(rng.integers(8, 65)), w=int(rng.integers(8, 65)))
    return cases.make_conv_case(f"fast{k}", 19000 + 13 * k, **kw)


@pytest.mark.parametrize("chunk", range(6))
def test_random_draws_from_the_specialised_kernels_shapes(port, chunk):
    for k in range(30 * chunk, 30 * chunk + 30):
        case = _fast_path_case(k)
        print(f"fast-path case {k}: x={case.x.info.shape} w={case.w.info.shape} params={case.params} act={case.act} "
              f"out={case.out_info.scale:.4f}/{case.out_info.offset}", flush=True)
        want = _oracle_conv(port, case)
        auto = _gpu_conv(case, shim.ALGO_AUTO)
        mx, exact = lsb_diff(auto.data, want.data)
        assert mx <= 1, (k, mx)
        assert exact >= 0.995, (k, exact)
        direct = _gpu_conv(case, shim.ALGO_DIRECT)
        np.testing.assert_array_equal(auto.data, direct.data, err_msg=f"fast-path case {k}")


@pytest.mark.parametrize("chunk", range(3))
def test_random_fully_connected(port, chunk):
    for k in range(20 * chunk, 20 * chunk + 20):
        rng = np.random.default_rng(27000 + k)
        in_u8 = bool(rng.integers(2))
        lo = 0 if in_u8 else -128
        m = int(rng.choice([1, 2, 3, 4, 5, 7, 16, 33, 64, 65, 130, 300]))
        kdim = int(rng.choice([16, 48, 64, 100, 128, 256, 1000, 1024, 2048]))
        o = int(rng.choice([1, 10, 16, 37, 64, 128, 1000, 1001]))
        case = cases.make_fc_case(f"fc{k}", 29000 + 7 * k, m=m, k=kdim, o=o, in_dtype=DataType.QAsymmU8 if in_u8 else DataType.QAsymmS8,
                                  in_scale=float(rng.uniform(0.005, 0.05)), in_offset=lo + int(rng.integers(0, 256)),
                                  out_scale=float(np.exp(rng.uniform(np.log(0.01), np.log(0.5)))), out_offset=lo + int(rng.integers(0, 256)))
        print(f"fc case {k}: m={m} k={kdim} o={o} u8={in_u8}", flush=True)
        fn, a, b = case.act
        want = port.fully_connected(case.x, case.w, case.b, case.out_info, transpose_weights=case.transpose_weights)
        if fn:
            want = port.activation(want, case.out_info, fn, a, b)
        kw = dict(transpose_weights=case.transpose_weights, activation=fn, act_a=a, act_b=b)
        auto = shim.fully_connected(case.x, case.w, case.b, case.out_info, algo=shim.ALGO_AUTO, **kw)
        mx, exact = lsb_diff(auto.data, want.data)
        assert mx <= 1, (k, mx)
        assert exact >= 0.995 or auto.data.size < 200, (k, exact)
        direct = shim.fully_connected(case.x, case.w, case.b, case.out_info, algo=shim.ALGO_DIRECT, **kw)
        np.testing.assert_array_equal(auto.data, direct.data, err_msg=f"fc case {k}")


_ZP_CONVS = [
    # (name, conv kwargs): per-tensor weights with a zero point, shapes the MFMA implicit GEMM takes (in_c % 16 == 0)
    ("u8_pointwise_c32", dict(n=3, h=14, w=14, ci=32, co=64, kh=1, kw=1, padding="valid", w_dtype=DataType.QAsymmU8, w_offset=93)),
    ("u8_pointwise_c128_ragged_co", dict(n=2, h=9, w=11, ci=128, co=200, kh=1, kw=1, padding="valid", w_dtype=DataType.QAsymmU8, w_offset=151)),
    ("u8_3x3_same_c64", dict(n=2, h=13, w=17, ci=64, co=128, kh=3, kw=3, padding="same", w_dtype=DataType.QAsymmU8, w_offset=120)),
    ("u8_3x3_s2_c48", dict(n=2, h=15, w=15, ci=48, co=32, kh=3, kw=3, stride=(2, 2), padding="same", w_dtype=DataType.QAsymmU8, w_offset=3)),
    ("u8_3x3_c128_uniform_tap", dict(n=1, h=12, w=12, ci=128, co=128, kh=3, kw=3, padding=(1, 0, 2, 1), w_dtype=DataType.QAsymmU8, w_offset=255)),
    ("u8_5x5_dilated_c16", dict(n=1, h=20, w=18, ci=16, co=48, kh=5, kw=5, dilation=(2, 2), padding="same", w_dtype=DataType.QAsymmU8, w_offset=0)),
    ("u8_zero_point_128_is_symmetric", dict(n=4, h=14, w=14, ci=64, co=64, kh=1, kw=1, padding="valid", w_dtype=DataType.QAsymmU8, w_offset=128)),
    ("s8_pointwise_c256", dict(n=2, h=7, w=7, ci=256, co=512, kh=1, kw=1, padding="valid", w_dtype=DataType.QAsymmS8, w_offset=-17)),
    ("s8_3x3_c32_big_batch", dict(n=16, h=28, w=28, ci=32, co=64, kh=3, kw=3, padding="same", w_dtype=DataType.QAsymmS8, w_offset=127)),
    ("s8_3x3_lowest_zero_point", dict(n=1, h=8, w=8, ci=16, co=16, kh=3, kw=3, padding="same", w_dtype=DataType.QAsymmS8, w_offset=-128)),
]


@pytest.mark.parametrize("in_u8", [False, True], ids=["s8_in", "u8_in"])
@pytest.mark.parametrize("name,kw", _ZP_CONVS, ids=[n for n, _ in _ZP_CONVS])
def test_weights_with_a_zero_point_on_the_matrix_cores(port, name, kw, in_u8):
    """Per-tensor QAsymmU8 / QAsymmS8 weights whose zero point is not 0: the implicit GEMM sums each pixel's activations
    beside the products; the bytes must be the direct kernel's and within 1 LSB of the checker."""
    seed = 31000 + 7 * [n for n, _ in _ZP_CONVS].index(name) + int(in_u8)
    case = cases.make_conv_case(name, seed, per_axis=False, in_dtype=DataType.QAsymmU8 if in_u8 else DataType.QAsymmS8,
                                in_offset=131 if in_u8 else -9, out_offset=100 if in_u8 else -20, act=(2, 6.0, 0.0), **kw)
    print(f"{name}: x={case.x.info.shape} w={case.w.info.shape} zw={case.w.info.offset}", flush=True)
    fn, a, b = case.act
    plan = shim.Conv2dPlan(case.x.info, case.w, case.b, case.out_info, activation=fn, act_a=a, act_b=b, algo=shim.ALGO_AUTO, **case.params)
    algo, desc = plan.algo()
    plan.destroy()
    print(f"  kernel: {desc}", flush=True)
    assert algo == shim.ALGO_MFMA
    assert ("weight zero point" in desc) == (case.w.info.offset != (128 if case.w.info.dtype == DataType.QAsymmU8 else 0))
    want = _oracle_conv(port, case)
    auto = _gpu_conv(case, shim.ALGO_AUTO)
    mx, exact = lsb_diff(auto.data, want.data)
    print(f"  max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    np.testing.assert_array_equal(auto.data, _gpu_conv(case, shim.ALGO_DIRECT).data)


@pytest.mark.parametrize("m", [1, 3, 4, 40, 64, 256])
@pytest.mark.parametrize("k", [512, 400], ids=["k512", "k400_half_last_step"])
@pytest.mark.parametrize("w_dtype,w_offset", [(DataType.QAsymmU8, 93), (DataType.QAsymmS8, -30)])
def test_fully_connected_weights_with_a_zero_point(port, m, k, w_dtype, w_offset):
    """Rows from one (matrix-vector kernel) over a few dozen (32x32 tiles with K split over the waves) to the tiled GEMM."""
    case = cases.make_fc_case(f"fc_zp_m{m}", 32000 + m + k, m=m, k=k, o=320, in_dtype=DataType.QAsymmU8, in_offset=63, w_dtype=w_dtype,
                              per_axis=False, w_offset=w_offset, out_offset=30)
    print(f"fc m={m} k={k} {w_dtype.name} zw={w_offset}", flush=True)
    kw = dict(transpose_weights=case.transpose_weights)
    want = port.fully_connected(case.x, case.w, case.b, case.out_info, **kw)
    auto = shim.fully_connected(case.x, case.w, case.b, case.out_info, algo=shim.ALGO_AUTO, **kw)
    mx, exact = lsb_diff(auto.data, want.data)
    print(f"  max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    direct = shim.fully_connected(case.x, case.w, case.b, case.out_info, algo=shim.ALGO_DIRECT, **kw)
    np.testing.assert_array_equal(auto.data, direct.data)


_ZP_DEPTHWISE = [
    ("u8_zp128_fits_int8", dict(n=2, h=20, w=20, ci=32, stride=(1, 1), w_dtype=DataType.QAsymmU8, w_offset=128), False),
    ("u8_zp93_two_halves", dict(n=3, h=19, w=23, ci=64, stride=(1, 1), w_dtype=DataType.QAsymmU8, w_offset=93), True),
    ("u8_zp160_stride2", dict(n=2, h=28, w=28, ci=96, stride=(2, 2), w_dtype=DataType.QAsymmU8, w_offset=160), True),
    ("u8_zp1_small_map", dict(n=5, h=7, w=7, ci=128, stride=(1, 1), w_dtype=DataType.QAsymmU8, w_offset=1), True),
    ("s8_zp-40", dict(n=2, h=16, w=16, ci=32, stride=(2, 2), w_dtype=DataType.QAsymmS8, w_offset=-40), True),
    ("s8_zp5_tall_batch", dict(n=16, h=56, w=56, ci=32, stride=(1, 1), w_dtype=DataType.QAsymmS8, w_offset=5), None),
]


@pytest.mark.parametrize("in_u8", [False, True], ids=["s8_in", "u8_in"])
@pytest.mark.parametrize("name,kw,halves", _ZP_DEPTHWISE, ids=[n for n, _, _ in _ZP_DEPTHWISE])
def test_depthwise_weights_with_a_zero_point(port, name, kw, halves, in_u8):
    """3x3 depthwise layers whose per-tensor weights have a zero point run on the v_dot4 kernel with the weights minus
    their zero point, as one int8 where that fits and as two halves otherwise."""
    seed = 33000 + 5 * [n for n, _, _ in _ZP_DEPTHWISE].index(name) + int(in_u8)
    case = cases.make_conv_case(name, seed, kh=3, kw=3, padding="same", depthwise=True, per_axis=False, w_std=60.0,
                                in_dtype=DataType.QAsymmU8 if in_u8 else DataType.QAsymmS8, in_offset=140 if in_u8 else 11,
                                out_offset=3 if in_u8 else -100, act=(2, 6.0, 0.0), **kw)
    fn, a, b = case.act
    plan = shim.Conv2dPlan(case.x.info, case.w, case.b, case.out_info, activation=fn, act_a=a, act_b=b, algo=shim.ALGO_AUTO, **case.params)
    algo, desc = plan.algo()
    plan.destroy()
    print(f"{name}: x={case.x.info.shape} zw={case.w.info.offset} kernel: {desc}", flush=True)
    assert "depthwise3x3_mfma" in desc
    if halves is not None:
        assert ("two int8 halves" in desc) == halves
    want = _oracle_conv(port, case)
    auto = _gpu_conv(case, shim.ALGO_AUTO)
    mx, exact = lsb_diff(auto.data, want.data)
    print(f"  max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    np.testing.assert_array_equal(auto.data, _gpu_conv(case, shim.ALGO_DIRECT).data)


def test_depthwise_weight_255_above_its_zero_point_takes_the_general_kernel(port):
    case = cases.make_conv_case("dw_d255", 33900, n=1, h=9, w=9, ci=32, kh=3, kw=3, padding="same", depthwise=True, per_axis=False,
                                in_dtype=DataType.QAsymmU8, in_offset=128, w_dtype=DataType.QAsymmU8, w_offset=0)
    case.w.data.reshape(-1)[5] = 255
    plan = shim.Conv2dPlan(case.x.info, case.w, case.b, case.out_info, algo=shim.ALGO_AUTO, **case.params)
    desc = plan.algo()[1]
    plan.destroy()
    assert desc == "depthwise_c4_valu"
    want = _oracle_conv(port, case)
    got = _gpu_conv(case, shim.ALGO_AUTO)
    assert lsb_diff(got.data, want.data)[0] <= 1


_ZP_STEMS = [
    ("u8_3x3_s2_rgb_two_halves", dict(n=2, h=33, w=35, ci=3, co=32, kh=3, kw=3, stride=(2, 2), w_dtype=DataType.QAsymmU8, w_offset=151, w_std=70.0), True),
    ("u8_3x3_s2_rgb_fits", dict(n=2, h=32, w=32, ci=3, co=32, kh=3, kw=3, stride=(2, 2), w_dtype=DataType.QAsymmU8, w_offset=128, w_std=30.0), False),
    ("u8_7x7_s2_rgb", dict(n=1, h=40, w=40, ci=3, co=64, kh=7, kw=7, stride=(2, 2), w_dtype=DataType.QAsymmU8, w_offset=60, w_std=70.0), True),
    ("s8_5x5_grey", dict(n=3, h=21, w=19, ci=1, co=8, kh=5, kw=5, stride=(1, 1), w_dtype=DataType.QAsymmS8, w_offset=-50, w_std=70.0), True),
    ("s8_1x1_rgba", dict(n=2, h=16, w=16, ci=4, co=16, kh=1, kw=1, stride=(1, 1), w_dtype=DataType.QAsymmS8, w_offset=9, w_std=20.0), False),
]


@pytest.mark.parametrize("in_u8", [False, True], ids=["s8_in", "u8_in"])
@pytest.mark.parametrize("name,kw,halves", _ZP_STEMS, ids=[n for n, _, _ in _ZP_STEMS])
def test_stem_weights_with_a_zero_point(port, name, kw, halves, in_u8):
    """Convolutions with at most 4 input channels whose per-tensor weights have a zero point stay on the v_dot4 stem kernel."""
    seed = 34000 + 5 * [n for n, _, _ in _ZP_STEMS].index(name) + int(in_u8)
    case = cases.make_conv_case(name, seed, padding="same", per_axis=False, in_dtype=DataType.QAsymmU8 if in_u8 else DataType.QAsymmS8,
                                in_offset=128 if in_u8 else -1, out_offset=0 if in_u8 else -128, act=(2, 6.0, 0.0), **kw)
    fn, a, b = case.act
    plan = shim.Conv2dPlan(case.x.info, case.w, case.b, case.out_info, activation=fn, act_a=a, act_b=b, algo=shim.ALGO_AUTO, **case.params)
    algo, desc = plan.algo()
    plan.destroy()
    print(f"{name}: x={case.x.info.shape} zw={case.w.info.offset} kernel: {desc}", flush=True)
    assert algo == shim.ALGO_DOT4
    assert ("two int8 halves" in desc) == halves
    want = _oracle_conv(port, case)
    auto = _gpu_conv(case, shim.ALGO_AUTO)
    mx, exact = lsb_diff(auto.data, want.data)
    print(f"  max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    np.testing.assert_array_equal(auto.data, _gpu_conv(case, shim.ALGO_DIRECT).data)


@pytest.mark.parametrize("c", [16, 48, 80, 144])
@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("w_kind", ["per_axis", "u8_zero_point"])
def test_depthwise_channel_counts_that_are_odd_multiples_of_16(port, c, stride, w_kind):
    """The 3x3 depthwise kernel works in blocks of 32 channels; a tensor with 16 more gets a last block that is half padding."""
    kw = dict(per_axis=True) if w_kind == "per_axis" else dict(per_axis=False, w_dtype=DataType.QAsymmU8, w_offset=101, w_std=70.0)
    case = cases.make_conv_case(f"dw_c{c}", 35000 + c + stride, n=3, h=19, w=21, ci=c, kh=3, kw=3, stride=(stride, stride), padding="same",
                                depthwise=True, in_dtype=DataType.QAsymmU8, in_offset=121, out_offset=4, act=(2, 6.0, 0.0), **kw)
    fn, a, b = case.act
    plan = shim.Conv2dPlan(case.x.info, case.w, case.b, case.out_info, activation=fn, act_a=a, act_b=b, algo=shim.ALGO_AUTO, **case.params)
    desc = plan.algo()[1]
    plan.destroy()
    print(f"c={c} stride={stride} {w_kind}: {desc}", flush=True)
    assert "depthwise3x3_mfma" in desc
    want = _oracle_conv(port, case)
    auto = _gpu_conv(case, shim.ALGO_AUTO)
    mx, exact = lsb_diff(auto.data, want.data)
    print(f"  max|d|={mx} exact={exact:.5f}", flush=True)
    assert mx <= 1 and exact >= 0.99
    np.testing.assert_array_equal(auto.data, _gpu_conv(case, shim.ALGO_DIRECT).data)
