"""GPU parity of the convolution entry points (implicit GEMM, fused Winograd, dispatcher, requantised int8) against the CPU
oracle on identical seeded inputs, through the C API.  Bars: int8 bit-exact; fp32 implicit GEMM rel-L2 <= 1e-5; fp32 Winograd
<= 1e-4; fp16 / bf16 <= 2e-3."""
import ctypes as C

import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu

BAR = {"f32": 1e-5, "f16": 2e-3, "bf16": 2e-3}


@pytest.fixture(autouse=True, params=["wavefront_tiles", "workgroup_tiles"])
def tiling(request):
    """Every test runs twice: with the kernel that gives each wavefront one 32 x 32 tile forced for whatever it can run
    (the launcher itself picks it for problems small in tiles and short in k), and with that kernel switched off, so that
    the same geometry goes through the 128 x 128 gather kernel, the image-tile kernel or the few-channel kernels."""
    lib = cb.load_library()
    lib.avhip_set_small_problem_threshold.restype = int
    previous = lib.avhip_set_small_problem_threshold(-1 if request.param == "wavefront_tiles" else 0)
    yield request.param
    lib.avhip_set_small_problem_threshold(previous)


def he(g, shape, dtype, orc):
    K, R, S, Cin = shape
    return h.rounded(orc, g.standard_normal(shape) * np.sqrt(2.0 / (R * S * Cin)), dtype)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_implicit_gemm_config1(oracle, dtype):
    """BASELINE config 1: N=8, 15x15, 64->64, 3x3 offset -1, bias U(-0.1,0.1), ReLU."""
    g = h.rng(20)
    x = h.rounded(oracle, g.standard_normal((8, 15, 15, 64)), dtype)
    w = he(g, (64, 3, 3, 64), dtype, oracle)
    b = g.uniform(-0.1, 0.1, 64).astype(np.float32).astype(np.float64)
    got = h.conv_forward("implicit_gemm", x, w, (8, 15, 15, 64), dtype, bias=b, activation=cb.ACTIVATION_RELU)
    want = oracle.conv2d(x, w, b, activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("implicit gemm %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR[dtype]


CASES = [
    # x shape, w shape, pad, stride, dilation, mode
    dict(x=(3, 13, 14, 135), w=(21, 3, 3, 135), pad=(-1, -1)),                                   # odd everything, scalar tails
    dict(x=(2, 12, 12, 32), w=(40, 5, 5, 32), pad=(-2, -2)),                                     # 5x5 "same"
    dict(x=(2, 11, 13, 48), w=(24, 1, 1, 48), pad=(0, 0)),                                       # pointwise
    dict(x=(2, 16, 16, 32), w=(48, 3, 3, 32), pad=(-1, -1), stride=(2, 2)),                       # downsampling
    dict(x=(2, 15, 15, 16), w=(20, 3, 3, 16), pad=(-2, -2), dilation=(2, 2)),                     # dilated
    dict(x=(2, 10, 9, 24), w=(36, 3, 3, 24), pad=(-1, -1), mode=1),                               # cross-correlation mode flips the kernel
    dict(x=(2, 9, 10, 4), w=(32, 3, 3, 4), pad=(-1, -1)),                                         # 4 input planes (tower stem)
    dict(x=(2, 8, 8, 160), w=(136, 3, 3, 160), pad=(-1, -1)),                                     # more than one filter block
    dict(x=(1, 9, 11, 20), w=(8, 3, 2, 20), pad=(-1, 0)),                                         # non-square filter, asymmetric offsets
]


def out_shape(orc, c):
    N, H, W, _ = c["x"]
    K, R, S, _ = c["w"]
    Ho, Wo = orc.conv_output_shape(H, W, R, S, c["pad"], c.get("stride", (1, 1)), c.get("dilation", (1, 1)))
    return (N, Ho, Wo, K)


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_implicit_gemm_geometry(oracle, dtype, case):
    g = h.rng(21)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, **kw)
    want = oracle.conv2d(x, w, **kw)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < BAR[dtype]


FEW_CHANNELS = [
    dict(x=(3, 15, 15, 4), w=(128, 3, 3, 4), pad=(-1, -1)),                                       # the tower's stem
    dict(x=(2, 9, 10, 3), w=(24, 3, 3, 3), pad=(-1, -1)),                                         # RGB
    dict(x=(2, 9, 10, 1), w=(24, 5, 5, 1), pad=(-2, -2), mode=1),                                 # one plane, flipped 5x5
    dict(x=(2, 11, 9, 2), w=(8, 3, 3, 2), pad=(-1, -1), stride=(2, 1)),
    dict(x=(2, 12, 12, 8), w=(40, 3, 3, 8), pad=(-2, -2), dilation=(2, 2)),
    dict(x=(2, 8, 9, 12), w=(136, 3, 3, 12), pad=(-1, -1)),                                       # k spans several steps, two filter blocks
    dict(x=(1, 7, 7, 16), w=(16, 5, 5, 16), pad=(-2, -2)),
    dict(x=(1, 7, 7, 5), w=(16, 3, 3, 5), pad=(0, 0)),                                            # valid convolution, odd channel count
    # 8-byte pixels (4 channels of a 16-bit type, 8 of int8) and at most 12 taps: the register-operand stem kernel
    dict(x=(2, 13, 11, 4), w=(72, 3, 3, 4), pad=(-1, -1), mode=1),                                # flipped, second filter block partial
    dict(x=(2, 14, 12, 4), w=(40, 2, 5, 4), pad=(0, -2), stride=(2, 1)),                          # ten taps, strided
    dict(x=(2, 12, 12, 4), w=(16, 3, 4, 4), pad=(-2, -3), dilation=(2, 2)),                       # twelve taps, dilated
    dict(x=(2, 13, 11, 8), w=(72, 3, 3, 8), pad=(-1, -1), mode=1),
    dict(x=(3, 14, 12, 8), w=(48, 4, 3, 8), pad=(-1, -1), stride=(1, 2)),
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", FEW_CHANNELS, ids=[str(i) for i in range(len(FEW_CHANNELS))])
def test_implicit_gemm_few_input_channels(oracle, dtype, case):
    """First-layer shapes: (tap, channel) packed into the k-steps; bias, residual and ReLU fused as in the tower."""
    g = h.rng(26)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, **kw)
    want = oracle.conv2d(x, w, b, z, activation=oracle.RELU, **kw)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < BAR[dtype]


@pytest.mark.parametrize("case", FEW_CHANNELS, ids=[str(i) for i in range(len(FEW_CHANNELS))])
def test_int8_few_input_channels_bit_exact(oracle, case):
    g = h.rng(27)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, case["w"][0]).astype(np.int32)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    got = h.conv_forward("implicit_gemm", x, w, out_shape(oracle, case), "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, **kw)
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, b, activation=cb.ACTIVATION_RELU, **kw))


# ---- filter counts that are not a multiple of four: branch-free loaders, element-wise stores -------------------------------------
ODD_FILTER_COUNTS = [
    dict(x=(2, 20, 21, 64), w=(21, 1, 1, 64), pad=(0, 0)),                                        # 21 classes
    dict(x=(2, 13, 13, 128), w=(255, 1, 1, 128), pad=(0, 0)),                                     # 3 x 85 box values, two filter blocks
    dict(x=(2, 17, 18, 64), w=(3, 3, 3, 64), pad=(-1, -1)),                                       # an image out
    dict(x=(2, 12, 14, 96), w=(35, 3, 3, 96), pad=(-1, -1), stride=(2, 1), mode=1),
    dict(x=(1, 10, 10, 32), w=(130, 5, 5, 32), pad=(-4, -4), dilation=(2, 2)),
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", ODD_FILTER_COUNTS, ids=[str(i) for i in range(len(ODD_FILTER_COUNTS))])
def test_odd_filter_counts(oracle, dtype, case):
    g = h.rng(44)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, **kw)
    want = oracle.conv2d(x, w, b, z, activation=oracle.RELU, **kw)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < BAR[dtype]
    # every filter separately: the last ones are the ones a vector store would get wrong
    per_filter = [oracle.rel_l2(got[..., k], want[..., k]) for k in range(ys[3])]
    assert max(per_filter) < 4 * BAR[dtype], int(np.argmax(per_filter))


@pytest.mark.parametrize("case", ODD_FILTER_COUNTS, ids=[str(i) for i in range(len(ODD_FILTER_COUNTS))])
def test_odd_filter_counts_int8_bit_exact(oracle, case):
    g = h.rng(45)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    K = case["w"][0]
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    ys = out_shape(oracle, case)
    got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, **kw)
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, b, activation=cb.ACTIVATION_RELU, **kw))
    scale = g.uniform(1e-4, 1e-3, K).astype(np.float32)
    got = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=cb.ACTIVATION_LINEAR, **kw)
    np.testing.assert_array_equal(got, oracle.requant_i8(oracle.conv2d_i8(x, w, b, **kw), scale))


# ---- few input channels, images large enough for 256-pixel tiles: the kernel that gathers its operand from a tile in LDS ------
THIN_CASES = [
    dict(x=(2, 40, 48, 3), w=(72, 7, 7, 3), pad=(-3, -3), stride=(2, 2)),                         # a residual network's first layer; the second filter block partial
    dict(x=(2, 33, 35, 3), w=(64, 5, 5, 3), pad=(-2, -2), mode=1),                                # flipped; partial tiles at both edges
    dict(x=(1, 50, 20, 1), w=(16, 9, 9, 1), pad=(-4, -4)),                                        # 81 taps of one plane
    dict(x=(2, 24, 40, 6), w=(32, 3, 5, 6), pad=(-2, -4), dilation=(2, 2)),                       # dilated
    dict(x=(2, 30, 30, 16), w=(40, 3, 3, 16), pad=(-1, -1), stride=(1, 2)),                       # whole 16-byte pieces
    dict(x=(3, 20, 20, 5), w=(24, 4, 4, 5), pad=(-1, -2)),                                        # odd channel count, even filter
    dict(x=(2, 70, 9, 4), w=(136, 7, 3, 4), pad=(-3, -1), stride=(3, 1), mode=1),                 # tall images, three filter blocks
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", THIN_CASES, ids=[str(i) for i in range(len(THIN_CASES))])
def test_thin_kernel_with_residual(oracle, dtype, case):
    g = h.rng(28)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    y0 = h.rounded(oracle, g.standard_normal(ys), dtype)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, **kw)
    want = oracle.conv2d(x, w, **kw)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < BAR[dtype]
    # every image separately: a tile that went to the wrong place would hide in a global norm
    assert max(oracle.rel_l2(got[i], want[i]) for i in range(ys[0])) < 2 * BAR[dtype]
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, activation=cb.ACTIVATION_RELU, **kw)
    assert oracle.rel_l2(got, oracle.conv2d(x, w, b, activation=oracle.RELU, **kw)) < BAR[dtype]
    a2, be = float(np.float32(0.7)), float(np.float32(0.3))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, y0=y0, alpha2=a2, beta=be, activation=cb.ACTIVATION_RELU, **kw)
    want = oracle.conv2d(x, w, b, z, y0, alpha2=a2, beta=be, activation=oracle.RELU, **kw)
    assert oracle.rel_l2(got, want) < BAR[dtype]


@pytest.mark.parametrize("case", THIN_CASES, ids=[str(i) for i in range(len(THIN_CASES))])
def test_thin_kernel_int8_bit_exact(oracle, case):
    g = h.rng(29)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    K = case["w"][0]
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    ys = out_shape(oracle, case)
    got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, **kw)
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, b, activation=cb.ACTIVATION_RELU, **kw))
    scale = g.uniform(1e-4, 1e-3, K).astype(np.float32)
    got = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=cb.ACTIVATION_LINEAR, **kw)
    np.testing.assert_array_equal(got, oracle.requant_i8(oracle.conv2d_i8(x, w, b, **kw), scale))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_implicit_gemm_full_epilogue(oracle, dtype):
    """alpha1, alpha2, beta, bias, residual and every activation, in the order of the reference's epilogue
    (src/winograd_nonfused.cu:407-417)."""
    g = h.rng(22)
    x = h.rounded(oracle, g.standard_normal((2, 9, 9, 32)), dtype)
    w = he(g, (24, 3, 3, 32), dtype, oracle)
    b = g.uniform(-0.1, 0.1, 24).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((2, 9, 9, 24)), dtype)
    y0 = h.rounded(oracle, g.standard_normal((2, 9, 9, 24)), dtype)
    a1, a2, be = float(np.float32(1.1)), float(np.float32(1.2)), float(np.float32(0.1))
    for act in range(9):
        got = h.conv_forward("implicit_gemm", x, w, y0.shape, dtype, bias=b, z=z, y0=y0, alpha1=a1, alpha2=a2, beta=be, activation=act)
        want = oracle.conv2d(x, w, b, z, y0, alpha1=a1, alpha2=a2, beta=be, activation=act)
        # EXPONENTIAL multiplies the relative error of its argument by |argument| (up to ~4 here), on top of the bf16
        # output-rounding floor of 1.65e-3, so it gets twice the bar; fp32 gets 3x for the same amplification
        slack = 3 if dtype == "f32" else (2 if act == cb.ACTIVATION_EXPONENTIAL else 1)
        assert oracle.rel_l2(got, want) < BAR[dtype] * slack, act


def test_implicit_gemm_padding_value(oracle):
    g = h.rng(23)
    x = h.rounded(oracle, g.standard_normal((2, 7, 8, 32)), "f32")
    w = he(g, (16, 3, 3, 32), "f32", oracle)
    got = h.conv_forward("implicit_gemm", x, w, (2, 7, 8, 16), "f32", padding_value=0.5)
    want = oracle.conv2d(x, w, padding_value=0.5)
    assert oracle.rel_l2(got, want) < 1e-5


# ---- the image-tile kernel: shapes that fill at least half of its 256-row tiles ----------------------------------------------
TILE_CASES = [
    dict(x=(3, 15, 15, 160), w=(72, 3, 3, 160), pad=(-1, -1)),            # several channel slices, the last partial; two filter blocks
    dict(x=(2, 14, 13, 64), w=(64, 3, 3, 64), pad=(-1, -1), mode=1),      # flipped 3x3
    dict(x=(2, 20, 21, 96), w=(40, 3, 3, 96), pad=(-1, -1)),              # several tiles per image, partial ones at the edges
    dict(x=(2, 16, 15, 32), w=(16, 3, 3, 32), pad=(-2, -2)),              # full convolution: output larger than input
    dict(x=(2, 15, 15, 64), w=(32, 5, 5, 64), pad=(-2, -2)),              # the general k loop (not 3x3)
    dict(x=(2, 15, 14, 72), w=(24, 3, 1, 72), pad=(-1, 0), mode=1),       # three taps only, flipped
    dict(x=(3, 32, 32, 64), w=(64, 5, 5, 64), pad=(-2, -2)),              # 8 x 32 tiles in dense row order, large-halo LDS layout
    dict(x=(2, 37, 41, 24), w=(40, 5, 5, 24), pad=(-2, -2), mode=1),      # the same with partial tiles at both edges, flipped
    dict(x=(2, 30, 50, 16), w=(24, 7, 7, 16), pad=(-3, -3)),              # 7 x 7
    dict(x=(2, 19, 70, 32), w=(16, 1, 7, 32), pad=(0, -3)),               # one line of seven taps over a wide image
    dict(x=(2, 40, 24, 32), w=(16, 5, 3, 32), pad=(-2, -1)),              # dense order in the usual LDS layout
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", TILE_CASES, ids=[str(i) for i in range(len(TILE_CASES))])
def test_tile_kernel_with_residual(oracle, dtype, case):
    """Bias, residual (alpha2 != 1) and ReLU fused, and then the same with beta != 0 on top."""
    g = h.rng(40)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    y0 = h.rounded(oracle, g.standard_normal(ys), dtype)
    kw = dict(pad=case["pad"], mode=case.get("mode", 0))
    a2 = float(np.float32(0.7))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, alpha2=a2, activation=cb.ACTIVATION_RELU, **kw)
    want = oracle.conv2d(x, w, b, z, alpha2=a2, activation=oracle.RELU, **kw)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < BAR[dtype]
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, **kw)
    assert oracle.rel_l2(got, oracle.conv2d(x, w, **kw)) < BAR[dtype]
    be = float(np.float32(0.3))
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, y0=y0, alpha2=a2, beta=be, activation=cb.ACTIVATION_RELU, **kw)
    want = oracle.conv2d(x, w, b, z, y0, alpha2=a2, beta=be, activation=oracle.RELU, **kw)
    assert oracle.rel_l2(got, want) < BAR[dtype]


@pytest.mark.parametrize("case", TILE_CASES, ids=[str(i) for i in range(len(TILE_CASES))])
def test_tile_kernel_int8_bit_exact(oracle, case):
    g = h.rng(41)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    K = case["w"][0]
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    kw = dict(pad=case["pad"], mode=case.get("mode", 0))
    ys = out_shape(oracle, case)
    got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, **kw)
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, b, activation=cb.ACTIVATION_RELU, **kw))
    if case.get("mode", 0) == 0:
        scale = g.uniform(1e-4, 1e-3, K).astype(np.float32)
        got = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=cb.ACTIVATION_LINEAR, pad=case["pad"])
        np.testing.assert_array_equal(got, oracle.requant_i8(oracle.conv2d_i8(x, w, b, pad=case["pad"]), scale))


WALK_CASES = [
    # more (image, tile) pairs than workgroups stay resident: several rounds of workgroups, several filter blocks
    dict(x=(48, 30, 30, 32), w=(136, 3, 3, 32), pad=(-1, -1)),       # 3 filter blocks, 5 tiles per image, a partial last round
    dict(x=(130, 15, 15, 64), w=(200, 3, 3, 64), pad=(-1, -1)),      # 4 filter blocks, one whole-image tile each
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", WALK_CASES, ids=[str(i) for i in range(len(WALK_CASES))])
def test_tile_kernel_many_tiles(oracle, tiling, dtype, case):
    if tiling != "workgroup_tiles":
        pytest.skip("same kernel either way: the shape is far above the small-problem threshold")
    g = h.rng(42)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, pad=case["pad"])
    want = oracle.conv2d(x, w, b, z, activation=oracle.RELU, pad=case["pad"])
    assert oracle.rel_l2(got, want) < BAR[dtype]
    # every image separately: a tile that went to the wrong place would hide in a global norm
    per_image = [oracle.rel_l2(got[i], want[i]) for i in range(ys[0])]
    assert max(per_image) < 2 * BAR[dtype], int(np.argmax(per_image))


@pytest.mark.parametrize("case", WALK_CASES, ids=[str(i) for i in range(len(WALK_CASES))])
def test_tile_kernel_many_tiles_int8(oracle, tiling, case):
    if tiling != "workgroup_tiles":
        pytest.skip("same kernel either way")
    g = h.rng(43)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    K = case["w"][0]
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    ys = out_shape(oracle, case)
    got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, pad=case["pad"])
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, b, activation=cb.ACTIVATION_RELU, pad=case["pad"]))
    scale = g.uniform(1e-4, 1e-3, K).astype(np.float32)
    got = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=cb.ACTIVATION_LINEAR, pad=case["pad"])
    np.testing.assert_array_equal(got, oracle.requant_i8(oracle.conv2d_i8(x, w, b, pad=case["pad"]), scale))


# ---- fused Winograd F(2x2, 3x3) ------------------------------------------------------------------------------------------
WINOGRAD_BAR = {"f32": 1e-4, "f16": 2e-3, "bf16": 2e-3}

FUSED_CASES = [
    dict(x=(8, 15, 15, 64), w=(64, 3, 3, 64), pad=(-1, -1)),        # config 1
    dict(x=(2, 13, 14, 40), w=(21, 3, 3, 40), pad=(-1, -1)),        # odd extents, ragged filters (scalar stores)
    dict(x=(1, 33, 35, 32), w=(32, 3, 3, 32), pad=(-1, -1)),        # several tile blocks per image, partial ones at the edges
    dict(x=(2, 9, 9, 136), w=(136, 3, 3, 136), pad=(-1, -1)),       # more than one channel block and more than one filter block
    dict(x=(2, 12, 11, 32), w=(48, 3, 3, 32), pad=(0, 0)),          # valid convolution: output smaller than input
    dict(x=(2, 6, 7, 32), w=(32, 3, 3, 32), pad=(-2, -2)),          # full convolution: output larger than input
    dict(x=(2, 10, 10, 48), w=(40, 3, 3, 48), pad=(-1, -1), mode=1),  # kernel rotated by 180 degrees
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", FUSED_CASES, ids=[str(i) for i in range(len(FUSED_CASES))])
def test_winograd_fused_geometry(oracle, dtype, case):
    g = h.rng(30)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    kw = dict(pad=case["pad"], mode=case.get("mode", 0))
    got = h.conv_forward("winograd_fused", x, w, ys, dtype, bias=b, activation=cb.ACTIVATION_RELU, **kw)
    want = oracle.conv2d(x, w, b, activation=oracle.RELU, **kw)
    assert got.shape == want.shape
    err = oracle.rel_l2(got, want)
    print("fused winograd %s case %s rel-L2 = %.3e" % (dtype, case["x"], err))
    assert err < WINOGRAD_BAR[dtype]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_winograd_fused_full_epilogue(oracle, dtype):
    g = h.rng(31)
    x = h.rounded(oracle, g.standard_normal((2, 9, 9, 32)), dtype)
    w = he(g, (24, 3, 3, 32), dtype, oracle)
    b = g.uniform(-0.1, 0.1, 24).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((2, 9, 9, 24)), dtype)
    y0 = h.rounded(oracle, g.standard_normal((2, 9, 9, 24)), dtype)
    a1, a2, be = float(np.float32(1.1)), float(np.float32(1.2)), float(np.float32(0.1))
    for act in range(9):
        got = h.conv_forward("winograd_fused", x, w, y0.shape, dtype, bias=b, z=z, y0=y0, alpha1=a1, alpha2=a2, beta=be, activation=act)
        want = oracle.conv2d(x, w, b, z, y0, alpha1=a1, alpha2=a2, beta=be, activation=act)
        slack = 2 if act == cb.ACTIVATION_EXPONENTIAL else 1  # see test_implicit_gemm_full_epilogue
        assert oracle.rel_l2(got, want) < WINOGRAD_BAR[dtype] * slack, act


def test_winograd_fused_sees_rewritten_weights(oracle):
    """The transformed weights are cached per memory block and version: a second call after the weights were overwritten
    through the API must use the new ones."""
    g = h.rng(32)
    x = h.rounded(oracle, g.standard_normal((1, 8, 8, 32)), "f32")
    w1 = he(g, (32, 3, 3, 32), "f32", oracle)
    w2 = he(g, (32, 3, 3, 32), "f32", oracle)
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=cb.DTYPE_FLOAT32)
        xt, wt, y = c.tensor(x, "f32"), c.tensor(w1, "f32"), c.empty((1, 8, 8, 32), "f32")

        def run():
            st = c.lib.cudaConvolutionWinogradFusedForward(c.ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, 0, 0, None, 0, 0, None,
                                                           y.desc, y.mem, cb.ACTIVATION_LINEAR)
            assert st == cb.STATUS_SUCCESS
            c.finish()
            return y.download()
        first = run()
        wt.upload(w2)
        second = run()
    assert oracle.rel_l2(first, oracle.conv2d(x, w1)) < 1e-4
    assert oracle.rel_l2(second, oracle.conv2d(x, w2)) < 1e-4


# ---- int8 ------------------------------------------------------------------------------------------------------------
INT8_CASES = [
    dict(x=(4, 20, 20, 128), w=(128, 3, 3, 128), pad=(-1, -1)),      # config 4 at a reduced batch
    dict(x=(4, 20, 20, 128), w=(128, 1, 1, 128), pad=(0, 0)),
    dict(x=(2, 9, 11, 36), w=(20, 3, 3, 36), pad=(-1, -1)),          # channels not a multiple of the 64-byte step
    dict(x=(2, 12, 12, 64), w=(72, 3, 3, 64), pad=(-1, -1), stride=(2, 2)),
    dict(x=(2, 10, 10, 16), w=(8, 5, 5, 16), pad=(-2, -2), mode=1),
    dict(x=(1, 6, 6, 7), w=(5, 3, 3, 7), pad=(-1, -1)),              # unaligned rows: element-wise loads
]


@pytest.mark.parametrize("case", INT8_CASES, ids=[str(i) for i in range(len(INT8_CASES))])
def test_int8_int32_bit_exact(oracle, case):
    g = h.rng(24)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, case["w"][0]).astype(np.int32)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), mode=case.get("mode", 0))
    ys = out_shape(oracle, case)
    for act in (cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU):
        got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=act, **kw)
        want = oracle.conv2d_i8(x, w, b, activation=act, **kw)
        np.testing.assert_array_equal(got, want)
    got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", **kw)
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, None, **kw))


def test_int8_padding_value_bit_exact(oracle):
    g = h.rng(25)
    x = g.integers(-127, 128, (2, 8, 8, 32), dtype=np.int8)
    w = g.integers(-127, 128, (16, 3, 3, 32), dtype=np.int8)
    got = h.conv_forward("implicit_gemm", x, w, (2, 8, 8, 16), "i8", y_dtype="i32", padding_value=-3)
    np.testing.assert_array_equal(got, oracle.conv2d_i8(x, w, None, padding_value=-3))


@pytest.mark.parametrize("case", INT8_CASES[:3], ids=["3x3", "1x1", "ragged"])
def test_int8_requantised_bit_exact(oracle, case):
    """q = sat_i8(rne(float(sum + bias) * scale[k])), scale ~ U(1e-4, 1e-3) per output channel."""
    g = h.rng(26)
    x = g.integers(-127, 128, case["x"], dtype=np.int8)
    w = g.integers(-127, 128, case["w"], dtype=np.int8)
    K = case["w"][0]
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    scale = g.uniform(1e-4, 1e-3, K).astype(np.float32)
    ys = out_shape(oracle, case)
    for act in (cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU):
        got = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=act, pad=case["pad"])
        want = oracle.requant_i8(oracle.conv2d_i8(x, w, b, pad=case["pad"], activation=act), scale)
        np.testing.assert_array_equal(got, want)
    assert np.abs(want).max() > 20  # the scale range really exercises the int8 range


@pytest.mark.parametrize("y_dtype", ["i32", "i8", "f32"])
def test_int8_float_epilogue(oracle, y_dtype):
    """The header's convention for integer tensors: cast the int32 sum to fp32, scale and add in fp32, round to nearest even
    and saturate on store (include/Avocado/cuda_backend.h:43-49, src/conv2d_implicit_gemm.cu:278-286,330-338).  The oracle's
    sequence of single roundings is pinned by hand-written cases in test_oracle.py, so the comparison is exact for LINEAR / RELU."""
    g = h.rng(27)
    x = g.integers(-127, 128, (2, 6, 6, 64), dtype=np.int8)
    w = g.integers(-127, 128, (16, 3, 3, 64), dtype=np.int8)
    acc = oracle.conv2d_i8(x, w, None)
    bias = g.uniform(-100, 100, 16).astype(np.float32)
    np_dt = {"i32": np.int32, "i8": np.int8, "f32": np.float32}[y_dtype]
    z = g.integers(-100, 100, acc.shape).astype(np_dt)
    y0 = g.integers(-100, 100, acc.shape).astype(np_dt)
    a1 = float(np.float32(1e-4 if y_dtype == "i8" else 0.37))
    a2, be = float(np.float32(1.2)), float(np.float32(0.1))
    got = h.conv_forward("implicit_gemm", x, w, acc.shape, "i8", y_dtype=y_dtype, bias=bias, bias_dtype="f32", z=z, y0=y0, alpha1=a1, alpha2=a2,
                         beta=be, activation=cb.ACTIVATION_RELU)
    want = oracle.conv2d_i8_float_epilogue(acc, bias, z, y0.copy(), a1, a2, be, oracle.RELU)
    if y_dtype == "f32":
        np.testing.assert_array_equal(np.asarray(got, dtype=np.float32), want)
    else:
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("y_dtype", ["i32", "i8"])
def test_int8_float_epilogue_saturates(oracle, y_dtype):
    """Scaled sums beyond the integer range clamp to the type's extremes (INT32_MAX although fp32 cannot hold it), ties go to even."""
    g = h.rng(28)
    x = g.integers(-127, 128, (2, 5, 5, 32), dtype=np.int8)
    w = g.integers(-127, 128, (8, 3, 3, 32), dtype=np.int8)
    acc = oracle.conv2d_i8(x, w, None)
    np_dt = {"i32": np.int32, "i8": np.int8}[y_dtype]
    for a1 in (0.5, 1.0e5 if y_dtype == "i32" else 0.01):
        got = h.conv_forward("implicit_gemm", x, w, acc.shape, "i8", y_dtype=y_dtype, alpha1=a1)
        want = oracle.conv2d_i8_float_epilogue(acc, None, None, np.zeros(acc.shape, np_dt), a1, 1.0, 0.0, oracle.LINEAR)
        np.testing.assert_array_equal(got, want)
    info = np.iinfo(np_dt)
    assert want.max() == info.max and want.min() == info.min


# ---- dispatcher and argument checking -----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,tol", [("f32", 1e-4), ("f16", 2e-3), ("bf16", 2e-3)])
def test_dispatcher_config1(oracle, dtype, tol):
    g = h.rng(28)
    x = h.rounded(oracle, g.standard_normal((8, 15, 15, 64)), dtype)
    w = he(g, (64, 3, 3, 64), dtype, oracle)
    b = g.uniform(-0.1, 0.1, 64).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((8, 15, 15, 64)), dtype)
    got = h.conv_forward("dispatch", x, w, (8, 15, 15, 64), dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU)
    want = oracle.conv2d(x, w, b, z, activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("dispatcher %s rel-L2 = %.3e" % (dtype, err))
    assert err < tol


def test_dispatcher_without_workspace_falls_back(oracle):
    g = h.rng(29)
    x = h.rounded(oracle, g.standard_normal((2, 15, 15, 64)), "f32")
    w = he(g, (64, 3, 3, 64), "f32", oracle)
    got = h.conv_forward("dispatch", x, w, (2, 15, 15, 64), "f32", workspace_bytes=0)
    assert oracle.rel_l2(got, oracle.conv2d(x, w)) < 1e-4
    # stride 2 and int8 never use Winograd
    got = h.conv_forward("dispatch", x, w, (2, 8, 8, 64), "f32", stride=(2, 2))
    assert oracle.rel_l2(got, oracle.conv2d(x, w, stride=(2, 2))) < 1e-5
    xi = g.integers(-127, 128, (2, 6, 6, 64), dtype=np.int8)
    wi = g.integers(-127, 128, (8, 3, 3, 64), dtype=np.int8)
    got = h.conv_forward("dispatch", xi, wi, (2, 6, 6, 8), "i8", y_dtype="i32")
    np.testing.assert_array_equal(got, oracle.conv2d_i8(xi, wi, None))


def test_dispatcher_large_fp32_layer_takes_workspace_and_sees_rewritten_weights(oracle):
    """A large fp32 3x3 layer asks for a workspace ([V | M] of non-fused F(4x4,3x3)) and, given it, runs the three-pass plan
    with weights transformed once and cached per memory block and version: overwriting the weights through the API must show
    in the next call; without the workspace the same call still succeeds (fused kernel)."""
    g = h.rng(33)
    N, H, W, Cin, K = 40, 15, 15, 64, 64       # 40 x 4 x 4 = 640 tiles of 4 x 4 ... below the threshold
    x = h.rounded(oracle, g.standard_normal((N, H, W, Cin)), "f32")
    w1, w2 = he(g, (K, 3, 3, Cin), "f32", oracle), he(g, (K, 3, 3, Cin), "f32", oracle)
    b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    got = h.conv_forward("dispatch", x, w1, (N, H, W, K), "f32", bias=b, activation=cb.ACTIVATION_RELU)
    assert oracle.rel_l2(got, oracle.conv2d(x, w1, b, activation=oracle.RELU)) < 1e-4
    N = 136                                    # 136 x 16 = 2176 tiles: the non-fused plan is preferred
    x = h.rounded(oracle, g.standard_normal((N, H, W, Cin)), "f32")
    z = h.rounded(oracle, g.standard_normal((N, H, W, K)), "f32")
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=cb.DTYPE_FLOAT32)
        xt, wt, bt, zt, y = c.tensor(x, "f32"), c.tensor(w1, "f32"), c.tensor(b, "f32"), c.tensor(z, "f32"), c.empty((N, H, W, K), "f32")
        need = h.C.c_int64(0)
        cb.check(c.lib.cudaGetConvolutionWorkspaceSize(c.ctx.handle, conv.handle, xt.desc, wt.desc, bt.desc, h.C.byref(need)), "workspace size")
        tiles = N * 4 * 4
        assert need.value >= 36 * tiles * (Cin + K) * 4
        ws = c.empty((need.value,), cb.DTYPE_UINT8)

        def run(workspace):
            st = c.lib.cudaConvolutionBiasActivationForward(c.ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, bt.desc, bt.mem, None,
                                                            zt.desc, zt.mem, None, y.desc, y.mem, cb.ACTIVATION_RELU, workspace)
            assert st == cb.STATUS_SUCCESS
            c.finish()
            return y.download()
        first = run(ws.mem)
        wt.upload(w2)
        second = run(ws.mem)
        third = run(0)
    want2 = oracle.conv2d(x, w2, b, z, activation=oracle.RELU)
    assert oracle.rel_l2(first, oracle.conv2d(x, w1, b, z, activation=oracle.RELU)) < 1e-4
    assert oracle.rel_l2(second, want2) < 1e-4
    assert oracle.rel_l2(third, want2) < 1e-4


def test_convolution_argument_errors(oracle):
    x = np.zeros((2, 6, 6, 8))
    w = np.zeros((4, 3, 3, 8))
    h.conv_forward("implicit_gemm", x, w, (2, 6, 6, 5), "f32", expect=cb.STATUS_BAD_PARAM)              # K mismatch
    h.conv_forward("implicit_gemm", x, np.zeros((4, 3, 3, 7)), (2, 6, 6, 4), "f32", expect=cb.STATUS_BAD_PARAM)   # C mismatch
    h.conv_forward("implicit_gemm", x, w, (2, 6, 6, 4), "f32", groups=2, expect=cb.STATUS_NOT_SUPPORTED)
    h.conv_forward("implicit_gemm", x, w, (2, 6, 6, 4), "f64", expect=cb.STATUS_UNSUPPORTED_DATATYPE)
    h.conv_forward("implicit_gemm", x, w, (2, 20, 20, 4), "f32", expect=cb.STATUS_BAD_PARAM)            # output larger than any window grid
    # an empty batch is refused, not skipped (the reference's launch with a zero-sized grid fails as well)
    h.conv_forward("implicit_gemm", np.zeros((0, 6, 6, 8)), w, (0, 6, 6, 4), "f32", expect=cb.STATUS_BAD_PARAM)
    h.conv_forward("winograd_fused", x, np.zeros((4, 5, 5, 8)), (2, 6, 6, 4), "f32", pad=(-2, -2), expect=cb.STATUS_NOT_SUPPORTED)


# ---- few output pixels, long k: the dispatcher splits k across workgroups when the caller lends it a workspace -----------------
SPLIT_CASES = [
    dict(x=(4, 7, 7, 512), w=(512, 3, 3, 512), pad=(-1, -1)),                        # the last stage of a residual network
    dict(x=(8, 7, 7, 2048), w=(256, 1, 1, 2048), pad=(0, 0)),                        # 1x1, thirty-two k-steps
    dict(x=(2, 14, 14, 256), w=(256, 3, 3, 256), pad=(-1, -1), stride=(2, 2)),       # strided
    dict(x=(3, 9, 8, 160), w=(72, 3, 3, 160), pad=(-1, -1), mode=1),                 # the last part of k shorter and odd; flipped; partial tiles
    dict(x=(2, 6, 6, 192), w=(40, 5, 5, 192), pad=(-2, -2), dilation=(1, 2)),        # 25 taps, dilated
]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", SPLIT_CASES, ids=[str(i) for i in range(len(SPLIT_CASES))])
def test_split_k_through_the_dispatcher(oracle, tiling, dtype, case):
    if tiling != "workgroup_tiles":
        pytest.skip("with the one-wavefront-per-tile kernel available the plan leaves layers this small to it")
    g = h.rng(43)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    y0 = h.rounded(oracle, g.standard_normal(ys), dtype)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    # the workspace query names the plan: partial sums of at least two parts
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(mode=kw["mode"], padding=kw["pad"], strides=kw["stride"], dilation=kw["dilation"], dtype=h.DT[dtype])
        xt, wt = c.tensor(x, dtype), c.tensor(w, dtype)
        need = C.c_int64(0)
        cb.check(c.lib.cudaGetConvolutionWorkspaceSize(c.ctx.handle, conv.handle, xt.desc, wt.desc, 0, C.byref(need)), "workspace size")
    fused_winograd = dtype == "f32" and case["w"][1:3] == (3, 3) and "stride" not in case
    if not fused_winograd:
        assert need.value >= 2 * 4 * ys[0] * ys[1] * ys[2] * ys[3], need.value
    a2, be = float(np.float32(0.7)), float(np.float32(0.3))
    for act, oact in ((cb.ACTIVATION_RELU, oracle.RELU), (cb.ACTIVATION_TANH, oracle.TANH)):
        got = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, z=z, y0=y0, alpha2=a2, beta=be, activation=act, **kw)
        want = oracle.conv2d(x, w, b, z, y0, alpha2=a2, beta=be, activation=oact, **kw)
        assert got.shape == want.shape
        assert oracle.rel_l2(got, want) < BAR[dtype] * (3 if dtype == "f32" else 1)
    # without a workspace the plain kernels take the layer: the same result to rounding
    plain = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, workspace_bytes=0, **kw)
    split = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, **kw)
    assert oracle.rel_l2(split, plain) < BAR[dtype] * (3 if dtype == "f32" else 1)
    assert oracle.rel_l2(split, oracle.conv2d(x, w, b, **kw)) < BAR[dtype] * (3 if dtype == "f32" else 1)


class _Shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("N", "H", "W", "C", "K", "R", "S", "Ho", "Wo", "pad_h", "pad_w", "stride_h", "stride_w", "dil_h", "dil_w",
                                       "mode")]


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("case", SPLIT_CASES, ids=[str(i) for i in range(len(SPLIT_CASES))])
def test_split_k_kernel_layer_entry(oracle, tiling, dtype, case):
    """avhip_conv2d_implicit_gemm_split_k called directly: it must TAKE every one of these layers (return 0: the two split kernels ran,
    which the dispatcher test cannot tell from its fallback), and decline a workspace that is short or not aligned with nothing launched."""
    if tiling != "workgroup_tiles":
        pytest.skip("with the one-wavefront-per-tile kernel available the plan leaves layers this small to it")
    lib = cb.load_library()
    g = h.rng(44)
    x = h.rounded(oracle, g.standard_normal(case["x"]), dtype)
    w = he(g, case["w"], dtype, oracle)
    ys = out_shape(oracle, case)
    b = g.uniform(-0.1, 0.1, ys[3]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    kw = dict(pad=case["pad"], stride=case.get("stride", (1, 1)), dilation=case.get("dilation", (1, 1)), mode=case.get("mode", 0))
    xs, ws = case["x"], case["w"]
    s = _Shape(xs[0], xs[1], xs[2], xs[3], ws[0], ws[1], ws[2], ys[1], ys[2], kw["pad"][0], kw["pad"][1], kw["stride"][0], kw["stride"][1],
               kw["dilation"][0], kw["dilation"][1], kw["mode"])
    need = C.c_int64(0)
    assert lib.avhip_conv2d_split_k_workspace(h.DT[dtype], C.byref(s), C.byref(need)) == 0
    assert need.value >= 2 * 4 * ys[0] * ys[1] * ys[2] * ys[3], "partial sums of at least two parts"
    lib.avhip_conv2d_implicit_gemm_split_k.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                       C.c_double, C.c_double, C.c_double, C.c_int, C.c_void_p, C.c_int64]
    with h.Call() as c:
        xt, wt, zt, bt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(z, dtype), c.tensor(b, "f32")
        y = c.empty(ys, dtype)
        space = c.empty((need.value + 256,), cb.DTYPE_UINT8)
        stream = C.c_void_p(c.ctx.stream())
        args = (stream, h.DT[dtype], C.addressof(s), xt.pointer(), wt.pointer(), bt.pointer(), zt.pointer(), y.pointer(), None, 1.0, 0.7, 0.0, cb.ACTIVATION_RELU)
        assert lib.avhip_conv2d_implicit_gemm_split_k(*args, space.pointer(), need.value) == 0
        c.finish()
        got = y.download()
        assert lib.avhip_conv2d_implicit_gemm_split_k(*args, space.pointer(), need.value - 1) == -1, "short workspace"
        assert lib.avhip_conv2d_implicit_gemm_split_k(*args, space.pointer() + 4, need.value) == -1, "workspace not aligned for 16-byte accesses"
    want = oracle.conv2d(x, w, b, z, alpha2=float(np.float32(0.7)), activation=oracle.RELU, **kw)
    assert oracle.rel_l2(got, want) < BAR[dtype] * (3 if dtype == "f32" else 1)
