"""Parity at BASELINE's full sizes.  The CPU oracle cannot redo these in seconds, so every case combines
  (a) the oracle on a handful of whole images picked from the batch (images are independent in a forward convolution, so this
      is an exact check of those images at the real launch geometry: full grids, every tile position, 32-bit offset ranges), with
  (b) size-independent properties over the WHOLE output: invariance under a permutation of the batch (bit-exact), linearity in
      the weights and delta kernels (int8, bit-exact), agreement of independent kernels (Winograd vs implicit GEMM)."""
import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu

BAR = {"f32": 1e-5, "f16": 2e-3, "bf16": 2e-3}


def he(g, shape):
    K, R, S, Cin = shape
    return g.standard_normal(shape) * np.sqrt(2.0 / (R * S * Cin))


def check_images(oracle, got, x, w, b, z, images, bar, **kw):
    for n in images:
        want = oracle.conv2d(x[n:n + 1], w, b, None if z is None else z[n:n + 1], activation=oracle.RELU, **kw)
        err = oracle.rel_l2(got[n:n + 1], want)
        assert err < bar, "image %d: rel-L2 %.3e" % (n, err)


@pytest.mark.parametrize("dtype", ["bf16", "f32"])
def test_config2_body_convolution(oracle, dtype):
    """N=256, 15x15, 128->128, bias + residual + ReLU, through the dispatcher (what the tower calls)."""
    g = h.rng(40)
    N = 256
    x = h.rounded(oracle, g.standard_normal((N, 15, 15, 128)), dtype)
    w = h.rounded(oracle, he(g, (128, 3, 3, 128)), dtype)
    b = g.uniform(-0.1, 0.1, 128).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((N, 15, 15, 128)), dtype)
    got = h.conv_forward("dispatch", x, w, x.shape, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU)
    bar = 1e-4 if dtype == "f32" else BAR[dtype]  # the dispatcher runs fp32 through the fused Winograd kernel
    check_images(oracle, got, x, w, b, z, (0, 1, 100, 255), bar)
    perm = g.permutation(N)
    again = h.conv_forward("dispatch", x[perm], w, x.shape, dtype, bias=b, z=z[perm], activation=cb.ACTIVATION_RELU)
    np.testing.assert_array_equal(again, got[perm])
    if dtype == "f32":
        direct = h.conv_forward("implicit_gemm", x, w, x.shape, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU)
        check_images(oracle, direct, x, w, b, z, (0, 255), BAR["f32"])
        assert oracle.rel_l2(got, direct) < 1e-4


def test_config2_stem_and_nonfused_winograd(oracle):
    """Stem 4->128 on sparse 0/1 planes (bf16), and the four-call non-fused F(4x4,3x3) sequence on the fp32 body shape."""
    g = h.rng(41)
    N = 256
    x0 = (g.random((N, 15, 15, 4)) < 0.15).astype(np.float64)
    w0 = h.rounded(oracle, he(g, (128, 3, 3, 4)), "bf16")
    b = g.uniform(-0.1, 0.1, 128).astype(np.float32).astype(np.float64)
    got = h.conv_forward("dispatch", x0, w0, (N, 15, 15, 128), "bf16", bias=b, activation=cb.ACTIVATION_RELU)
    check_images(oracle, got, x0, w0, b, None, (0, 17, 255), BAR["bf16"])

    x = h.rounded(oracle, g.standard_normal((N, 15, 15, 128)), "f32")
    w = h.rounded(oracle, he(g, (128, 3, 3, 128)), "f32")
    U = h.winograd_weight_transform(w, "f32", 4)
    V = h.winograd_input_transform(x, w.shape, "f32", 4, (-1, -1))
    M = h.gemm(V, U, np.zeros((36, V.shape[1], 128)), "f32", opB=True, batched=True)
    y = h.winograd_output_transform(M, x.shape, w.shape, "f32", 4, bias=b, activation=cb.ACTIVATION_RELU)
    check_images(oracle, y, x, w, b, None, (0, 128, 255), 1e-4)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_config3_large_spatial(oracle, dtype):
    """N=64, 56x56, 256->256: implicit GEMM and fused Winograd against the oracle on sampled images, and against each other."""
    g = h.rng(42)
    N = 64
    x = h.rounded(oracle, g.standard_normal((N, 56, 56, 256)), dtype)
    w = h.rounded(oracle, he(g, (256, 3, 3, 256)), dtype)
    b = g.uniform(-0.1, 0.1, 256).astype(np.float32).astype(np.float64)
    direct = h.conv_forward("implicit_gemm", x, w, x.shape, dtype, bias=b, activation=cb.ACTIVATION_RELU)
    check_images(oracle, direct, x, w, b, None, (0, 63), BAR[dtype])
    fused = h.conv_forward("winograd_fused", x, w, x.shape, dtype, bias=b, activation=cb.ACTIVATION_RELU)
    check_images(oracle, fused, x, w, b, None, (31,), BAR[dtype])
    assert oracle.rel_l2(fused, direct) < 2 * BAR[dtype]


@pytest.mark.parametrize("dtype,m,mat,acc", [("bf16", 2, "f16", "f32"), ("f16", 2, "f16", "f32"), ("f16", 2, "f16", "f16"), ("bf16", 2, "f16", "f16"), ("bf16", 4, "f32", "f32"),
                                               ("f16", 4, "f32", "f32")])
def test_config3_nonfused_winograd(oracle, dtype, m, mat, acc):
    """N=64, 56x56, 256->256 as the four-call non-fused Winograd sequence (src/winograd_nonfused.cu:906,932, src/gemm.cpp:126-209 of
    the reference; call order of app/CudaBackend.cu:401-420), matrices resident on the device: F(2x2,3x3) with fp16 matrices (and
    fp16 M for fp16 tensors), F(4x4,3x3) with fp32 matrices, bias + ReLU fused in the output transform; sampled images against the
    oracle at the 16-bit bar 2e-3."""
    g = h.rng(45)
    N = 64
    x = h.rounded(oracle, g.standard_normal((N, 56, 56, 256)), dtype)
    w = h.rounded(oracle, he(g, (256, 3, 3, 256)), dtype)
    b = g.uniform(-0.1, 0.1, 256).astype(np.float32).astype(np.float64)
    print("config 3 non-fused", dtype, "F(%d,3)" % m, "matrices", mat, "M", acc, flush=True)
    got = h.winograd_nonfused(x, w, dtype, m, mat, acc, bias=b, activation=cb.ACTIVATION_RELU)
    check_images(oracle, got, x, w, b, None, (0, 37, 63), BAR[dtype])


def test_config4_int8(oracle):
    """N=128, 20x20, 128->128 int8: sampled images exact, requantised exact, linearity in the weights and delta kernels exact."""
    g = h.rng(43)
    N = 128
    x = g.integers(-127, 128, (N, 20, 20, 128), dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, 128).astype(np.int32)
    scale = g.uniform(1e-4, 1e-3, 128).astype(np.float32)
    for R, pad in ((3, (-1, -1)), (1, (0, 0))):
        w = g.integers(-127, 128, (128, R, R, 128), dtype=np.int8)
        got = h.conv_forward("implicit_gemm", x, w, (N, 20, 20, 128), "i8", y_dtype="i32", bias=b, bias_dtype="i32", pad=pad)
        for n in (0, 64, 127):
            np.testing.assert_array_equal(got[n:n + 1], oracle.conv2d_i8(x[n:n + 1], w, b, pad=pad))
        q = h.conv_forward("requant", x, w, (N, 20, 20, 128), "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, pad=pad)
        np.testing.assert_array_equal(q, oracle.requant_i8(got, scale))
        # linearity: conv(x, w1) + conv(x, w2) == conv(x, w1 + w2) in exact integer arithmetic (no bias)
        w1 = g.integers(-60, 61, w.shape, dtype=np.int8)
        w2 = g.integers(-60, 61, w.shape, dtype=np.int8)
        y1 = h.conv_forward("implicit_gemm", x, w1, (N, 20, 20, 128), "i8", y_dtype="i32", pad=pad)
        y2 = h.conv_forward("implicit_gemm", x, w2, (N, 20, 20, 128), "i8", y_dtype="i32", pad=pad)
        y12 = h.conv_forward("implicit_gemm", x, (w1 + w2).astype(np.int8), (N, 20, 20, 128), "i8", y_dtype="i32", pad=pad)
        np.testing.assert_array_equal(y1 + y2, y12)
    # delta kernel at tap (0, 0) of a 3x3 filter with offset -1: y[n, oh, ow, k] = 3 * x[n, oh - 1, ow - 1, k]
    wd = np.zeros((128, 3, 3, 128), dtype=np.int8)
    wd[np.arange(128), 0, 0, np.arange(128)] = 3
    yd = h.conv_forward("implicit_gemm", x, wd, (N, 20, 20, 128), "i8", y_dtype="i32")
    want = np.zeros((N, 20, 20, 128), dtype=np.int32)
    want[:, 1:, 1:, :] = 3 * x[:, :-1, :-1, :].astype(np.int32)
    np.testing.assert_array_equal(yd, want)


CONFIG5 = [
    dict(x=(64, 56, 56, 128), w=(256, 3, 3, 128), pad=(-1, -1), stride=(2, 2)),
    dict(x=(64, 28, 28, 256), w=(512, 1, 1, 256), pad=(0, 0), stride=(1, 1)),
    dict(x=(64, 32, 32, 64), w=(64, 5, 5, 64), pad=(-2, -2), stride=(1, 1)),
]


@pytest.mark.parametrize("case", CONFIG5, ids=["3x3s2", "1x1", "5x5"])
def test_config5_bf16(oracle, case):
    g = h.rng(44)
    x = h.rounded(oracle, g.standard_normal(case["x"]), "bf16")
    w = h.rounded(oracle, he(g, case["w"]), "bf16")
    K = case["w"][0]
    b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    Ho, Wo = oracle.conv_output_shape(case["x"][1], case["x"][2], case["w"][1], case["w"][2], case["pad"], case["stride"])
    got = h.conv_forward("dispatch", x, w, (case["x"][0], Ho, Wo, K), "bf16", bias=b, activation=cb.ACTIVATION_RELU, pad=case["pad"], stride=case["stride"])
    check_images(oracle, got, x, w, b, None, (0, 63), BAR["bf16"], pad=case["pad"], stride=case["stride"])
    perm = g.permutation(case["x"][0])
    again = h.conv_forward("dispatch", x[perm], w, got.shape, "bf16", bias=b, activation=cb.ACTIVATION_RELU, pad=case["pad"], stride=case["stride"])
    np.testing.assert_array_equal(again, got[perm])


LARGE_FILTER_CASES = [
    dict(x=(40, 37, 32, 64), w=(72, 5, 5, 64), pad=(-2, -2)),    # 5 x 5: dense 8 x 32 tiles in the large-halo layout, a partial last tile, a partial filter block
    dict(x=(48, 30, 33, 64), w=(64, 7, 7, 64), pad=(-3, -3)),    # 7 x 7
    dict(x=(96, 12, 70, 64), w=(64, 1, 9, 64), pad=(0, -4)),     # one line of nine taps over wide rows
]


@pytest.mark.parametrize("case", LARGE_FILTER_CASES, ids=["5x5", "7x7", "1x9"])
def test_large_filters_many_images(oracle, case):
    """Enough (image, tile) pairs that the image-tile kernel takes its layout with one workgroup per compute unit and tiles in
    dense row order; bf16 against the oracle on sampled images, int8 -> int32 bit-exact on the same images."""
    g = h.rng(47)
    K = case["w"][0]
    N = case["x"][0]
    images = (0, N // 2, N - 1)
    Ho, Wo = oracle.conv_output_shape(case["x"][1], case["x"][2], case["w"][1], case["w"][2], case["pad"])
    x = h.rounded(oracle, g.standard_normal(case["x"]), "bf16")
    w = h.rounded(oracle, he(g, case["w"]), "bf16")
    b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((N, Ho, Wo, K)), "bf16")
    got = h.conv_forward("implicit_gemm", x, w, (N, Ho, Wo, K), "bf16", bias=b, z=z, activation=cb.ACTIVATION_RELU, pad=case["pad"])
    check_images(oracle, got, x, w, b, z, images, BAR["bf16"], pad=case["pad"])
    xi = g.integers(-127, 128, case["x"], dtype=np.int8)
    wi = g.integers(-127, 128, case["w"], dtype=np.int8)
    bi = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    goti = h.conv_forward("implicit_gemm", xi, wi, (N, Ho, Wo, K), "i8", y_dtype="i32", bias=bi, bias_dtype="i32", activation=cb.ACTIVATION_RELU, pad=case["pad"])
    for n in images:
        np.testing.assert_array_equal(goti[n:n + 1], oracle.conv2d_i8(xi[n:n + 1], wi, bi, pad=case["pad"], activation=cb.ACTIVATION_RELU))


def test_written_out_5x5_int8_bit_exact(oracle):
    """5 x 5 over one 128-byte channel slice (128 int8 channels) and enough images for the large-halo layout: the written-out
    25-tap instance, int32 and requantised int8 results bit-exact on sampled images, partial tiles at the lower edge."""
    g = h.rng(48)
    shape, wshape, pad = (40, 37, 32, 128), (72, 5, 5, 128), (-2, -2)
    N, K = shape[0], wshape[0]
    x = g.integers(-127, 128, shape, dtype=np.int8)
    w = g.integers(-127, 128, wshape, dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    scale = g.uniform(1e-5, 1e-4, K).astype(np.float32)
    ys = (N, 37, 32, K)
    got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, pad=pad)
    q = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=cb.ACTIVATION_RELU, pad=pad)
    for n in (0, 17, N - 1):
        want = oracle.conv2d_i8(x[n:n + 1], w, b, pad=pad, activation=cb.ACTIVATION_RELU)
        np.testing.assert_array_equal(got[n:n + 1], want)
        np.testing.assert_array_equal(q[n:n + 1], oracle.requant_i8(want, scale))


@pytest.mark.parametrize("dtype,channels", [("f32", 32), ("f16", 64), ("bf16", 48)])
def test_written_out_5x5_floating(oracle, dtype, channels):
    """The same instance for the floating types (one channel slice each; 48 bf16 channels leave the slice partly empty), with
    bias, residual and ReLU, flipped filters included."""
    g = h.rng(49)
    shape, wshape, pad = (40, 37, 32, channels), (72, 5, 5, channels), (-2, -2)
    N, K = shape[0], wshape[0]
    x = h.rounded(oracle, g.standard_normal(shape), dtype)
    w = h.rounded(oracle, he(g, wshape), dtype)
    b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((N, 37, 32, K)), dtype)
    for mode in (0, 1):
        got = h.conv_forward("implicit_gemm", x, w, (N, 37, 32, K), dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, pad=pad, mode=mode)
        check_images(oracle, got, x, w, b, z, (0, 21, N - 1), BAR[dtype], pad=pad, mode=mode)
