"""Pins the CPU oracle against things that do not come from the oracle itself: torch's fp64 conv2d,
hand-computed cases, closed forms and invariants.  The reference holds no golden vectors for this path
(its tests are differential against a CPU backend that is a separate project)."""
import numpy as np
import pytest
import torch

RNG = np.random.default_rng(0xA70CAD0)


def torch_conv(x, w, pad, stride=(1, 1), dilation=(1, 1), groups=1):
    """NHWC/KRSC fp64 cross-check: Avocado CONVOLUTION mode == torch conv2d (no kernel flip), padding = -offset."""
    xt = torch.from_numpy(np.ascontiguousarray(x.transpose(0, 3, 1, 2)))
    wt = torch.from_numpy(np.ascontiguousarray(w.transpose(0, 3, 1, 2)))
    y = torch.nn.functional.conv2d(xt, wt, None, stride, (-pad[0], -pad[1]), dilation, groups)
    return y.numpy().transpose(0, 2, 3, 1)


@pytest.mark.parametrize("shape", [
    dict(x=(2, 7, 9, 5), w=(4, 3, 3, 5), pad=(-1, -1)),
    dict(x=(3, 8, 8, 6), w=(7, 5, 5, 6), pad=(-2, -2)),
    dict(x=(2, 6, 5, 8), w=(3, 1, 1, 8), pad=(0, 0)),
    dict(x=(2, 11, 12, 4), w=(6, 3, 3, 4), pad=(-1, -1), stride=(2, 2)),
    dict(x=(1, 9, 9, 3), w=(2, 3, 3, 3), pad=(-2, -2), dilation=(2, 2)),
    dict(x=(2, 6, 6, 8), w=(4, 3, 3, 4), pad=(-1, -1), groups=2),
    dict(x=(2, 6, 7, 3), w=(4, 3, 3, 3), pad=(0, 0)),
])
def test_conv_matches_torch_fp64(oracle, shape):
    x = RNG.standard_normal(shape["x"])
    w = RNG.standard_normal(shape["w"])
    kw = {k: v for k, v in shape.items() if k in ("stride", "dilation", "groups")}
    got = oracle.conv2d(x, w, pad=shape["pad"], **kw)
    want = torch_conv(x, w, shape["pad"], **kw)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-12)


def test_cross_correlation_mode_flips_the_kernel(oracle):
    x = RNG.standard_normal((2, 6, 7, 3))
    w = RNG.standard_normal((4, 3, 3, 3))
    got = oracle.conv2d(x, w, mode=oracle.CROSS_CORRELATION)
    want = torch_conv(x, np.ascontiguousarray(w[:, ::-1, ::-1, :]), (-1, -1))
    np.testing.assert_allclose(got, want, atol=1e-12)


def test_conv_hand_computed(oracle):
    # 1 image 3x3, 1 channel, values 1..9; 3x3 kernel of taps 1..9; offset -1.
    x = np.arange(1, 10, dtype=np.float64).reshape(1, 3, 3, 1)
    w = np.arange(1, 10, dtype=np.float64).reshape(1, 3, 3, 1)
    y = oracle.conv2d(x, w)
    # centre: sum i*i = 285; corner (0,0): taps 5,6,8,9 over pixels 1,2,4,5 = 5+12+32+45 = 94
    assert y[0, 1, 1, 0] == 285.0
    assert y[0, 0, 0, 0] == 94.0
    # corner (2,2): taps 1,2,4,5 over pixels 5,6,8,9 = 5+12+32+45 = 94
    assert y[0, 2, 2, 0] == 94.0
    # edge (0,1): taps 4..9 over pixels 1..6 = 4+10+18+28+40+54 = 154
    assert y[0, 0, 1, 0] == 154.0
    # non-zero padding value 2 at the corner adds 2*(1+2+3+4+7) = 34
    y2 = oracle.conv2d(x, w, padding_value=2.0)
    assert y2[0, 0, 0, 0] == 94.0 + 34.0


def test_conv_invariants(oracle):
    x = RNG.standard_normal((2, 5, 6, 3))
    # delta kernel at tap (0, 2) of channel c -> copy shifted by (pad + 0, pad + 2)
    w = np.zeros((3, 3, 3, 3))
    for k in range(3):
        w[k, 0, 2, k] = 1.0
    y = oracle.conv2d(x, w)
    want = np.zeros_like(x)
    want[:, 1:, :-1, :] = x[:, :-1, 1:, :]
    np.testing.assert_array_equal(y, want)
    # all-ones input and kernel: window population count
    ones = oracle.conv2d(np.ones((1, 4, 4, 1)), np.ones((1, 3, 3, 1)))[0, :, :, 0]
    np.testing.assert_array_equal(ones, np.array([[4, 6, 6, 4], [6, 9, 9, 6], [6, 9, 9, 6], [4, 6, 6, 4]], dtype=float))
    # linearity in x and w
    x2 = RNG.standard_normal(x.shape)
    w1, w2 = RNG.standard_normal((4, 3, 3, 3)), RNG.standard_normal((4, 3, 3, 3))
    a = oracle.conv2d(2.0 * x + x2, w1 - 3.0 * w2)
    b = 2 * oracle.conv2d(x, w1) - 6 * oracle.conv2d(x, w2) + oracle.conv2d(x2, w1) - 3 * oracle.conv2d(x2, w2)
    np.testing.assert_allclose(a, b, atol=1e-11)
    # 1x1 == matmul
    w11 = RNG.standard_normal((5, 1, 1, 3))
    np.testing.assert_allclose(oracle.conv2d(x, w11, pad=(0, 0)), x @ w11[:, 0, 0, :].T, atol=1e-13)


def test_conv_epilogue_order(oracle):
    x = RNG.standard_normal((2, 4, 5, 3))
    w = RNG.standard_normal((6, 3, 3, 3))
    b = RNG.standard_normal(6)
    z = RNG.standard_normal((2, 4, 5, 6))
    y0 = RNG.standard_normal((2, 4, 5, 6))
    conv = torch_conv(x, w, (-1, -1))
    got = oracle.conv2d(x, w, b, z, y0, alpha1=1.1, alpha2=1.2, beta=0.1, activation=oracle.RELU)
    want = np.maximum(1.1 * conv + 1.2 * z + b, 0.0) + 0.1 * y0
    np.testing.assert_allclose(got, want, atol=1e-12)
    got = oracle.conv2d(x, w, None, None, y0, alpha1=0.5, beta=0.0, activation=oracle.TANH)
    np.testing.assert_allclose(got, np.tanh(0.5 * conv), atol=1e-12)


def test_activations_against_numpy(oracle):
    v = np.linspace(-4, 4, 41)
    np.testing.assert_allclose(oracle.activation(oracle.SIGMOID, v), 1 / (1 + np.exp(-v)), atol=1e-15)
    np.testing.assert_allclose(oracle.activation(oracle.TANH, v), np.tanh(v), atol=1e-15)
    np.testing.assert_allclose(oracle.activation(oracle.RELU, v), np.maximum(v, 0))
    np.testing.assert_allclose(oracle.activation(oracle.ELU, v), np.where(v >= 0, v, np.expm1(v)), atol=1e-15)
    np.testing.assert_allclose(oracle.activation(oracle.SELU, v), 1.05070098 * np.where(v >= 0, v, 1.67326324 * np.expm1(v)), atol=1e-15)
    np.testing.assert_allclose(oracle.activation(oracle.EXPONENTIAL, v), np.exp(v), rtol=1e-15)
    np.testing.assert_allclose(oracle.activation(oracle.SOFTPLUS, v), np.log1p(np.exp(v)), atol=1e-15)
    np.testing.assert_allclose(oracle.activation(oracle.SOFTSIGN, v), v / (1 + np.abs(v)), atol=1e-15)


def test_int8_conv_is_exact(oracle):
    x = RNG.integers(-127, 128, (2, 6, 7, 16), dtype=np.int8)
    w = RNG.integers(-127, 128, (5, 3, 3, 16), dtype=np.int8)
    b = RNG.integers(-2 ** 15, 2 ** 15, 5, dtype=np.int32)
    got = oracle.conv2d_i8(x, w, b)
    # independent integer route: zero-padded windows through an int64 einsum
    xp = np.pad(x.astype(np.int64), ((0, 0), (1, 1), (1, 1), (0, 0)))
    want = np.zeros((2, 6, 7, 5), dtype=np.int64)
    for i in range(3):
        for j in range(3):
            want += np.einsum("nhwc,kc->nhwk", xp[:, i:i + 6, j:j + 7, :], w[:, i, j, :].astype(np.int64))
    want += b
    np.testing.assert_array_equal(got, want.astype(np.int32))
    # and the fp64 routine is exact at these magnitudes
    f = oracle.conv2d(x.astype(np.float64), w.astype(np.float64), b.astype(np.float64))
    np.testing.assert_array_equal(f, want.astype(np.float64))
    relu = oracle.conv2d_i8(x, w, b, activation=oracle.RELU)
    np.testing.assert_array_equal(relu, np.maximum(want, 0).astype(np.int32))
    # 1x1 and stride 2
    w1 = RNG.integers(-127, 128, (5, 1, 1, 16), dtype=np.int8)
    np.testing.assert_array_equal(oracle.conv2d_i8(x, w1, None, pad=(0, 0)), np.einsum("nhwc,kc->nhwk", x.astype(np.int64), w1[:, 0, 0].astype(np.int64)))
    s2 = oracle.conv2d_i8(x, w, b, stride=(2, 2))
    np.testing.assert_array_equal(s2, want[:, ::2, ::2, :].astype(np.int32))


def test_requant_hand_cases(oracle):
    """q = sat_i8(rne(float(acc) * scale)), every expected value written out.  Scales are powers of two (or small
    integers), so each product is exact and the expected value follows from the rounding rule alone."""
    table = [  # acc, scale, q
        (0, 2.0 ** -10, 0),
        (512, 2.0 ** -10, 0),        # 0.5 ties to even
        (1536, 2.0 ** -10, 2),       # 1.5 -> 2
        (2560, 2.0 ** -10, 2),       # 2.5 -> 2
        (3584, 2.0 ** -10, 4),       # 3.5 -> 4
        (-512, 2.0 ** -10, 0),       # -0.5 -> -0
        (-1536, 2.0 ** -10, -2),
        (-2560, 2.0 ** -10, -2),
        (513, 2.0 ** -10, 1),        # just above the tie
        (-513, 2.0 ** -10, -1),
        (1023, 2.0 ** -10, 1),       # 0.999 -> 1
        (130048, 2.0 ** -10, 127),   # 127.0
        (130560, 2.0 ** -10, 127),   # 127.5 -> 128 -> saturates
        (-131072, 2.0 ** -10, -128),  # -128.0
        (-131584, 2.0 ** -10, -128),  # -128.5 -> -128
        (-132096, 2.0 ** -10, -128),  # -129 saturates
        (2 ** 30, 2.0 ** -10, 127),
        (-2 ** 30, 2.0 ** -10, -128),
        (2 ** 31 - 1, 1.0, 127),
        (-2 ** 31, 1.0, -128),
        (16777217, 2.0 ** -18, 64),  # int32 -> fp32 rounds 2^24+1 to 2^24 first: 64.0 exactly
        (100, 0.0, 0),
        (7, 3.0, 21),
        (-43, 3.0, -128),            # -129
    ]
    acc = np.array([[t[0] for t in table]], dtype=np.int64).astype(np.int32)
    scale = np.array([t[1] for t in table], dtype=np.float32)
    want = np.array([[t[2] for t in table]], dtype=np.int8)
    np.testing.assert_array_equal(oracle.requant_i8(acc, scale), want)
    # the scale belongs to the filter (last axis), not to the row
    acc2 = np.array([[1024, 1024], [3072, 3072]], dtype=np.int32)
    np.testing.assert_array_equal(oracle.requant_i8(acc2, np.array([2.0 ** -10, 2.0 ** -9], dtype=np.float32)), np.array([[1, 2], [3, 6]], dtype=np.int8))
    # a non-trivial scale: 1e-3f = 0x3A83126F = 0.001000000047497451...; 500 * that = 0.50000002..., which fp32 rounds to 0.5 -> 0
    assert np.float32(1e-3).view(np.uint32) == 0x3A83126F
    np.testing.assert_array_equal(oracle.requant_i8(np.array([[500, 1500, -1500, 2500]], dtype=np.int32), np.full(4, 1e-3, dtype=np.float32)),
                                  np.array([[0, 2, -2, 2]], dtype=np.int8))


def _float_epilogue_1(oracle, acc, out_dtype, bias=None, z=None, y0=0, alpha1=1.0, alpha2=1.0, beta=0.0, activation=0):
    """One element through the float epilogue of the integer convolution."""
    a = np.array([[acc]], dtype=np.int32)
    b = None if bias is None else np.array([bias], dtype=np.float32)
    zz = None if z is None else np.array([[z]], dtype=out_dtype)
    y = np.array([[y0]], dtype=out_dtype)
    return oracle.conv2d_i8_float_epilogue(a, b, zz, y, alpha1, alpha2, beta, activation)[0, 0]


def test_int8_float_epilogue_reduces_to_exact_integer_path(oracle):
    """alpha1 = 1, integer-valued fp32 bias, |sum| < 2^24: every fp32 step is exact, so the float epilogue must reproduce the
    exact integer convolution (pinned above) bit for bit, as int32 and, after clamping, as int8.
    (src/conv2d_implicit_gemm.cu:278-286,330-338)"""
    x = RNG.integers(-127, 128, (2, 5, 6, 16), dtype=np.int8)
    w = RNG.integers(-127, 128, (7, 3, 3, 16), dtype=np.int8)
    b = RNG.integers(-2 ** 15, 2 ** 15, 7).astype(np.int32)
    raw = oracle.conv2d_i8(x, w, None)
    assert np.abs(raw.astype(np.int64)).max() + 2 ** 15 < 2 ** 24
    for act in (oracle.LINEAR, oracle.RELU):
        exact = oracle.conv2d_i8(x, w, b, activation=act)
        got32 = oracle.conv2d_i8_float_epilogue(raw, b.astype(np.float32), None, np.zeros(raw.shape, np.int32), 1.0, 1.0, 0.0, act)
        np.testing.assert_array_equal(got32, exact)
        got8 = oracle.conv2d_i8_float_epilogue(raw, b.astype(np.float32), None, np.zeros(raw.shape, np.int8), 1.0, 1.0, 0.0, act)
        np.testing.assert_array_equal(got8, np.clip(exact, -128, 127).astype(np.int8))
        gotf = oracle.conv2d_i8_float_epilogue(raw, b.astype(np.float32), None, np.zeros(raw.shape, np.float32), 1.0, 1.0, 0.0, act)
        np.testing.assert_array_equal(gotf, exact.astype(np.float32))
    # no bias: the term is skipped
    np.testing.assert_array_equal(oracle.conv2d_i8_float_epilogue(raw, None, None, np.zeros(raw.shape, np.int32), 1.0, 1.0, 0.0, 0), raw)
    # integer-valued residual and old output with power-of-two scalars stay exact as well
    z = RNG.integers(-1000, 1000, raw.shape).astype(np.int32)
    y0 = RNG.integers(-1000, 1000, raw.shape).astype(np.int32)
    want = np.maximum(raw.astype(np.int64) + b + 2 * z.astype(np.int64), 0) + 4 * y0.astype(np.int64)
    got = oracle.conv2d_i8_float_epilogue(raw, b.astype(np.float32), z, y0.copy(), 1.0, 2.0, 4.0, oracle.RELU)
    np.testing.assert_array_equal(got, want.astype(np.int32))


def test_int8_float_epilogue_rounding_hand_cases(oracle):
    """Cast back to the integer type: round to nearest even, saturate, NaN -> 0.  Expected values written out by hand."""
    i32, i8, f32 = np.int32, np.int8, np.float32
    one = lambda *a, **k: _float_epilogue_1(oracle, *a, **k)
    # ties, alpha1 = 0.5 (products exact)
    for acc, want in [(1, 0), (3, 2), (5, 2), (7, 4), (-1, 0), (-3, -2), (-5, -2), (2, 1), (-2, -1)]:
        assert one(acc, i32, alpha1=0.5) == want
        assert one(acc, i8, alpha1=0.5) == want
        assert one(acc, f32, alpha1=0.5) == acc / 2.0  # fp32 output is not rounded to an integer
    # -0.5 rounds to minus zero, which is integer 0
    assert one(-1, i32, alpha1=0.5) == 0
    # saturation of int8
    assert one(255, i8, alpha1=0.5) == 127       # 127.5 -> 128 -> 127
    assert one(254, i8, alpha1=0.5) == 127
    assert one(253, i8, alpha1=0.5) == 126       # 126.5 -> 126
    assert one(-257, i8, alpha1=0.5) == -128     # -128.5 -> -128
    assert one(-259, i8, alpha1=0.5) == -128     # -129.5 -> saturates
    assert one(10 ** 9, i8) == 127
    assert one(-10 ** 9, i8) == -128
    # saturation of int32: 2^30 * 2 = 2^31 and beyond clamp to INT32_MAX; -2^31 is representable; below it clamps
    assert one(2 ** 30, i32, alpha1=2.0) == 2 ** 31 - 1
    assert one(2 ** 30, i32, alpha1=1024.0) == 2 ** 31 - 1
    assert one(-2 ** 30, i32, alpha1=2.0) == -2 ** 31
    assert one(-2 ** 30, i32, alpha1=4.0) == -2 ** 31
    assert one(2 ** 30, i32, alpha1=1.0) == 2 ** 30
    assert one(2 ** 31 - 1, i32) == 2 ** 31 - 1            # float(2^31 - 1) = 2^31 -> saturates to INT32_MAX
    assert one(2 ** 31 - 129, i32) == 2 ** 31 - 128        # float() rounds to the nearest multiple of 128
    assert one(2147483520, i32) == 2147483520              # largest fp32 below 2^31 passes unchanged
    # NaN (inf * 0, NaN bias) -> 0; infinities saturate
    assert one(0, i32, alpha1=float("inf")) == 0
    assert one(5, i8, bias=float("nan")) == 0
    assert one(1, i32, alpha1=float("inf")) == 2 ** 31 - 1
    assert one(-1, i8, alpha1=float("inf")) == -128
    assert np.isnan(one(5, f32, bias=float("nan")))
    # int32 -> fp32 conversion of the sum is itself a rounding: 2^24 + 1 -> 2^24 (ties to even), 2^24 + 3 -> 2^24 + 4
    assert one(2 ** 24 + 1, f32) == 16777216.0
    assert one(2 ** 24 + 3, f32) == 16777220.0
    assert one(2 ** 24 + 1, i32) == 16777216
    # separate roundings, no fused multiply-add and no wider intermediate:
    #   alpha1 = 1 + 2^-12, acc = 4097: exact product 4098 + 2^-12 lies half-way between 4098 and 4098 + 2^-11 -> 4098 (even);
    #   + bias -4098 -> 0.  A fused multiply-add or a double intermediate gives 2^-12.
    assert one(4097, f32, bias=-4098.0, alpha1=1.0 + 2.0 ** -12) == 0.0
    #   alpha1 = 4097, acc = 4097: 4097^2 = 2^24 + 8193 is odd, fp32 spacing there is 2 -> ties to 16785408; - 16785408 -> 0 (wider: 1)
    assert one(4097, i32, bias=-16785408.0, alpha1=4097.0) == 0
    #   product rounds, then the bias addition rounds again: 2^24 (+1 -> tie -> 2^24) (+ 1*z=1 -> tie -> 2^24); adding b + z first gives 2^24 + 2
    assert one(2 ** 24, f32, bias=1.0, z=1.0) == 16777216.0
    assert one(2 ** 24, i32, bias=1.0, z=1) == 16777216
    # a product that is inexact in fp32: 0.1f = 0x3DCCCCCD; 3 * 0.1f = 0.3000000044703484 -> 0x3E99999A; + 0.2f (0x3E4CCCCD) = 0.5000000149 -> 0x3F000000
    r = one(3, f32, bias=np.float32(0.2), alpha1=np.float32(0.1))
    assert np.float32(r).view(np.uint32) == 0x3F000000
    r = one(3, f32, alpha1=np.float32(0.1))
    assert np.float32(r).view(np.uint32) == 0x3E99999A
    # -56228 * 0x3FF35336 + 0xC28E560E: two roundings give 0xC7D0E7A7, one rounding of the exact value 0xC7D0E7A6
    a1 = np.array([0x3FF35336], dtype=np.uint32).view(np.float32)[0]
    bb = np.array([0xC28E560E], dtype=np.uint32).view(np.float32)[0]
    r = one(-56228, f32, bias=bb, alpha1=a1)
    assert np.float32(r).view(np.uint32) == 0xC7D0E7A7


def test_int8_float_epilogue_order(oracle):
    """t = alpha1*float(sum); t += b; t += alpha2*z; t = act(t); t += beta*y_old  (src/conv2d_implicit_gemm.cu:278-286 with the
    bias term of include/Avocado/cuda_backend.h:796).  Every other order of these steps gives a different number here."""
    i32, i8, f32 = np.int32, np.int8, np.float32
    one = lambda *a, **k: _float_epilogue_1(oracle, *a, **k)
    # sum -10, b 2, z 3, y_old 8, beta 0.5, ReLU:  relu(-10 + 2 + 3) = 0, + 4 = 4
    #   beta*y before the activation: relu(-5 + 4) = 0;  bias after the activation: relu(-7) + 2 = 2;  z after the activation: relu(-8) + 3 = 3
    for dt in (i32, i8, f32):
        assert one(-10, dt, bias=2.0, z=3, y0=8, beta=0.5, activation=oracle.RELU) == 4
    # alpha2 scales z only, alpha1 the sum only: 3*5 + 1 + 2*4 = 24
    for dt in (i32, i8, f32):
        assert one(5, dt, bias=1.0, z=4, alpha1=3.0, alpha2=2.0) == 24
    # beta = 0: the old output is not read (a NaN there must not leak); beta != 0 reads it
    assert one(5, f32, y0=float("nan"), beta=0.0) == 5.0
    assert np.isnan(one(5, f32, y0=float("nan"), beta=1.0))
    # z and y_old are of the output's kind: int8 z = -128, y_old = 127
    assert one(0, i8, z=-128, alpha2=0.5) == -64
    assert one(0, i8, y0=127, beta=1.0) == 127
    assert one(1, i8, y0=127, beta=1.0) == 127     # 128 saturates
    # fp32 kind keeps fractions of z
    assert one(1, f32, z=0.25, alpha2=2.0) == 1.5
    # another activation than ReLU sits at the same place: tanh(0.5*2 + 0) + 1*3
    np.testing.assert_allclose(one(2, f32, y0=3.0, alpha1=0.5, beta=1.0, activation=oracle.TANH), np.float32(np.tanh(1.0)) + np.float32(3.0), rtol=1e-6)
    # filters index the bias (last axis)
    acc = np.array([[1, 1, 1], [2, 2, 2]], dtype=np.int32)
    got = oracle.conv2d_i8_float_epilogue(acc, np.array([10, 20, 30], dtype=np.float32), None, np.zeros((2, 3), np.int32), 1.0, 1.0, 0.0, 0)
    np.testing.assert_array_equal(got, [[11, 21, 31], [12, 22, 32]])


@pytest.mark.parametrize("m,r", [(2, 3), (4, 3), (2, 5)])
def test_winograd_tables_reproduce_correlation(oracle, m, r):
    """A^T[(G g G^T) .* (B^T d B)]A equals the direct correlation of a t x t patch with an r x r kernel."""
    G, BT, AT = (oracle.winograd_table(m, r, i) for i in range(3))
    t = m + r - 1
    d = RNG.standard_normal((t, t))
    g = RNG.standard_normal((r, r))
    y = AT @ ((G @ g @ G.T) * (BT @ d @ BT.T)) @ AT.T
    want = np.array([[np.sum(d[a:a + r, b:b + r] * g) for b in range(m)] for a in range(m)])
    np.testing.assert_allclose(y, want, atol=1e-12)


@pytest.mark.parametrize("m,r,pad", [(2, 3, (-1, -1)), (4, 3, (-1, -1)), (2, 5, (-2, -2)), (4, 3, (0, -2))])
@pytest.mark.parametrize("mode", [0, 1])
def test_winograd_pipeline_equals_direct(oracle, m, r, pad, mode):
    """weight transform -> input transform -> batched GEMM -> output transform == direct convolution,
    on odd sizes (partial tiles), with bias, residual, activation and beta."""
    N, H, W, Cin, K = 2, 7, 9, 5, 3
    x = RNG.standard_normal((N, H, W, Cin))
    w = RNG.standard_normal((K, r, r, Cin))
    b = RNG.standard_normal(K)
    U = oracle.winograd_weight_transform(w, m, invert=(mode == 1))
    V = oracle.winograd_input_transform(x, m, r, pad)
    Mx = oracle.gemm_batched(V, U, opA=False, opB=True)
    if pad == (-(r // 2), -(r // 2)):
        z = RNG.standard_normal((N, H, W, K))
        y0 = RNG.standard_normal((N, H, W, K))
        got = oracle.winograd_output_transform(Mx, (N, H, W, K), m, r, b, z, y0, 1.1, 1.2, 0.1, oracle.RELU)
        want = oracle.conv2d(x, w, b, z, y0, pad=pad, mode=mode, alpha1=1.1, alpha2=1.2, beta=0.1, activation=oracle.RELU)
        np.testing.assert_allclose(got, want, atol=1e-11)
    else:
        # asymmetric offsets: the tile grid of the output transform still covers H x W outputs, the direct
        # convolution with the same offsets is defined wherever the window start is (out_shape forces H x W)
        got = oracle.winograd_output_transform(Mx, (N, H, W, K), m, r)
        want = oracle.conv2d(x, w, pad=pad, mode=mode, out_shape=(H, W))
        np.testing.assert_allclose(got, want, atol=1e-11)


def test_winograd_layouts(oracle):
    """[t*t, tiles, C] layout, tile index (n*Th + th)*Tw + tw, padding value substitution."""
    m, r = 2, 3
    x = RNG.standard_normal((2, 3, 5, 2))
    V = oracle.winograd_input_transform(x, m, r, (-1, -1), padding_value=0.5)
    BT = oracle.winograd_table(m, r, 1)
    Th, Tw = 2, 3
    assert V.shape == (16, 2 * Th * Tw, 2)
    n, th, tw, c = 1, 1, 2, 1
    d = np.full((4, 4), 0.5)
    for a in range(4):
        for b in range(4):
            ih, iw = -1 + th * 2 + a, -1 + tw * 2 + b
            if 0 <= ih < 3 and 0 <= iw < 5:
                d[a, b] = x[n, ih, iw, c]
    want = BT @ d @ BT.T
    np.testing.assert_allclose(V[:, (n * Th + th) * Tw + tw, c].reshape(4, 4), want, atol=1e-13)
    w = RNG.standard_normal((3, 3, 3, 2))
    U = oracle.winograd_weight_transform(w, m)
    G = oracle.winograd_table(m, r, 0)
    np.testing.assert_allclose(U[:, 2, 1].reshape(4, 4), G @ w[2, :, :, 1] @ G.T, atol=1e-13)
    Ui = oracle.winograd_weight_transform(w, m, invert=True)
    np.testing.assert_allclose(Ui[:, 2, 1].reshape(4, 4), G @ w[2, ::-1, ::-1, 1] @ G.T, atol=1e-13)


@pytest.mark.parametrize("m,r", [(2, 3), (4, 3), (2, 5)])
def test_winograd_training_tables_reproduce_weight_gradient(oracle, m, r):
    """U'[(G' dy G'^T) .* (B^T d B)]U'^T equals the r x r correlation of a t x t input patch with an m x m tile of dy."""
    BT, GR, UP = (oracle.winograd_table(m, r, i) for i in (1, 3, 4))
    t = m + r - 1
    assert GR.shape == (t, m) and UP.shape == (r, t)
    d = RNG.standard_normal((t, t))
    dy = RNG.standard_normal((m, m))
    dw = UP @ ((GR @ dy @ GR.T) * (BT @ d @ BT.T)) @ UP.T
    want = np.array([[np.sum(d[i:i + m, j:j + m] * dy) for j in range(r)] for i in range(r)])
    np.testing.assert_allclose(dw, want, atol=1e-12)


@pytest.mark.parametrize("m,r", [(2, 3), (4, 3), (2, 5)])
def test_winograd_weight_gradient_pipeline_matches_torch(oracle, m, r):
    """input transform (x) and gradient transform (dy) -> batched GEMM (T, N) -> update transform == the weight gradient
    torch's fp64 autograd gives for conv2d, on odd sizes (partial tiles); alpha and beta of the update transform applied."""
    N, H, W, Cin, K = 2, 7, 9, 3, 4
    x = RNG.standard_normal((N, H, W, Cin))
    dy = RNG.standard_normal((N, H, W, K))
    xt = torch.tensor(x.transpose(0, 3, 1, 2).copy(), dtype=torch.float64)
    wt = torch.zeros((K, Cin, r, r), dtype=torch.float64, requires_grad=True)
    y = torch.nn.functional.conv2d(xt, wt, padding=r // 2)
    y.backward(torch.tensor(dy.transpose(0, 3, 1, 2).copy(), dtype=torch.float64))
    want = wt.grad.numpy().transpose(0, 2, 3, 1)  # [K, r, r, C]
    V = oracle.winograd_input_transform(x, m, r, (-(r // 2), -(r // 2)))
    Mg = oracle.winograd_gradient_transform(dy, m, r)
    dU = oracle.gemm_batched(Mg, V, opA=True, opB=False)
    got = oracle.winograd_update_transform(dU, m, r)
    np.testing.assert_allclose(got, want, atol=1e-10)
    dw0 = RNG.standard_normal((K, r, r, Cin))
    got = oracle.winograd_update_transform(dU, m, r, dw=dw0, alpha=0.5, beta=-2.0)
    np.testing.assert_allclose(got, 0.5 * want - 2.0 * dw0, atol=1e-10)


def test_winograd_training_layouts(oracle):
    """gradient transform: non-overlapping tiles, zeros past the border, [t*t, tiles, K]; update transform: [t*t, K, C] -> [K, r, r, C]."""
    m, r = 2, 3
    dy = RNG.standard_normal((2, 3, 5, 2))
    Mg = oracle.winograd_gradient_transform(dy, m, r)
    GR, UP = oracle.winograd_table(m, r, 3), oracle.winograd_table(m, r, 4)
    Th, Tw = 2, 3
    assert Mg.shape == (16, 2 * Th * Tw, 2)
    n, th, tw, k = 1, 1, 2, 1
    d = np.zeros((2, 2))
    d[0, 0] = dy[n, 2, 4, k]  # rows 2..3, columns 4..5 of a 3 x 5 map: only (2, 4) exists
    np.testing.assert_allclose(Mg[:, (n * Th + th) * Tw + tw, k].reshape(4, 4), GR @ d @ GR.T, atol=1e-13)
    Mx = RNG.standard_normal((16, 3, 2))
    dw = oracle.winograd_update_transform(Mx, m, r)
    assert dw.shape == (3, 3, 3, 2)
    np.testing.assert_allclose(dw[2, :, :, 1], UP @ Mx[:, 2, 1].reshape(4, 4) @ UP.T, atol=1e-13)


@pytest.mark.parametrize("opA", [False, True])
@pytest.mark.parametrize("opB", [False, True])
def test_gemm_batched_matches_numpy(oracle, opA, opB):
    b, M, N, K = 3, 23, 45, 67
    A = RNG.standard_normal((b, K, M) if opA else (b, M, K))
    B = RNG.standard_normal((b, N, K) if opB else (b, K, N))
    C0 = RNG.standard_normal((b, M, N))
    got = oracle.gemm_batched(A, B, C0, opA, opB, 1.1, 0.1)
    a = A.transpose(0, 2, 1) if opA else A
    bb = B.transpose(0, 2, 1) if opB else B
    np.testing.assert_allclose(got, 1.1 * np.matmul(a, bb) + 0.1 * C0, atol=1e-12)


def test_add_bias_formula(oracle):
    x = RNG.standard_normal((23, 45, 67))
    z = RNG.standard_normal(x.shape)
    y0 = RNG.standard_normal(x.shape)
    b = RNG.standard_normal(67)
    a1, a2, b1, b2, b3 = 1.1, 1.2, 0.1, 0.2, 0.3
    got = oracle.add_bias(x, b, z, y0, a1, a2, b1, b2, b3, oracle.SIGMOID)
    want = a1 / (1 + np.exp(-(a2 * x + b + b1 * z))) + b2 * z + b3 * y0
    np.testing.assert_allclose(got, want, atol=1e-13)
    got = oracle.add_bias(x, b, None, None, a1, a2, activation=oracle.RELU)
    np.testing.assert_allclose(got, a1 * np.maximum(a2 * x + b, 0), atol=1e-13)


@pytest.mark.parametrize("R,pad,mode", [(3, (-1, -1), 0), (5, (-2, -2), 0), (3, (-1, -1), 1)])
def test_im2row_times_weights_is_conv(oracle, R, pad, mode):
    x = RNG.standard_normal((2, 6, 7, 4))
    w = RNG.standard_normal((3, R, R, 4))
    rows = oracle.im2row(x, R, R, pad, mode)
    got = (rows @ w.reshape(3, -1).T).reshape(2, 6, 7, 3)
    np.testing.assert_allclose(got, oracle.conv2d(x, w, pad=pad, mode=mode), atol=1e-12)


@pytest.mark.parametrize("R,pad,stride,dilation,mode", [(3, (-1, -1), (2, 2), (1, 1), 0), (3, (-2, -2), (1, 1), (2, 2), 0), (3, (-1, 0), (2, 1), (1, 2), 1),
                                                         (5, (-2, -1), (3, 2), (1, 1), 0), (2, (0, -1), (2, 3), (2, 1), 1)])
def test_im2row_with_strides_and_dilations_times_weights_is_conv(oracle, R, pad, stride, dilation, mode):
    """The strided and asymmetric cases the reference's test leaves commented out (test/test_im2row.cpp:31-48): the rows
    against the already pinned direct convolution with the same geometry."""
    x = RNG.standard_normal((2, 11, 10, 3))
    w = RNG.standard_normal((4, R, R, 3))
    Ho, Wo = oracle.conv_output_shape(11, 10, R, R, pad, stride, dilation)
    rows = oracle.im2row(x, R, R, pad, mode, 0.0, stride, dilation)
    assert rows.shape == (2 * Ho * Wo, R * R * 3)
    got = (rows @ w.reshape(4, -1).T).reshape(2, Ho, Wo, 4)
    np.testing.assert_allclose(got, oracle.conv2d(x, w, pad=pad, stride=stride, dilation=dilation, mode=mode), atol=1e-12)


def test_bf16_rounding_helpers(oracle):
    v = np.array([1.0, 1.00390625, 1.01171875, -3.0e38, 1e-40, np.inf], dtype=np.float32)
    bits = oracle.f32_to_bf16_bits(v)
    back = oracle.bf16_bits_to_f32(bits)
    # 1.00390625 = 1 + 2^-8 is a tie between 1.0 and 1.0078125 -> even mantissa (1.0)
    assert back[0] == 1.0 and back[1] == 1.0
    # 1.01171875 = 1 + 3*2^-8 is a tie between 1.0078125 (odd) and 1.015625 (even)
    assert back[2] == np.float32(1.015625)
    t = torch.tensor(v).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(back, t)
    big = RNG.standard_normal(10000).astype(np.float32)
    np.testing.assert_array_equal(oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(big)), torch.tensor(big).to(torch.bfloat16).to(torch.float32).numpy())


# ---- per-channel transforms: affine forward and batch normalisation in inference (src/batchnorm.cu:28-69) ---------------
def test_affine_forward_reduces_to_add_bias_and_broadcast_form(oracle):
    g = np.random.default_rng(77)
    x = g.standard_normal((5, 6, 7, 12))
    w = g.standard_normal(12)
    b = g.standard_normal(12)
    y0 = g.standard_normal(x.shape)
    for act in (oracle.LINEAR, oracle.RELU, oracle.TANH):
        # weight 1: the add-bias routine, which has its own pins (y = alpha1 * act(x + b) + beta3 * y)
        got = oracle.affine_forward(x, np.ones(12), b, y0, alpha=1.3, beta=0.4, activation=act)
        want = oracle.add_bias(x, b, None, y0, alpha1=1.3, alpha2=1.0, beta3=0.4, activation=act)
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-14)
        # general weight: x * w is x with its channels pre-scaled
        got = oracle.affine_forward(x, w, b, None, alpha=0.7, activation=act)
        want = oracle.add_bias(x * w, b, alpha1=0.7, activation=act)
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-14)
    # parameters spanning the two trailing dimensions
    w2, b2 = g.standard_normal((7, 12)), g.standard_normal((7, 12))
    np.testing.assert_allclose(oracle.affine_forward(x, w2, b2), x * w2 + b2, rtol=0, atol=1e-14)


def test_batchnorm_inference_matches_torch_and_folded_affine(oracle):
    import torch
    g = np.random.default_rng(78)
    x = g.standard_normal((4, 5, 6, 16)) * 2 + 0.5
    scale, bias, mean = g.standard_normal(16), g.standard_normal(16), g.standard_normal(16)
    var = g.uniform(0.1, 2.0, 16)
    eps = 1e-3
    got = oracle.batchnorm_inference(x, scale, bias, mean, var, epsilon=eps)
    # independent library routine: channels-last data moved to torch's channel-second layout
    t = torch.nn.functional.batch_norm(torch.from_numpy(x).permute(0, 3, 1, 2), torch.from_numpy(mean), torch.from_numpy(var), torch.from_numpy(scale),
                                       torch.from_numpy(bias), training=False, eps=eps)
    np.testing.assert_allclose(got, t.permute(0, 2, 3, 1).numpy(), rtol=0, atol=1e-12)
    s = scale / np.sqrt(var + eps)
    y0 = g.standard_normal(x.shape)
    got = oracle.batchnorm_inference(x, scale, bias, mean, var, y0, alpha=1.1, beta=0.3, epsilon=eps, activation=oracle.RELU)
    want = oracle.affine_forward(x, s, bias - mean * s, y0, alpha=1.1, beta=0.3, activation=oracle.RELU)
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-13)
    # identity statistics leave x unchanged
    np.testing.assert_allclose(oracle.batchnorm_inference(x, np.ones(16), np.zeros(16), np.zeros(16), np.ones(16), epsilon=0.0), x, rtol=0, atol=0)
