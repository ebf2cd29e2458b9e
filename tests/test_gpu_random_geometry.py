"""Seeded random sweep over convolution geometries, data types, epilogue terms and kernel selections, against the CPU oracle.
The hand-picked cases of the other files pin known edges; this sweep looks for the ones nobody thought of (ragged channel and
filter counts, windows hanging over any border, non-square filters with asymmetric offsets, strides and dilations that do not
divide the image).  Bars as everywhere: int8 bit-exact, fp32 1e-5 (1e-4 through Winograd), fp16 / bf16 2e-3."""
import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu

CHANNELS = [1, 2, 3, 4, 5, 8, 12, 16, 20, 32, 36, 64, 72, 136]
FILTERS = [1, 3, 4, 8, 20, 32, 40, 64, 132]


def random_case(g):
    R, S = int(g.choice([1, 2, 3, 5])), int(g.choice([1, 2, 3, 5]))
    dil = (int(g.choice([1, 1, 2])), int(g.choice([1, 1, 2])))
    stride = (int(g.choice([1, 1, 2, 3])), int(g.choice([1, 1, 2, 3])))
    H, W = int(g.integers(3, 21)), int(g.integers(3, 21))
    pad = (-int(g.integers(0, (R - 1) * dil[0] + 1)), -int(g.integers(0, (S - 1) * dil[1] + 1)))  # up to the full convolution
    return dict(x=(int(g.integers(1, 4)), H, W, int(g.choice(CHANNELS))), w=(int(g.choice(FILTERS)), R, S), pad=pad, stride=stride, dilation=dil,
                mode=int(g.integers(0, 2)))


def output_shape(orc, c):
    N, H, W, _ = c["x"]
    K, R, S = c["w"]
    Ho = (H - 2 * c["pad"][0] - ((R - 1) * c["dilation"][0] + 1)) // c["stride"][0] + 1
    Wo = (W - 2 * c["pad"][1] - ((S - 1) * c["dilation"][1] + 1)) // c["stride"][1] + 1
    return (N, Ho, Wo, K)


@pytest.mark.parametrize("tiling", ["wavefront_tiles", "workgroup_tiles"])
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_random_geometries_floating(oracle, dtype, tiling):
    lib = cb.load_library()
    lib.avhip_set_small_problem_threshold.restype = int
    previous = lib.avhip_set_small_problem_threshold(-1 if tiling == "wavefront_tiles" else 0)
    try:
        g = h.rng(50 + ["f32", "f16", "bf16"].index(dtype))
        done = 0
        while done < 120:
            c = random_case(g)
            ys = output_shape(oracle, c)
            if ys[1] < 1 or ys[2] < 1:
                continue
            done += 1
            x = h.rounded(oracle, g.standard_normal(c["x"]), dtype)
            ws = (c["w"][0], c["w"][1], c["w"][2], c["x"][3])
            w = h.rounded(oracle, g.standard_normal(ws) * np.sqrt(2.0 / (ws[1] * ws[2] * ws[3])), dtype)
            b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64) if g.random() < 0.7 else None
            z = h.rounded(oracle, g.standard_normal(ys), dtype) if g.random() < 0.5 else None
            act = int(g.choice([cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU, cb.ACTIVATION_RELU, cb.ACTIVATION_TANH]))
            kw = dict(pad=c["pad"], stride=c["stride"], dilation=c["dilation"], mode=c["mode"])
            want = oracle.conv2d(x, w, b, z, activation=act, **kw)
            assert want.shape == ys, (c, want.shape, ys)
            for entry in ("implicit_gemm", "dispatch"):
                got = h.conv_forward(entry, x, w, ys, dtype, bias=b, z=z, activation=act, **kw)
                bar = {"f32": 1e-4 if entry == "dispatch" else 1e-5, "f16": 2e-3, "bf16": 2e-3}[dtype]
                err = oracle.rel_l2(got, want)
                assert err < bar, "case %d %s %s: rel-L2 %.3e  %r bias=%s z=%s act=%d" % (done, entry, dtype, err, c, b is not None, z is not None, act)
            if ws[1] == 3 and ws[2] == 3 and c["stride"] == (1, 1) and c["dilation"] == (1, 1) and ws[3] % (4 if dtype == "f32" else 8) == 0:
                got = h.conv_forward("winograd_fused", x, w, ys, dtype, bias=b, z=z, activation=act, pad=c["pad"], mode=c["mode"])
                err = oracle.rel_l2(got, want)
                assert err < (1e-4 if dtype == "f32" else 2e-3), "case %d fused %s: rel-L2 %.3e  %r" % (done, dtype, err, c)
    finally:
        lib.avhip_set_small_problem_threshold(previous)


@pytest.mark.parametrize("tiling", ["wavefront_tiles", "workgroup_tiles"])
def test_random_geometries_int8(oracle, tiling):
    lib = cb.load_library()
    lib.avhip_set_small_problem_threshold.restype = int
    previous = lib.avhip_set_small_problem_threshold(-1 if tiling == "wavefront_tiles" else 0)
    try:
        g = h.rng(53)
        done = 0
        while done < 120:
            c = random_case(g)
            ys = output_shape(oracle, c)
            if ys[1] < 1 or ys[2] < 1:
                continue
            done += 1
            ws = (c["w"][0], c["w"][1], c["w"][2], c["x"][3])
            x = g.integers(-127, 128, c["x"], dtype=np.int8)
            w = g.integers(-127, 128, ws, dtype=np.int8)
            b = g.integers(-2 ** 15, 2 ** 15, ws[0]).astype(np.int32)
            scale = g.uniform(1e-4, 1e-3, ws[0]).astype(np.float32)
            act = int(g.choice([cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU]))
            kw = dict(pad=c["pad"], stride=c["stride"], dilation=c["dilation"], mode=c["mode"])
            want = oracle.conv2d_i8(x, w, b, activation=act, **kw)
            got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=act, **kw)
            np.testing.assert_array_equal(got, want, err_msg="case %d %r" % (done, c))
            q = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=act, **kw)
            np.testing.assert_array_equal(q, oracle.requant_i8(want, scale), err_msg="requant case %d %r" % (done, c))
    finally:
        lib.avhip_set_small_problem_threshold(previous)


@pytest.mark.parametrize("dtype", ["bf16", "i8"])
def test_random_wide_images_and_large_filters(oracle, dtype):
    """Stride-1 layers with wide images, many images and filters up to 7 x 7: the shapes for which the image-tile kernel picks
    between its two row orders and its two LDS layouts.  Sampled images against the oracle; int8 -> int32 bit-exact."""
    g = h.rng(57 if dtype == "bf16" else 58)
    done = 0
    while done < 24:
        R, S = int(g.choice([1, 2, 3, 4, 5, 7])), int(g.choice([1, 2, 3, 4, 5, 7]))
        if R * S == 1:
            continue
        N, H, W = int(g.integers(8, 49)), int(g.integers(8, 41)), int(g.integers(20, 73))
        Cin, K = int(g.choice([64, 128, 192])) if dtype == "i8" else int(g.choice([32, 64, 128])), int(g.choice([16, 64, 72]))
        pad = (-int(g.integers(0, R)), -int(g.integers(0, S)))
        mode = int(g.integers(0, 2))
        Ho, Wo = oracle.conv_output_shape(H, W, R, S, pad)
        if Ho < 1 or Wo < 1:
            continue
        done += 1
        images = sorted(set(int(i) for i in g.integers(0, N, 2)))
        if dtype == "i8":
            x = g.integers(-127, 128, (N, H, W, Cin), dtype=np.int8)
            w = g.integers(-127, 128, (K, R, S, Cin), dtype=np.int8)
            b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
            got = h.conv_forward("implicit_gemm", x, w, (N, Ho, Wo, K), "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, pad=pad, mode=mode)
            for n in images:
                want = oracle.conv2d_i8(x[n:n + 1], w, b, pad=pad, mode=mode, activation=cb.ACTIVATION_RELU)
                assert np.array_equal(got[n:n + 1], want), "case %d: N=%d %dx%d C=%d K=%d %dx%d pad=%r mode=%d image %d" % (done, N, H, W, Cin, K, R, S, pad, mode, n)
        else:
            x = h.rounded(oracle, g.standard_normal((N, H, W, Cin)), dtype)
            w = h.rounded(oracle, g.standard_normal((K, R, S, Cin)) * np.sqrt(2.0 / (R * S * Cin)), dtype)
            b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
            z = h.rounded(oracle, g.standard_normal((N, Ho, Wo, K)), dtype)
            got = h.conv_forward("dispatch", x, w, (N, Ho, Wo, K), dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, pad=pad, mode=mode)
            for n in images:
                want = oracle.conv2d(x[n:n + 1], w, b, z[n:n + 1], activation=oracle.RELU, pad=pad, mode=mode)
                err = oracle.rel_l2(got[n:n + 1], want)
                assert err < 2e-3, "case %d: N=%d %dx%d C=%d K=%d %dx%d pad=%r mode=%d image %d: rel-L2 %.3e" % (done, N, H, W, Cin, K, R, S, pad, mode, n, err)


@pytest.mark.parametrize("dtype", ["bf16", "f32", "i8"])
def test_random_few_channel_layers(oracle, dtype):
    """First-layer shapes: 1 to 12 input planes, filters up to 9 x 9, strides, dilations, both modes, images large enough for
    the kernel that gathers its operand from an image tile in LDS (piece sizes 1 to 16 bytes, with and without 16-byte image
    rows, one to three filter blocks, several tiles per image).  Sampled images against the oracle; int8 -> int32 bit-exact."""
    g = h.rng({"bf16": 61, "f32": 62, "i8": 63}[dtype])
    bar = {"bf16": 2e-3, "f32": 1e-5}
    done = 0
    while done < 30:
        R, S = int(g.integers(1, 10)), int(g.integers(1, 10))
        Cin = int(g.integers(1, 13))
        elem = {"bf16": 2, "f32": 4, "i8": 1}[dtype]
        if R * S == 1 or R * S * Cin * elem > 1024:
            continue
        stride = (int(g.integers(1, 4)), int(g.integers(1, 4)))
        dilation = (int(g.integers(1, 3)), int(g.integers(1, 3)))
        N, H, W = int(g.integers(1, 6)), int(g.integers(16, 70)), int(g.integers(16, 70))
        if g.integers(0, 2) == 1:
            W = (W + 7) // 8 * 8  # image rows of whole 16-byte pieces
        K = int(g.choice([8, 24, 64, 72, 136]))
        pad = (-int(g.integers(0, (R - 1) * dilation[0] + 1)), -int(g.integers(0, (S - 1) * dilation[1] + 1)))
        mode = int(g.integers(0, 2))
        Ho, Wo = oracle.conv_output_shape(H, W, R, S, pad, stride, dilation)
        if Ho < 1 or Wo < 1 or Ho * Wo < 100:
            continue
        done += 1
        kw = dict(pad=pad, stride=stride, dilation=dilation, mode=mode)
        what = "case %d: N=%d %dx%d C=%d K=%d %dx%d %r" % (done, N, H, W, Cin, K, R, S, kw)
        images = sorted(set(int(i) for i in g.integers(0, N, 2)))
        if dtype == "i8":
            x = g.integers(-127, 128, (N, H, W, Cin), dtype=np.int8)
            w = g.integers(-127, 128, (K, R, S, Cin), dtype=np.int8)
            b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
            got = h.conv_forward("implicit_gemm", x, w, (N, Ho, Wo, K), "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=cb.ACTIVATION_RELU, **kw)
            for n in images:
                want = oracle.conv2d_i8(x[n:n + 1], w, b, activation=cb.ACTIVATION_RELU, **kw)
                assert np.array_equal(got[n:n + 1], want), what + " image %d" % n
        else:
            x = h.rounded(oracle, g.standard_normal((N, H, W, Cin)), dtype)
            w = h.rounded(oracle, g.standard_normal((K, R, S, Cin)) * np.sqrt(2.0 / (R * S * Cin)), dtype)
            b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
            got = h.conv_forward("implicit_gemm", x, w, (N, Ho, Wo, K), dtype, bias=b, activation=cb.ACTIVATION_RELU, **kw)
            for n in images:
                want = oracle.conv2d(x[n:n + 1], w, b, activation=oracle.RELU, **kw)
                err = oracle.rel_l2(got[n:n + 1], want)
                assert err < bar[dtype], what + " image %d: rel-L2 %.3e" % (n, err)
