"""GPU parity of the parity-plane kernel for 3x3 stride-2 layers of 16-bit tensors: its weight layout against the closed form, the kernel
through the kernel-layer C-ABI and through the dispatcher against the CPU oracle on identical seeded inputs.  Bar: rel-L2 <= 2e-3
(fp16 / bf16).  The strided geometries follow the cases test/test_im2row.cpp:31-48 of the reference leaves commented out."""
import ctypes as C

import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu

BAR = 2e-3


class Shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("N", "H", "W", "C", "K", "R", "S", "Ho", "Wo", "pad_h", "pad_w", "stride_h", "stride_w", "dil_h", "dil_w",
                                       "mode")]


def shape_of(oracle, x, w, pad=(-1, -1), stride=(2, 2), dilation=(1, 1), mode=0):
    Ho, Wo = oracle.conv_output_shape(x[1], x[2], w[1], w[2], pad, stride, dilation)
    return Shape(x[0], x[1], x[2], x[3], w[0], w[1], w[2], Ho, Wo, pad[0], pad[1], stride[0], stride[1], dilation[0], dilation[1], mode)


@pytest.fixture
def strided_forced():
    """The dispatcher takes the parity-plane kernel for every layer it can run, whatever its size."""
    lib = cb.load_library()
    lib.avhip_set_conv_strided.restype = int
    previous = lib.avhip_set_conv_strided(2)
    yield lib
    lib.avhip_set_conv_strided(previous)


def transforms(lib):
    n = C.c_int64(0)
    assert lib.avhipGetWeightCacheState(None, None, C.byref(n)) == cb.STATUS_SUCCESS
    return n.value


def he(g, shape, dtype, orc):
    K, R, S, Cin = shape
    return h.rounded(orc, g.standard_normal(shape) * np.sqrt(2.0 / (R * S * Cin)), dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("mode", [0, 1])
def test_weight_layout(oracle, dtype, mode):
    """The weights themselves (taps reversed in the flipping mode) in the register layout of the kernel's MFMA operand:
    [C / 32][9 taps][K / 32][2 slabs][64 lanes][8], lane l = filter l % 32, channels 8 * (l / 32) .. + 7 of the 16-channel slab."""
    lib = cb.load_library()
    lib.avhip_conv2d_strided_weight_bytes.restype = C.c_int64
    K, Cin = 256, 64
    g = h.rng(411)
    w = he(g, (K, 3, 3, Cin), dtype, oracle)
    nbytes = lib.avhip_conv2d_strided_weight_bytes(K, Cin)
    assert nbytes == 9 * K * Cin * 2
    with h.Call() as c:
        wt = c.tensor(w, dtype)
        U = c.empty((nbytes // 2,), dtype)
        lib.avhip_conv2d_strided_weight_layout.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        assert lib.avhip_conv2d_strided_weight_layout(C.c_void_p(c.ctx.stream()), h.DT[dtype], mode, wt.pointer(), U.pointer(), K, Cin) == 0
        c.finish()
        got = U.download().reshape(Cin // 32, 9, K // 32, 2, 64, 8)
    ww = (w[:, ::-1, ::-1, :] if mode else w).reshape(K // 32, 32, 9, Cin // 32, 2, 2, 8)  # tile, filter, tap, phase, slab, half, 8
    want = ww.transpose(3, 2, 0, 4, 5, 1, 6).reshape(Cin // 32, 9, K // 32, 2, 64, 8)  # lane = half * 32 + filter
    assert np.array_equal(got, want), "a re-ordering of the weights: exact"


CASES = [
    # x, w, keyword arguments
    dict(x=(2, 56, 56, 128), w=(256, 3, 3, 128)),                                     # BASELINE config 5, first layer, two images
    dict(x=(3, 28, 28, 64), w=(256, 3, 3, 64), mode=1, z=True),                        # one trip of two phases, flipped taps, residual
    dict(x=(2, 15, 17, 256), w=(512, 3, 3, 256), pad=(0, 0), z=True, relu=False, alpha1=1.1, alpha2=1.2),  # no padding, odd sizes, two filter blocks
    dict(x=(1, 112, 112, 64), w=(256, 3, 3, 64)),                                     # 56 x 56 outputs: tiles across and down
    dict(x=(2, 30, 9, 192), w=(256, 3, 3, 192), pad=(-2, -1)),                         # six phases, asymmetric offsets, narrow image
    dict(x=(2, 8, 8, 64), w=(256, 3, 3, 64)),                                         # an image much smaller than a tile
    dict(x=(2, 16, 16, 64), w=(256, 3, 3, 64), bias=False, relu=False),                  # no bias, no activation: the accumulators as they are
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_through_the_dispatcher(oracle, strided_forced, dtype, case):
    cs = CASES[case]
    g = h.rng(430 + case)
    xs, ws = cs["x"], cs["w"]
    pad, mode = cs.get("pad", (-1, -1)), cs.get("mode", 0)
    s = shape_of(oracle, xs, ws, pad=pad, mode=mode)
    assert strided_forced.avhip_conv2d_strided_plan(h.DT[dtype], C.byref(s), None, None) == 0, "the kernel must take this layer"
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64) if cs.get("bias", True) else None
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype) if cs.get("z") else None
    relu = cs.get("relu", True)
    a1, a2 = cs.get("alpha1"), cs.get("alpha2")
    before = transforms(strided_forced)
    got = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, z=z, alpha1=a1, alpha2=a2, activation=cb.ACTIVATION_RELU if relu else 0, pad=pad, stride=(2, 2),
                         mode=mode)
    assert transforms(strided_forced) == before + 1, "the plan lays the weights out once; the gather kernel never does"
    want = oracle.conv2d(x, w, b, z=z, pad=pad, stride=(2, 2), mode=mode, alpha1=1.0 if a1 is None else a1, alpha2=1.0 if a2 is None else a2,
                         activation=oracle.RELU if relu else oracle.LINEAR)
    err = oracle.rel_l2(got, want)
    print("strided %s case %d rel-L2 = %.3e" % (dtype, case, err))
    assert err < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_through_the_implicit_gemm_entry(oracle, strided_forced, dtype):
    """cudaConvolutionImplicitGemmForward takes the same kernel: it is an implicit GEMM with the weights in another order."""
    cs = CASES[1]
    g = h.rng(470)
    xs, ws = cs["x"], cs["w"]
    pad, mode = cs.get("pad", (-1, -1)), cs.get("mode", 0)
    s = shape_of(oracle, xs, ws, pad=pad, mode=mode)
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    before = transforms(strided_forced)
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, pad=pad, stride=(2, 2), mode=mode)
    assert transforms(strided_forced) == before + 1, "the general kernels never lay weights out"
    want = oracle.conv2d(x, w, b, z=z, pad=pad, stride=(2, 2), mode=mode, activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("through the implicit-GEMM entry %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_kernel_layer_entry(oracle, dtype):
    """avhip_conv2d_strided_weight_layout + avhip_conv2d_strided called as a foreign host would: raw device pointers."""
    lib = cb.load_library()
    lib.avhip_conv2d_strided_weight_bytes.restype = C.c_int64
    g = h.rng(450)
    xs, ws = (3, 20, 22, 128), (256, 3, 3, 128)
    s = shape_of(oracle, xs, ws)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    lib.avhip_conv2d_strided.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_double,
                                         C.c_double, C.c_int]
    lib.avhip_conv2d_strided_weight_layout.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    with h.Call() as c:
        xt, wt, zt, bt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(z, dtype), c.tensor(b, "f32")
        y = c.empty(ys, dtype)
        U = c.empty((lib.avhip_conv2d_strided_weight_bytes(ws[0], ws[3]) // 2,), dtype)
        stream = C.c_void_p(c.ctx.stream())
        assert lib.avhip_conv2d_strided_weight_layout(stream, h.DT[dtype], 0, wt.pointer(), U.pointer(), ws[0], ws[3]) == 0
        args = (stream, h.DT[dtype], C.addressof(s), xt.pointer(), U.pointer(), bt.pointer(), zt.pointer(), y.pointer())
        assert lib.avhip_conv2d_strided(*args, 1.0, 1.0, 0.0, cb.ACTIVATION_RELU) == 0
        c.finish()
        got = y.download()
        assert lib.avhip_conv2d_strided(*args, 1.0, 1.0, 0.5, cb.ACTIVATION_RELU) == -1  # beta
        assert lib.avhip_conv2d_strided(*args, 1.0, 1.0, 0.0, cb.ACTIVATION_SIGMOID) == -1
        s1 = shape_of(oracle, xs, ws, stride=(1, 1))
        assert lib.avhip_conv2d_strided(stream, h.DT[dtype], C.addressof(s1), *args[3:], 1.0, 1.0, 0.0, 0) == -1  # stride 1
        assert lib.avhip_conv2d_strided(stream, h.DT["f32"], C.addressof(s), *args[3:], 1.0, 1.0, 0.0, 0) == -2
    want = oracle.conv2d(x, w, b, z=z, stride=(2, 2), activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("strided kernel layer %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR


def test_plan_declines_what_the_kernel_cannot_run(oracle, strided_forced):
    lib = strided_forced
    ok = shape_of(oracle, (4, 56, 56, 128), (256, 3, 3, 128))
    groups, rows = C.c_int(0), C.c_int(0)
    assert lib.avhip_conv2d_strided_plan(h.DT["bf16"], C.byref(ok), C.byref(groups), C.byref(rows)) == 0
    assert groups.value == 16 and rows.value == 196  # four tiles of 7 x 28 output pixels per image
    for bad in (shape_of(oracle, (4, 56, 56, 128), (256, 3, 3, 128), stride=(1, 1)), shape_of(oracle, (4, 56, 56, 128), (256, 5, 5, 128), pad=(-2, -2)),
                shape_of(oracle, (4, 56, 56, 96), (256, 3, 3, 96)), shape_of(oracle, (4, 56, 56, 128), (128, 3, 3, 128)),
                shape_of(oracle, (4, 56, 56, 128), (256, 3, 3, 128), pad=(-2, -2), dilation=(2, 2))):
        assert lib.avhip_conv2d_strided_plan(h.DT["bf16"], C.byref(bad), None, None) == -1
    assert lib.avhip_conv2d_strided_plan(h.DT["f32"], C.byref(ok), None, None) == -1
    lib.avhip_set_conv_strided(0)
    assert lib.avhip_conv2d_strided_plan(h.DT["bf16"], C.byref(ok), None, None) == -1
    lib.avhip_set_conv_strided(2)
