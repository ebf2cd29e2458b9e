"""GPU parity of the pixel-block kernel for 1x1 layers of 16-bit tensors (blocks of pixels resident in LDS, filters from L2 in
MFMA layout, results stored from the accumulators): its weight layout against the closed form, the kernel through the kernel-layer
C-ABI and through the dispatcher against the CPU oracle on identical seeded inputs.  Bar: rel-L2 <= 2e-3 (fp16 / bf16)."""
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


def shape_of(x, w, pad=(0, 0), stride=(1, 1), mode=0):
    Ho, Wo = (x[1] + 2 * -pad[0] - w[1]) // stride[0] + 1, (x[2] + 2 * -pad[1] - w[2]) // stride[1] + 1
    return Shape(x[0], x[1], x[2], x[3], w[0], w[1], w[2], Ho, Wo, pad[0], pad[1], stride[0], stride[1], 1, 1, mode)


@pytest.fixture
def block_forced():
    """The dispatcher takes the pixel-block kernel for every layer it can run, whatever its size."""
    lib = cb.load_library()
    lib.avhip_set_pointwise_block.restype = int
    previous = lib.avhip_set_pointwise_block(2)
    yield lib
    lib.avhip_set_pointwise_block(previous)


def transforms(lib):
    n = C.c_int64(0)
    assert lib.avhipGetWeightCacheState(None, None, C.byref(n)) == cb.STATUS_SUCCESS
    return n.value


def he(g, shape, dtype, orc):
    K, R, S, Cin = shape
    return h.rounded(orc, g.standard_normal(shape) * np.sqrt(2.0 / (R * S * Cin)), dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_weight_layout(oracle, dtype):
    """The weights themselves in the register layout of the kernel's MFMA operand: [K / 32][C / 16 slabs][64 lanes][8],
    lane l = filter l % 32, channels 8 * (l / 32) .. + 7 of the slab."""
    lib = cb.load_library()
    lib.avhip_conv2d_pointwise_block_weight_bytes.restype = C.c_int64
    K, Cin = 512, 128
    g = h.rng(511)
    w = he(g, (K, 1, 1, Cin), dtype, oracle)
    nbytes = lib.avhip_conv2d_pointwise_block_weight_bytes(K, Cin)
    assert nbytes == K * Cin * 2
    with h.Call() as c:
        wt = c.tensor(w, dtype)
        U = c.empty((nbytes // 2,), dtype)
        lib.avhip_conv2d_pointwise_block_weight_layout.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        assert lib.avhip_conv2d_pointwise_block_weight_layout(C.c_void_p(c.ctx.stream()), h.DT[dtype], wt.pointer(), U.pointer(), K, Cin) == 0
        c.finish()
        got = U.download().reshape(K // 32, Cin // 16, 64, 8)
    ww = w.reshape(K // 32, 32, Cin // 16, 2, 8)  # tile, filter, slab, half, 8
    want = ww.transpose(0, 2, 3, 1, 4).reshape(K // 32, Cin // 16, 64, 8)  # lane = half * 32 + filter
    assert np.array_equal(got, want), "a re-ordering of the weights: exact"


CASES = [
    # x, w, keyword arguments
    dict(x=(4, 28, 28, 256), w=(512, 1, 1, 256)),                                        # BASELINE config 5, second layer, four images: 14 blocks of 224
    dict(x=(3, 14, 14, 128), w=(512, 1, 1, 128), z=True),                                 # 588 pixels: a last block of 140, residual
    dict(x=(2, 9, 7, 256), w=(1024, 1, 1, 256), z=True, relu=False, alpha1=1.1, alpha2=1.2),  # one block of 126 pixels, two filter blocks
    dict(x=(1, 5, 5, 128), w=(512, 1, 1, 128)),                                           # 25 pixels: less than one MFMA tile
    dict(x=(2, 33, 31, 256), w=(512, 1, 1, 256), relu=False),                             # 2046 pixels: ten blocks, the last one short
    dict(x=(2, 12, 12, 128), w=(512, 1, 1, 128), bias=False, relu=False),                 # no bias, no activation: the accumulators as they are
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_through_the_dispatcher(oracle, block_forced, dtype, case):
    cs = CASES[case]
    g = h.rng(530 + case)
    xs, ws = cs["x"], cs["w"]
    s = shape_of(xs, ws)
    assert block_forced.avhip_conv2d_pointwise_block_plan(h.DT[dtype], C.byref(s), None, None) == 0, "the kernel must take this layer"
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64) if cs.get("bias", True) else None
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype) if cs.get("z") else None
    relu = cs.get("relu", True)
    a1, a2 = cs.get("alpha1"), cs.get("alpha2")
    before = transforms(block_forced)
    got = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, z=z, alpha1=a1, alpha2=a2, activation=cb.ACTIVATION_RELU if relu else 0, pad=(0, 0))
    assert transforms(block_forced) == before + 1, "the plan lays the weights out once; the other 1x1 kernels never do"
    want = oracle.conv2d(x, w, b, z=z, pad=(0, 0), alpha1=1.0 if a1 is None else a1, alpha2=1.0 if a2 is None else a2,
                         activation=oracle.RELU if relu else oracle.LINEAR)
    err = oracle.rel_l2(got, want)
    print("pixel-block %s case %d rel-L2 = %.3e" % (dtype, case, err))
    assert err < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_through_the_implicit_gemm_entry(oracle, block_forced, dtype):
    """cudaConvolutionImplicitGemmForward takes the same kernel: it is an implicit GEMM with the weights in another order."""
    cs = CASES[1]
    g = h.rng(470)
    xs, ws = cs["x"], cs["w"]
    pad, mode = cs.get("pad", (0, 0)), cs.get("mode", 0)
    s = shape_of(xs, ws, pad=pad)
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    before = transforms(block_forced)
    got = h.conv_forward("implicit_gemm", x, w, ys, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU, pad=(0, 0))
    assert transforms(block_forced) == before + 1, "the general kernels never lay weights out"
    want = oracle.conv2d(x, w, b, z=z, pad=(0, 0), activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("through the implicit-GEMM entry %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_kernel_layer_entry(oracle, dtype):
    """avhip_conv2d_pointwise_block_weight_layout + avhip_conv2d_pointwise_block called as a foreign host would: raw device pointers."""
    lib = cb.load_library()
    lib.avhip_conv2d_pointwise_block_weight_bytes.restype = C.c_int64
    g = h.rng(550)
    xs, ws = (3, 20, 22, 128), (512, 1, 1, 128)
    s = shape_of(xs, ws)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(ys), dtype)
    lib.avhip_conv2d_pointwise_block.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double,
                                                 C.c_double, C.c_double, C.c_int]
    lib.avhip_conv2d_pointwise_block_weight_layout.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    with h.Call() as c:
        xt, wt, zt, bt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(z, dtype), c.tensor(b, "f32")
        y = c.empty(ys, dtype)
        U = c.empty((lib.avhip_conv2d_pointwise_block_weight_bytes(ws[0], ws[3]) // 2,), dtype)
        stream = C.c_void_p(c.ctx.stream())
        assert lib.avhip_conv2d_pointwise_block_weight_layout(stream, h.DT[dtype], wt.pointer(), U.pointer(), ws[0], ws[3]) == 0
        args = (stream, h.DT[dtype], C.addressof(s), xt.pointer(), U.pointer(), bt.pointer(), zt.pointer(), y.pointer())
        assert lib.avhip_conv2d_pointwise_block(*args, 1.0, 1.0, 0.0, cb.ACTIVATION_RELU) == 0
        c.finish()
        got = y.download()
        assert lib.avhip_conv2d_pointwise_block(*args, 1.0, 1.0, 0.5, cb.ACTIVATION_RELU) == -1  # beta
        assert lib.avhip_conv2d_pointwise_block(*args, 1.0, 1.0, 0.0, cb.ACTIVATION_SIGMOID) == -1
        s3 = shape_of(xs, (512, 3, 3, 128), pad=(-1, -1))
        assert lib.avhip_conv2d_pointwise_block(stream, h.DT[dtype], C.addressof(s3), *args[3:], 1.0, 1.0, 0.0, 0) == -1  # 3x3
        assert lib.avhip_conv2d_pointwise_block(stream, h.DT["f32"], C.addressof(s), *args[3:], 1.0, 1.0, 0.0, 0) == -2
    want = oracle.conv2d(x, w, b, z=z, pad=(0, 0), activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("pixel-block kernel layer %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR


def test_plan_declines_what_the_kernel_cannot_run(block_forced):
    lib = block_forced
    ok = shape_of((64, 28, 28, 256), (512, 1, 1, 256))
    groups, rows = C.c_int(0), C.c_int(0)
    assert lib.avhip_conv2d_pointwise_block_plan(h.DT["bf16"], C.byref(ok), C.byref(groups), C.byref(rows)) == 0
    assert groups.value == 256 and rows.value == 196  # 50176 pixels: one block per compute unit
    for bad in (shape_of((64, 28, 28, 256), (512, 1, 1, 256), stride=(2, 2)), shape_of((64, 28, 28, 256), (512, 3, 3, 256), pad=(-1, -1)),
                shape_of((64, 28, 28, 64), (512, 1, 1, 64)), shape_of((64, 28, 28, 256), (256, 1, 1, 256)),
                shape_of((64, 28, 28, 256), (512, 1, 1, 256), pad=(-1, -1))):
        assert lib.avhip_conv2d_pointwise_block_plan(h.DT["bf16"], C.byref(bad), None, None) == -1
    assert lib.avhip_conv2d_pointwise_block_plan(h.DT["f32"], C.byref(ok), None, None) == -1
    lib.avhip_set_pointwise_block(0)
    assert lib.avhip_conv2d_pointwise_block_plan(h.DT["bf16"], C.byref(ok), None, None) == -1
    lib.avhip_set_pointwise_block(2)
