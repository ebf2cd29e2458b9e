"""GPU parity of the row-wise Winograd F(2,3) kernel (16-bit 3x3 stride-1 layers whose image bands fit a compute unit's LDS):
its weight transform against the closed form, the kernel through the kernel-layer C-ABI and through the dispatcher against the
CPU oracle on identical seeded inputs.  Bar: rel-L2 <= 2e-3 for fp16 / bf16 (the layer's bar; nothing tighter is claimed)."""
import ctypes as C

import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu

BAR = 2e-3
G = np.array([[1, 0, 0], [0.5, 0.5, 0.5], [0.5, -0.5, 0.5], [0, 0, 1]], dtype=np.float64)


class Shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("N", "H", "W", "C", "K", "R", "S", "Ho", "Wo", "pad_h", "pad_w", "stride_h", "stride_w", "dil_h", "dil_w",
                                       "mode")]


def shape_of(x, w, pad=(-1, -1), stride=(1, 1), dilation=(1, 1), mode=0):
    N, H, W, Cin = x
    K, R, S, _ = w
    Ho = (H + 2 * (-pad[0]) - ((R - 1) * dilation[0] + 1)) // stride[0] + 1
    Wo = (W + 2 * (-pad[1]) - ((S - 1) * dilation[1] + 1)) // stride[1] + 1
    return Shape(N, H, W, Cin, K, R, S, Ho, Wo, pad[0], pad[1], stride[0], stride[1], dilation[0], dilation[1], mode)


@pytest.fixture
def rows_forced():
    """The dispatcher takes the row-Winograd kernel for every layer it can run, whatever its size."""
    lib = cb.load_library()
    lib.avhip_set_winograd_rows.restype = int
    previous = lib.avhip_set_winograd_rows(2)
    yield lib
    lib.avhip_set_winograd_rows(previous)


def transforms(lib):
    n = C.c_int64(0)
    assert lib.avhipGetWeightCacheState(None, None, C.byref(n)) == cb.STATUS_SUCCESS
    return n.value


def he(g, shape, dtype, orc):
    K, R, S, Cin = shape
    return h.rounded(orc, g.standard_normal(shape) * np.sqrt(2.0 / (R * S * Cin)), dtype)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("mode", [0, 1])
def test_weight_transform_layout(oracle, dtype, mode):
    """U_p[i] = sum_j G[p][j] w[k, i, j] (taps reversed in the flipping mode), fp16, in the register layout of the kernel's MFMA
    operand: [C / 32][3][4][K / 32][2][64 lanes][8], lane l = filter l % 32, channels 8 * (l / 32) .. + 7 of the 16-channel slab."""
    lib = cb.load_library()
    lib.avhip_winograd_rows_weight_bytes.restype = C.c_int64
    K, Cin = 128, 64
    g = h.rng(311)
    w = he(g, (K, 3, 3, Cin), dtype, oracle)
    nbytes = lib.avhip_winograd_rows_weight_bytes(K, Cin)
    assert nbytes == 12 * K * Cin * 2
    with h.Call() as c:
        wt = c.tensor(w, dtype)
        U = c.empty((nbytes // 2,), "f16")
        stream = C.c_void_p(c.ctx.stream())
        lib.avhip_winograd_rows_weight_transform.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
        assert lib.avhip_winograd_rows_weight_transform(stream, h.DT[dtype], mode, wt.pointer(), U.pointer(), K, Cin) == 0
        c.finish()
        got = U.download().reshape(Cin // 32, 3, 4, K // 32, 2, 64, 8)
    ww = w[:, ::-1, ::-1, :] if mode else w
    want = np.einsum("pj,kijc->pikc", G, ww)  # [p, i, K, C]
    want = want.reshape(4, 3, K // 32, 32, Cin // 32, 2, 2, 8)  # p, i, tile, filter, phase, slab, half, 8
    want = want.transpose(4, 1, 0, 2, 5, 6, 3, 7).reshape(Cin // 32, 3, 4, K // 32, 2, 64, 8)  # lane = half * 32 + filter
    want16 = want.astype(np.float32).astype(np.float16).astype(np.float64)
    assert np.max(np.abs(got - want16)) <= 2.0 ** -10 * np.max(np.abs(want16))
    assert oracle.rel_l2(got, want) < 5e-4


ROWS_CASES = [
    # x, w, keyword arguments
    dict(x=(6, 15, 15, 128), w=(128, 3, 3, 128)),                                        # BASELINE config 2 body layer, a few images
    dict(x=(3, 15, 15, 128), w=(256, 3, 3, 128), z=True, relu=False, alpha1=1.1, alpha2=1.2),  # two filter blocks, test/test_winograd.cpp:32-38 scalars
    dict(x=(4, 14, 14, 64), w=(128, 3, 3, 64), mode=1),                                  # one 64-channel slice, flipped taps
    dict(x=(3, 20, 20, 128), w=(128, 3, 3, 128), z=True),                                # two bands per image
    dict(x=(2, 28, 28, 128), w=(128, 3, 3, 128)),                                        # four bands, 14 pairs
    dict(x=(3, 15, 13, 128), w=(128, 3, 3, 128), pad=(0, 0)),                            # no padding: 13 x 11 outputs, odd width
    dict(x=(3, 9, 31, 64), w=(128, 3, 3, 64), pad=(-2, -1)),                             # asymmetric offsets: rows outside the image on both sides
    dict(x=(2, 56, 56, 64), w=(128, 3, 3, 64)),                                          # wide rows: bands of two rows
    dict(x=(2, 5, 7, 128), w=(128, 3, 3, 128), z=True),                                  # an image much smaller than a workgroup's tile
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(ROWS_CASES)))
def test_through_the_dispatcher(oracle, rows_forced, dtype, case):
    cs = ROWS_CASES[case]
    g = h.rng(330 + case)
    xs, ws = cs["x"], cs["w"]
    pad, mode = cs.get("pad", (-1, -1)), cs.get("mode", 0)
    s = shape_of(xs, ws, pad=pad, mode=mode)
    assert rows_forced.avhip_conv2d_winograd_rows_plan(h.DT[dtype], C.byref(s), None, None) == 0, "the kernel must take this layer"
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype) if cs.get("z") else None
    relu = cs.get("relu", True)
    a1, a2 = cs.get("alpha1"), cs.get("alpha2")
    before = transforms(rows_forced)
    got = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, z=z, alpha1=a1, alpha2=a2, activation=cb.ACTIVATION_RELU if relu else 0, pad=pad, mode=mode)
    assert transforms(rows_forced) == before + 1, "the row-Winograd plan transforms the weights once; the direct kernels never do"
    want = oracle.conv2d(x, w, b, z=z, pad=pad, mode=mode, alpha1=1.0 if a1 is None else a1, alpha2=1.0 if a2 is None else a2,
                         activation=oracle.RELU if relu else oracle.LINEAR)
    err = oracle.rel_l2(got, want)
    print("rows %s case %d rel-L2 = %.3e" % (dtype, case, err))
    assert err < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("channels", [64, 128, 256])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("residual", [False, True])
def test_every_instance_of_the_kernel(oracle, rows_forced, dtype, channels, relu, residual):
    """The kernel is instantiated per tensor type, channel count (2, 4 or 8 phases), activation and residual: every one of the 24
    on a small layer with two bands per image and a ragged last band."""
    g = h.rng(370 + channels + 2 * relu + residual)
    xs, ws = (3, 19, 14, channels), (128, 3, 3, channels)
    s = shape_of(xs, ws)
    assert rows_forced.avhip_conv2d_winograd_rows_plan(h.DT[dtype], C.byref(s), None, None) == 0, "the kernel must take this layer"
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype) if residual else None
    got = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, z=z, alpha1=0.9, alpha2=1.3 if residual else None,
                         activation=cb.ACTIVATION_RELU if relu else 0)
    want = oracle.conv2d(x, w, b, z=z, alpha1=0.9, alpha2=1.3 if residual else 1.0, activation=oracle.RELU if relu else oracle.LINEAR)
    err = oracle.rel_l2(got, want)
    print("rows instance %s C=%d relu=%d z=%d rel-L2 = %.3e" % (dtype, channels, relu, residual, err))
    assert err < BAR


ROUNDS_CASES = [
    # layers of more workgroups than the device has compute units (several rounds of workgroups)
    dict(x=(70, 28, 28, 64), w=(128, 3, 3, 64)),                                          # 280 workgroups
    dict(x=(44, 20, 20, 128), w=(512, 3, 3, 128), z=True),                                # 2 bands x 4 filter blocks x 44 images = 352, residual
    dict(x=(10, 56, 56, 256), w=(256, 3, 3, 256), relu=False),                            # config 3's layer on 10 images: 140 tiles x 2 filter blocks, eight phases
]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(ROUNDS_CASES)))
def test_several_rounds_of_workgroups(oracle, rows_forced, dtype, case):
    cs = ROUNDS_CASES[case]
    g = h.rng(390 + case)
    xs, ws = cs["x"], cs["w"]
    s = shape_of(xs, ws)
    groups = C.c_int(0)
    assert rows_forced.avhip_conv2d_winograd_rows_plan(h.DT[dtype], C.byref(s), C.byref(groups), None) == 0
    assert groups.value > 256, "the case must be more than one round of workgroups on the 256 compute units of an MI355X"
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    ys = (xs[0], s.Ho, s.Wo, ws[0])
    z = h.rounded(oracle, g.standard_normal(ys), dtype) if cs.get("z") else None
    relu = cs.get("relu", True)
    got = h.conv_forward("dispatch", x, w, ys, dtype, bias=b, z=z, activation=cb.ACTIVATION_RELU if relu else 0)
    want = oracle.conv2d(x, w, b, z=z, activation=oracle.RELU if relu else oracle.LINEAR)
    err = oracle.rel_l2(got, want)
    print("rows rounds %s case %d rel-L2 = %.3e" % (dtype, case, err))
    assert err < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_kernel_layer_entry(oracle, dtype):
    """avhip_winograd_rows_weight_transform + avhip_conv2d_winograd_rows called as a foreign host would: raw device pointers."""
    lib = cb.load_library()
    lib.avhip_winograd_rows_weight_bytes.restype = C.c_int64
    g = h.rng(350)
    xs, ws = (5, 15, 15, 128), (128, 3, 3, 128)
    x = h.rounded(oracle, np.maximum(g.standard_normal(xs), 0), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, 128).astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal(xs), dtype)
    s = shape_of(xs, ws)
    conv_args = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_double, C.c_double, C.c_double, C.c_int]
    lib.avhip_conv2d_winograd_rows.argtypes = conv_args
    lib.avhip_winograd_rows_weight_transform.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int]
    with h.Call() as c:
        xt, wt, zt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(z, dtype)
        bt = c.tensor(b, "f32")
        y = c.empty(xs, dtype)
        U = c.empty((lib.avhip_winograd_rows_weight_bytes(128, 128) // 2,), "f16")
        stream = C.c_void_p(c.ctx.stream())
        assert lib.avhip_winograd_rows_weight_transform(stream, h.DT[dtype], 0, wt.pointer(), U.pointer(), 128, 128) == 0
        args = (stream, h.DT[dtype], C.addressof(s), xt.pointer(), U.pointer(), bt.pointer(), zt.pointer(), y.pointer())
        assert lib.avhip_conv2d_winograd_rows(*args, 1.0, 1.0, 0.0, cb.ACTIVATION_RELU) == 0
        c.finish()
        got = y.download()
        # what the kernel does not do is declined with nothing launched
        assert lib.avhip_conv2d_winograd_rows(*args, 1.0, 1.0, 0.5, cb.ACTIVATION_RELU) == -1  # beta
        assert lib.avhip_conv2d_winograd_rows(*args, 1.0, 1.0, 0.0, cb.ACTIVATION_TANH) == -1
        s2 = shape_of((5, 15, 15, 96), (128, 3, 3, 96))
        assert lib.avhip_conv2d_winograd_rows(stream, h.DT[dtype], C.addressof(s2), *args[3:], 1.0, 1.0, 0.0, 0) == -1  # C = 96
        assert lib.avhip_conv2d_winograd_rows(stream, h.DT["f32"], C.addressof(s), *args[3:], 1.0, 1.0, 0.0, 0) == -2
    want = oracle.conv2d(x, w, b, z=z, activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("rows kernel layer %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR


def test_plan_declines_what_the_kernel_cannot_run(rows_forced):
    lib = rows_forced
    ok = shape_of((4, 15, 15, 128), (128, 3, 3, 128))
    groups, rows = C.c_int(0), C.c_int(0)
    assert lib.avhip_conv2d_winograd_rows_plan(h.DT["bf16"], C.byref(ok), C.byref(groups), C.byref(rows)) == 0
    assert groups.value == 4 and rows.value == 120  # one workgroup per image; 15 rows x 8 pairs of its 128 GEMM rows
    for bad in (shape_of((4, 15, 15, 128), (128, 3, 3, 128), stride=(2, 2)), shape_of((4, 15, 15, 128), (128, 5, 5, 128), pad=(-2, -2)),
                shape_of((4, 15, 15, 96), (128, 3, 3, 96)), shape_of((4, 15, 15, 128), (64, 3, 3, 128)),
                shape_of((4, 15, 15, 128), (128, 3, 3, 128), pad=(-2, -2), dilation=(2, 2))):
        assert lib.avhip_conv2d_winograd_rows_plan(h.DT["bf16"], C.byref(bad), None, None) == -1
    assert lib.avhip_conv2d_winograd_rows_plan(h.DT["f32"], C.byref(ok), None, None) == -1
    lib.avhip_set_winograd_rows(0)
    assert lib.avhip_conv2d_winograd_rows_plan(h.DT["bf16"], C.byref(ok), None, None) == -1
    lib.avhip_set_winograd_rows(2)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_epilogues_the_kernel_leaves_to_the_direct_kernels(oracle, rows_forced, dtype):
    """beta != 0 and the seven non-trivial activations: the dispatcher must not take the row-Winograd plan and the result stays right."""
    g = h.rng(360)
    xs, ws = (3, 15, 15, 128), (128, 3, 3, 128)
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = he(g, ws, dtype, oracle)
    b = g.uniform(-0.1, 0.1, 128).astype(np.float32).astype(np.float64)
    y0 = h.rounded(oracle, g.standard_normal(xs), dtype)
    before = transforms(rows_forced)
    got = h.conv_forward("dispatch", x, w, xs, dtype, bias=b, y0=y0, beta=0.1, activation=cb.ACTIVATION_RELU)
    assert oracle.rel_l2(got, oracle.conv2d(x, w, b, y=y0, beta=0.1, activation=oracle.RELU)) < BAR
    got = h.conv_forward("dispatch", x, w, xs, dtype, bias=b, activation=cb.ACTIVATION_TANH)
    assert oracle.rel_l2(got, oracle.conv2d(x, w, b, activation=oracle.TANH)) < BAR
    assert transforms(rows_forced) == before


def test_large_magnitudes_within_the_fp16_range(oracle, rows_forced):
    """The transformed input is held in fp16: bf16 activations up to a few thousand keep the bar (the documented domain of the plan
    is |x| < 3e4)."""
    g = h.rng(370)
    xs, ws = (3, 15, 15, 128), (128, 3, 3, 128)
    x = h.rounded(oracle, g.standard_normal(xs) * 2000.0, "bf16")
    w = he(g, ws, "bf16", oracle)
    got = h.conv_forward("dispatch", x, w, xs, "bf16", activation=0)
    assert oracle.rel_l2(got, oracle.conv2d(x, w)) < BAR


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_through_the_fused_winograd_entry(oracle, rows_forced, dtype):
    """cudaConvolutionWinogradFusedForward on 16-bit tensors takes the row-wise kernel where it can: the transformed weights it
    caches then have the row-wise layout's size (12 K C fp16 values), not the two-dimensional one's (16 K C)."""
    lib = rows_forced
    g = h.rng(480)
    xs, ws = (3, 15, 15, 128), (128, 3, 3, 128)
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = h.rounded(oracle, g.standard_normal(ws) * np.sqrt(2.0 / (9 * ws[3])), dtype)
    b = g.uniform(-0.1, 0.1, ws[0]).astype(np.float32).astype(np.float64)
    ys = (xs[0], xs[1], xs[2], ws[0])
    nbytes = C.c_int64(0)
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=h.DT[dtype])
        xt, wt, bt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(b, "f32")
        y = c.empty(ys, dtype)
        assert lib.avhipGetWeightCacheState(None, C.byref(nbytes), None) == cb.STATUS_SUCCESS
        before = nbytes.value
        cb.check(lib.cudaConvolutionWinogradFusedForward(c.ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, bt.desc, bt.mem, None, 0, 0,
                                                          None, y.desc, y.mem, cb.ACTIVATION_RELU), "fused Winograd entry")
        assert lib.avhipGetWeightCacheState(None, C.byref(nbytes), None) == cb.STATUS_SUCCESS
        assert nbytes.value - before == 12 * ws[0] * ws[3] * 2, "the new cache entry has the row-wise layout's size"
        c.finish()
        got = y.download()
    want = oracle.conv2d(x, w, b, activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("through the fused-Winograd entry %s rel-L2 = %.3e" % (dtype, err))
    assert err < BAR
