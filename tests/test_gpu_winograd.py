"""GPU parity of the non-fused Winograd transforms (forward: weight, input, output; weight gradient: gradient, update) and of
the whole non-fused pipelines, through the C API,
against the CPU oracle on identical seeded inputs.  Shapes follow the reference's own tests
(test/test_winograd.cpp:28,32-38,174: x {12,13,14,135}, w {21,3,3,135} / {21,5,5,135}, alpha1 1.1, alpha2 1.2, beta 0.1,
all four bias / residual combinations) plus channel counts that take the vectorised code path."""
import numpy as np
import pytest

import helpers as h

pytestmark = pytest.mark.gpu

# rel-L2 bound of one transform whose result is rounded once to the storage type
TOL = {"f64": 1e-12, "f32": 2e-6, "f16": 5e-4, "bf16": 3e-3}  # 16-bit: storing the result alone is 2.1e-4 / 1.7e-3 rel-L2
CASES = [(2, 3), (4, 3), (2, 5)]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("m,r", CASES)
@pytest.mark.parametrize("C", [135, 64])
def test_weight_transform(oracle, dtype, m, r, C):
    g = h.rng(1)
    w = h.rounded(oracle, g.standard_normal((21, r, r, C)) * 0.2, dtype)
    for mode in (0, 1):
        got = h.winograd_weight_transform(w, dtype, m, mode)
        want = oracle.winograd_weight_transform(w, m, invert=(mode == 1))
        assert oracle.rel_l2(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("m,r", CASES)
@pytest.mark.parametrize("shape", [(12, 13, 14, 135), (3, 15, 15, 64)])
def test_input_transform(oracle, dtype, m, r, shape):
    g = h.rng(2)
    x = h.rounded(oracle, g.standard_normal(shape), dtype)
    pad = (-(r // 2), -(r // 2))
    got = h.winograd_input_transform(x, (21, r, r, shape[3]), dtype, m, pad)
    want = oracle.winograd_input_transform(x, m, r, pad)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < TOL[dtype]


def test_input_transform_padding_value_and_offsets(oracle):
    g = h.rng(3)
    x = h.rounded(oracle, g.standard_normal((2, 9, 7, 12)), "f32")
    got = h.winograd_input_transform(x, (5, 3, 3, 12), "f32", 4, (0, -2), padding_value=0.75)
    want = oracle.winograd_input_transform(x, 4, 3, (0, -2), padding_value=0.75)
    assert oracle.rel_l2(got, want) < TOL["f32"]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("m,r", CASES)
@pytest.mark.parametrize("use_bias,use_z", [(True, True), (True, False), (False, True), (False, False)])
def test_output_transform(oracle, dtype, m, r, use_bias, use_z):
    g = h.rng(4)
    N, H, W, K = 12, 13, 14, 21
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    M = h.rounded(oracle, g.standard_normal((t * t, tiles, K)), dtype)
    bias = g.uniform(-0.1, 0.1, K) if use_bias else None
    if bias is not None and dtype != "f64":
        bias = bias.astype(np.float32).astype(np.float64)
    z = h.rounded(oracle, g.standard_normal((N, H, W, K)), dtype) if use_z else None
    y0 = h.rounded(oracle, g.standard_normal((N, H, W, K)), dtype)
    a1, a2, be = (1.1, 1.2, 0.1) if dtype == "f64" else (float(np.float32(1.1)), float(np.float32(1.2)), float(np.float32(0.1)))
    got = h.winograd_output_transform(M, (N, H, W, K), (K, r, r, 8), dtype, m, bias, z, y0, a1, a2, be, activation=3)
    want = oracle.winograd_output_transform(M, (N, H, W, K), m, r, bias, z, y0, a1, a2, be, oracle.RELU)
    assert oracle.rel_l2(got, want) < TOL[dtype]


def test_output_transform_vector_path_and_activations(oracle):
    g = h.rng(5)
    N, H, W, K = 3, 15, 15, 64
    M = h.rounded(oracle, g.standard_normal((36, N * 16, K)), "f32")
    bias = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    for act in range(9):
        got = h.winograd_output_transform(M * 0.2, (N, H, W, K), (K, 3, 3, 8), "f32", 4, bias, activation=act)
        want = oracle.winograd_output_transform(M * 0.2, (N, H, W, K), 4, 3, bias, activation=act)
        assert oracle.rel_l2(got, want) < 5e-6, act


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("use_bias,use_z,beta", [(True, True, 0.0), (True, False, 0.0), (False, True, 0.0), (True, True, 0.1)])
@pytest.mark.parametrize("shape", [(5, 15, 15, 64), (2, 13, 14, 72), (3, 9, 16, 8)])
def test_output_transform_sixteen_bit_matrices_wide_work_items(oracle, dtype, use_bias, use_z, beta, shape):
    """F(2x2, 3x3) with fp16 matrices and a filter count that divides by 8: small problems run with 8 filters per work-item
    (16-byte accesses); odd heights and widths exercise the clipped tiles.  Same bar as the narrow instance."""
    g = h.rng(41)
    N, H, W, K = shape
    tiles = N * ((H + 1) // 2) * ((W + 1) // 2)
    M = h.rounded(oracle, g.standard_normal((16, tiles, K)), "f16")
    bias = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64) if use_bias else None
    z = h.rounded(oracle, g.standard_normal(shape), dtype) if use_z else None
    y0 = h.rounded(oracle, g.standard_normal(shape), dtype)
    a1, a2, be = float(np.float32(1.1)), float(np.float32(1.2)), float(np.float32(beta))
    got = h.winograd_output_transform(M, shape, (K, 3, 3, 8), dtype, 2, bias, z, y0, a1, a2, be, activation=3, mat_dtype="f16")
    want = oracle.winograd_output_transform(M, shape, 2, 3, bias, z, y0, a1, a2, be, oracle.RELU)
    assert oracle.rel_l2(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("m,r", CASES)
@pytest.mark.parametrize("shape", [(12, 13, 14, 21), (3, 15, 15, 64)])
def test_gradient_transform(oracle, dtype, m, r, shape):
    """reference shapes test/test_winograd.cpp:101 (dy {12,13,14,21}) plus a vector-path channel count"""
    g = h.rng(7)
    dy = h.rounded(oracle, g.standard_normal(shape), dtype)
    got = h.winograd_gradient_transform(dy, (shape[3], r, r, 8), dtype, m)
    want = oracle.winograd_gradient_transform(dy, m, r)
    assert got.shape == want.shape
    assert oracle.rel_l2(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("m,r", CASES)
@pytest.mark.parametrize("C", [135, 64])
def test_update_transform(oracle, dtype, m, r, C):
    g = h.rng(8)
    K, t = 21, m + r - 1
    M = h.rounded(oracle, g.standard_normal((t * t, K, C)), dtype)
    got = h.winograd_update_transform(M, (K, r, r, C), dtype, m)
    want = oracle.winograd_update_transform(M, m, r)
    assert oracle.rel_l2(got, want) < TOL[dtype]
    dw0 = h.rounded(oracle, g.standard_normal((K, r, r, C)), dtype)
    a, b = (1.1, 0.1) if dtype == "f64" else (float(np.float32(1.1)), float(np.float32(0.1)))
    got = h.winograd_update_transform(M, (K, r, r, C), dtype, m, dw0, a, b)
    want = oracle.winograd_update_transform(M, m, r, dw0, a, b)
    assert oracle.rel_l2(got, want) < TOL[dtype]


@pytest.mark.parametrize("m,r", CASES)
def test_weight_gradient_pipeline_matches_direct_correlation(oracle, m, r):
    """dw through the Winograd domain (input transform of x, gradient transform of dy, batched GEMM (T, N) over the tiles,
    update transform) against the direct sum dw[k,i,j,c] = sum dy[n,h,w,k] * x[n,h+i-p,w+j-p,c] in fp64, fp32 tensors."""
    import cudabackend_amd as cb
    g = h.rng(9)
    N, H, W, Cin, K = 4, 15, 15, 32, 24
    x = h.rounded(oracle, g.standard_normal((N, H, W, Cin)), "f32")
    dy = h.rounded(oracle, g.standard_normal((N, H, W, K)), "f32")
    t, p = m + r - 1, r // 2
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=(-p, -p))
        xt, dyt = c.tensor(x, "f32"), c.tensor(dy, "f32")
        wt = c.empty((K, r, r, Cin), "f32")
        V, Mg, dU = c.empty((t * t, tiles, Cin), "f32"), c.empty((t * t, tiles, K), "f32"), c.empty((t * t, K, Cin), "f32")
        dw = c.empty((K, r, r, Cin), "f32")
        lib, ctx = c.lib, c.ctx.handle
        cb.check(lib.cudaWinogradInputTransform(ctx, conv.handle, m, wt.desc, xt.desc, xt.mem, V.desc, V.mem), "input")
        cb.check(lib.cudaWinogradGradientTransform(ctx, conv.handle, m, wt.desc, dyt.desc, dyt.mem, Mg.desc, Mg.mem), "gradient")
        cb.check(lib.cudaGemmBatched(ctx, cb.GEMM_OPERATION_T, cb.GEMM_OPERATION_N, None, Mg.desc, Mg.mem, V.desc, V.mem, None, dU.desc, dU.mem), "gemm")
        cb.check(lib.cudaWinogradUpdateTransform(ctx, conv.handle, m, None, dU.desc, dU.mem, None, dw.desc, dw.mem), "update")
        c.finish()
        got = dw.download()
    xp = np.pad(x, ((0, 0), (p, p), (p, p), (0, 0)))
    want = np.zeros((K, r, r, Cin))
    for i in range(r):
        for j in range(r):
            want[:, i, j, :] = np.einsum("nhwk,nhwc->kc", dy, xp[:, i:i + H, j:j + W, :])
    err = oracle.rel_l2(got, want)
    print("weight gradient F(%d,%d) rel-L2 = %.3e" % (m, r, err))
    assert err < 1e-4  # the fp32 Winograd bar


def test_unsupported_combinations_return_status(oracle):
    import cudabackend_amd as cb
    w = np.zeros((4, 5, 5, 8))
    h.winograd_weight_transform(w, "f32", 4, expect=cb.STATUS_NOT_SUPPORTED)  # F(4x4, 5x5) does not exist (reference :640-650)
    w7 = np.zeros((4, 7, 7, 8))
    h.winograd_weight_transform(w7, "f32", 2, expect=cb.STATUS_NOT_SUPPORTED)
    h.winograd_weight_transform(np.zeros((4, 3, 3, 8)), "f32", 2, mat_dtype="bf16", expect=cb.STATUS_UNSUPPORTED_DATATYPE)


@pytest.mark.parametrize("dtype,mat_dtype,m,tol", [
    ("f32", "f32", 4, 1e-4),   # fp32 Winograd bar
    ("f32", "f32", 2, 1e-4),
    ("f16", "f16", 2, 2e-3),   # 16-bit bar
    ("bf16", "f16", 2, 2e-3),  # bf16 tensors keep fp16 matrices: bf16 matrices would not meet the bar
    ("bf16", "f32", 4, 2e-3),
    ("f16", "f32", 4, 2e-3),
])
def test_nonfused_pipeline_matches_direct_convolution(oracle, dtype, mat_dtype, m, tol):
    """BASELINE config 1: N=8, 15x15, 64->64, inputs N(0,1), He-normal weights, bias U(-0.1,0.1), ReLU, run as the four-call
    sequence of app/CudaBackend.cu:401-420 (weight transform, input transform, batched GEMM (N,T), output transform)."""
    import cudabackend_amd as cb
    g = h.rng(6)
    N, H, W, Cin, K, r = 8, 15, 15, 64, 64, 3
    x = h.rounded(oracle, g.standard_normal((N, H, W, Cin)), dtype)
    w = h.rounded(oracle, g.standard_normal((K, r, r, Cin)) * np.sqrt(2.0 / (9 * Cin)), dtype)
    bias = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor()
        xt, wt, bt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(bias, "f32")
        U, V = c.empty((t * t, K, Cin), mat_dtype), c.empty((t * t, tiles, Cin), mat_dtype)
        # the product of two 16-bit matrices is kept in fp32 so that the output transform sees unrounded sums
        Mx = c.empty((t * t, tiles, K), "f32" if mat_dtype != "f64" else "f64")
        y = c.empty((N, H, W, K), dtype)
        lib, ctx = c.lib, c.ctx.handle
        cb.check(lib.cudaWinogradWeightTransform(ctx, conv.handle, m, wt.desc, wt.mem, U.desc, U.mem), "weight")
        cb.check(lib.cudaWinogradInputTransform(ctx, conv.handle, m, wt.desc, xt.desc, xt.mem, V.desc, V.mem), "input")
        cb.check(lib.cudaGemmBatched(ctx, cb.GEMM_OPERATION_N, cb.GEMM_OPERATION_T, None, V.desc, V.mem, U.desc, U.mem, None, Mx.desc, Mx.mem), "gemm")
        cb.check(lib.cudaWinogradOutputTransform(ctx, conv.handle, m, wt.desc, None, Mx.desc, Mx.mem, y.desc, y.mem, bt.desc, bt.mem, None, 0, 0, None,
                                                 cb.ACTIVATION_RELU), "output")
        c.finish()
        got = y.download()
    want = oracle.conv2d(x, w, bias, activation=oracle.RELU)
    err = oracle.rel_l2(got, want)
    print("nonfused %s/%s F(%d,3) rel-L2 = %.3e" % (dtype, mat_dtype, m, err))
    assert err < tol
