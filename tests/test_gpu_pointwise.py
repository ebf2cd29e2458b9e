"""GPU parity of 1x1 convolutions large enough that the persistent kernel's workgroups walk several tiles each (more than
2 x 256 tiles of 128 pixels x 128 filters), against the CPU oracle on identical seeded inputs, through the C API: ragged pixel
and filter counts, one to four k-steps per tile (the odd counts are padded with a step of zeros), residual, beta and both
int8 outputs.  Bars as everywhere: int8 bit-exact, fp32 rel-L2 <= 1e-5, fp16 / bf16 <= 2e-3."""
import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["b_resident", "both_through_lds"])
def short_k_engine(request):
    yield from h.short_k_engine_fixture(request)

BAR = {"f32": 1e-5, "f16": 2e-3, "bf16": 2e-3}

FLOAT_CASES = [
    # dtype, x shape, filters, what the epilogue carries
    ("bf16", (4, 63, 63, 192), 648, "bias+z+relu"),   # 125 x 6 = 750 tiles, 3 k-steps
    ("f16", (2, 90, 90, 64), 640, "plain"),           # 127 x 5 = 635 tiles, 1 k-step
    ("f32", (4, 63, 63, 96), 520, "bias+beta"),       # 125 x 5 = 625 tiles, 3 k-steps
    ("bf16", (3, 75, 75, 256), 512, "bias+relu"),     # 132 x 4 = 528 tiles, 4 k-steps
    ("f32", (1, 40, 40, 32), 136, "bias+relu"),       # 13 x 2 tiles: fewer tiles than resident workgroups
    ("bf16", (1, 37, 41, 64), 72, "bias+z+relu"),     # one step; 1517 pixels: ranges that end in a partial granule
    ("f16", (2, 100, 100, 128), 128, "bias+relu"),    # two steps, one column block: 512 ranges of 40 rows (one short tile each)
]


@pytest.mark.parametrize("dtype,xs,K,what", FLOAT_CASES, ids=["%s-%s" % (c[0], c[3]) for c in FLOAT_CASES])
def test_pointwise_float(oracle, dtype, xs, K, what):
    g = h.rng(61)
    N, H, W, Cin = xs
    x = h.rounded(oracle, g.standard_normal(xs), dtype)
    w = h.rounded(oracle, g.standard_normal((K, 1, 1, Cin)) * np.sqrt(2.0 / Cin), dtype)
    bias = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64) if "bias" in what else None
    z = h.rounded(oracle, g.standard_normal((N, H, W, K)), dtype) if "+z" in what else None
    y0 = h.rounded(oracle, g.standard_normal((N, H, W, K)), dtype) if "beta" in what else None
    act = cb.ACTIVATION_RELU if "relu" in what else cb.ACTIVATION_LINEAR
    a2 = float(np.float32(0.7)) if z is not None else None
    be = float(np.float32(0.3)) if y0 is not None else None
    print("pointwise", dtype, xs, K, what, flush=True)
    got = h.conv_forward("implicit_gemm", x, w, (N, H, W, K), dtype, bias=bias, z=z, y0=y0, alpha2=a2, beta=be, activation=act, pad=(0, 0))
    want = oracle.conv2d(x, w, bias, z, y0, pad=(0, 0), alpha2=a2 if a2 is not None else 1.0, beta=be if be is not None else 0.0, activation=act)
    err = oracle.rel_l2(got, want)
    print("rel-L2 = %.3e" % err)
    assert err < BAR[dtype]


@pytest.mark.parametrize("Cin,K", [(128, 648), (64, 640), (192, 520)], ids=["1step", "halfstep", "2steps"])
def test_pointwise_int8_bit_exact(oracle, Cin, K):
    g = h.rng(62)
    xs = (4, 63, 63, Cin)
    x = g.integers(-127, 128, xs, dtype=np.int8)
    w = g.integers(-127, 128, (K, 1, 1, Cin), dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    scale = g.uniform(1e-4, 1e-3, K).astype(np.float32)
    ys = (4, 63, 63, K)
    print("pointwise int8", xs, K, flush=True)
    for act in (cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU):
        acc = oracle.conv2d_i8(x, w, b, pad=(0, 0), activation=act)
        got = h.conv_forward("implicit_gemm", x, w, ys, "i8", y_dtype="i32", bias=b, bias_dtype="i32", activation=act, pad=(0, 0))
        np.testing.assert_array_equal(got, acc)
        got = h.conv_forward("requant", x, w, ys, "i8", y_dtype="i8", bias=b, bias_dtype="i32", scale=scale, activation=act, pad=(0, 0))
        np.testing.assert_array_equal(got, oracle.requant_i8(acc, scale))
