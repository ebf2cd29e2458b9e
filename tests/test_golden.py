"""Golden fixtures of tests/golden/ (written by tests/golden/make_fixtures.py from the pinned CPU oracle).

CPU part: the oracle still reproduces every fixture exactly (a change of the oracle cannot go unnoticed).
GPU part: the HIP path, through the C API, matches the fixtures to the bars of the task: int8 bit-exact, fp32 implicit GEMM
rel-L2 <= 1e-5, fp32 Winograd <= 1e-4, fp16 / bf16 <= 2e-3."""
import glob
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as f:
        return {k: f[k] for k in f.files}


CONV = ["conv_f32_3x3_same", "conv_f32_5x5_flipped_stride2", "conv_bf16_3x3_dilated", "conv_f16_1x1", "conv_bf16_stem_4_planes"]
INT8 = ["int8_3x3", "int8_1x1", "int8_3x3_stride2_flipped"]
WINOGRAD = ["winograd_f4_nonfused", "winograd_f2_nonfused"]


def conv_kwargs(c):
    return dict(pad=tuple(int(v) for v in c["pad"]), stride=tuple(int(v) for v in c["stride"]), mode=int(c["mode"]))


def test_every_fixture_is_covered():
    names = sorted(os.path.splitext(os.path.basename(p))[0] for p in glob.glob(os.path.join(GOLDEN, "*.npz")))
    assert names == sorted(CONV + INT8 + WINOGRAD)


@pytest.mark.parametrize("name", CONV)
def test_oracle_reproduces_conv_fixture(oracle, name):
    c = load(name)
    kw = conv_kwargs(c)
    kw["dilation"] = tuple(int(v) for v in c["dilation"])
    z = c["z"].astype(np.float64) if "z" in c else None
    y = oracle.conv2d(c["x"].astype(np.float64), c["w"].astype(np.float64), c["bias"].astype(np.float64), z, activation=int(c["activation"]), **kw)
    np.testing.assert_array_equal(y, c["y"])


@pytest.mark.parametrize("name", INT8)
def test_oracle_reproduces_int8_fixture(oracle, name):
    c = load(name)
    acc = oracle.conv2d_i8(c["x"], c["w"], c["bias"], activation=oracle.RELU, **conv_kwargs(c))
    np.testing.assert_array_equal(acc, c["y_i32"])
    np.testing.assert_array_equal(oracle.requant_i8(acc, c["scale"]), c["y_i8"])


@pytest.mark.parametrize("name", WINOGRAD)
def test_oracle_reproduces_winograd_fixture(oracle, name):
    c = load(name)
    m, pad = int(c["m"]), tuple(int(v) for v in c["pad"])
    x, w = c["x"].astype(np.float64), c["w"].astype(np.float64)
    np.testing.assert_array_equal(oracle.winograd_weight_transform(w, m), c["U"])
    np.testing.assert_array_equal(oracle.winograd_input_transform(x, m, 3, pad), c["V"])
    # the fixture's end result is the convolution itself (Winograd identity), to rounding
    direct = oracle.conv2d(x, w, c["bias"].astype(np.float64), pad=pad, activation=oracle.RELU)
    assert oracle.rel_l2(c["y"], direct) < 1e-12


# ---------------------------------------------------------------------------------------------------------------- GPU
BAR = {"f32": 1e-5, "f16": 2e-3, "bf16": 2e-3}


@pytest.mark.gpu
@pytest.mark.parametrize("name", CONV)
def test_hip_matches_conv_fixture(oracle, name):
    import helpers as h
    c = load(name)
    dtype = str(c["dtype"])
    kw = conv_kwargs(c)
    kw["dilation"] = tuple(int(v) for v in c["dilation"])
    z = c["z"].astype(np.float64) if "z" in c else None
    for entry in ("implicit_gemm", "dispatch"):
        got = h.conv_forward(entry, c["x"].astype(np.float64), c["w"].astype(np.float64), c["y"].shape, dtype, bias=c["bias"].astype(np.float64), z=z,
                             activation=int(c["activation"]), **kw)
        # the dispatcher may pick a Winograd kernel for fp32 3x3 stride-1 cases: Winograd bar
        bar = 1e-4 if (entry == "dispatch" and dtype == "f32") else BAR[dtype]
        assert oracle.rel_l2(got, c["y"]) < bar, entry


@pytest.mark.gpu
@pytest.mark.parametrize("name", INT8)
def test_hip_matches_int8_fixture(oracle, name):
    import cudabackend_amd as cb
    import helpers as h
    c = load(name)
    kw = conv_kwargs(c)
    got = h.conv_forward("implicit_gemm", c["x"], c["w"], c["y_i32"].shape, "i8", y_dtype="i32", bias=c["bias"], bias_dtype="i32",
                         activation=cb.ACTIVATION_RELU, **kw)
    np.testing.assert_array_equal(got, c["y_i32"])
    q = h.conv_forward("requant", c["x"], c["w"], c["y_i8"].shape, "i8", y_dtype="i8", bias=c["bias"], bias_dtype="i32", scale=c["scale"],
                       activation=cb.ACTIVATION_RELU, **kw)
    np.testing.assert_array_equal(q, c["y_i8"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", WINOGRAD)
def test_hip_matches_winograd_fixture(oracle, name):
    import cudabackend_amd as cb
    import helpers as h
    c = load(name)
    m, pad = int(c["m"]), tuple(int(v) for v in c["pad"])
    x, w, b = c["x"].astype(np.float64), c["w"].astype(np.float64), c["bias"].astype(np.float64)
    U = h.winograd_weight_transform(w, "f32", m)
    V = h.winograd_input_transform(x, w.shape, "f32", m, pad)
    assert oracle.rel_l2(U, c["U"]) < 1e-6
    assert oracle.rel_l2(V, c["V"]) < 1e-6
    M = h.gemm(V, U, np.zeros(c["M"].shape), "f32", opB=True, batched=True)
    assert oracle.rel_l2(M, c["M"]) < 1e-5
    y = h.winograd_output_transform(M, c["y"].shape, w.shape, "f32", m, bias=b, activation=cb.ACTIVATION_RELU)
    assert oracle.rel_l2(y, c["y"]) < 1e-4
    fused = h.conv_forward("winograd_fused", x, w, c["y"].shape, "f32", bias=b, activation=cb.ACTIVATION_RELU, pad=pad)
    assert oracle.rel_l2(fused, c["y"]) < 1e-4
