"""GPU parity of cudaGemm / cudaGemmBatched against the CPU oracle.  Shapes and scalars of the reference's tests
(test/test_gemm.cpp:16-130: 23 x 45 x 67, all four operand forms, alpha 1.1, beta 0.1) plus the batched (N, T) form at
Winograd shapes and the int8 -> int32 product of app/CudaBackend.cu:239."""
import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["b_resident", "both_through_lds"])
def short_k_engine(request):
    yield from h.short_k_engine_fixture(request)

TOL = {"f64": 1e-12, "f32": 2e-6, "f16": 4e-4, "bf16": 3e-3}  # 16-bit: the rounding of the result itself is 2.1e-4 / 1.7e-3 rel-L2


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f32", "f64"])
@pytest.mark.parametrize("opA", [False, True])
@pytest.mark.parametrize("opB", [False, True])
def test_gemm_23x45x67(oracle, dtype, opA, opB):
    g = h.rng(10)
    M, N, K = 23, 45, 67
    A = h.rounded(oracle, g.standard_normal((K, M) if opA else (M, K)), dtype)
    B = h.rounded(oracle, g.standard_normal((N, K) if opB else (K, N)), dtype)
    C0 = h.rounded(oracle, g.standard_normal((M, N)), dtype)
    a, b = (1.1, 0.1) if dtype == "f64" else (float(np.float32(1.1)), float(np.float32(0.1)))
    got = h.gemm(A, B, C0, dtype, opA, opB, a, b)
    want = oracle.gemm_batched(A, B, C0, opA, opB, a, b)
    assert oracle.rel_l2(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype,c_dtype", [("f32", "f32"), ("f16", "f16"), ("bf16", "bf16"), ("f16", "f32"), ("bf16", "f32"), ("f64", "f64")])
@pytest.mark.parametrize("shape", [(36, 128, 64, 64), (16, 200, 72, 40), (3, 23, 45, 67), (2, 300, 130, 136)])
def test_gemm_batched_nt(oracle, dtype, c_dtype, shape):
    """M[b] = V[b] U[b]^T: the matrix-core stage of non-fused Winograd (config 1 is 36 x 128 x 64 x 64); ragged sizes cover
    partial tiles in every dimension and leading dimensions that are not multiples of the vector width."""
    g = h.rng(11)
    batch, M, N, K = shape
    A = h.rounded(oracle, g.standard_normal((batch, M, K)), dtype)
    B = h.rounded(oracle, g.standard_normal((batch, N, K)), dtype)
    got = h.gemm(A, B, np.zeros((batch, M, N)), dtype, False, True, None, None, c_dtype=c_dtype, batched=True)
    want = oracle.gemm_batched(A, B, None, False, True)
    tol = TOL[c_dtype] if c_dtype != "f32" else 2e-6
    assert oracle.rel_l2(got, want) < tol


@pytest.mark.parametrize("dtype,c_dtype", [("f32", "f32"), ("f16", "f32"), ("bf16", "bf16"), ("bf16", "f32")])
def test_gemm_batched_nt_random_shapes(oracle, dtype, c_dtype):
    """Seeded random batched (N, T) products with alpha and beta: short k (the persistent kernel: one to four 128-byte steps,
    several rounds of tiles per workgroup, ragged last row block) and k, n that send the call to the one-tile kernel (k beyond
    four steps, n not a multiple of the 16-byte run)."""
    g = h.rng(13)
    esz = 4 if dtype == "f32" else 2
    for case in range(10):
        if case == 0:
            batch, M, N, K = 9, 64 * 130 + 7, 128, 96 // esz * 2     # more tiles than resident workgroups
        else:
            batch = int(g.integers(1, 6))
            M = int(g.integers(1, 700))
            N = int(g.choice([8, 24, 64, 128, 136, 200, 45]))
            K = int(g.choice([8, 16, 32, 64, 96, 128, 256, 67])) if case < 8 else int(g.choice([512, 384]))
        A = h.rounded(oracle, g.standard_normal((batch, M, K)), dtype)
        B = h.rounded(oracle, g.standard_normal((batch, N, K)), dtype)
        C0 = h.rounded(oracle, g.standard_normal((batch, M, N)), c_dtype)
        a, b = (float(np.float32(0.7)), float(np.float32(0.3))) if case % 2 else (None, None)
        print("gemm", dtype, c_dtype, batch, M, N, K, a, b, flush=True)
        got = h.gemm(A, B, C0, dtype, False, True, a, b, c_dtype=c_dtype, batched=True)
        want = oracle.gemm_batched(A, B, C0, False, True, a if a is not None else 1.0, b if b is not None else 0.0)
        tol = TOL[c_dtype] if c_dtype != "f32" else 2e-6
        assert oracle.rel_l2(got, want) < tol, (batch, M, N, K)


@pytest.mark.parametrize("opA,opB", [(False, False), (True, False), (True, True)])
def test_gemm_batched_other_forms(oracle, opA, opB):
    g = h.rng(12)
    batch, M, N, K = 3, 23, 45, 67
    A = g.standard_normal((batch, K, M) if opA else (batch, M, K)).astype(np.float32).astype(np.float64)
    B = g.standard_normal((batch, N, K) if opB else (batch, K, N)).astype(np.float32).astype(np.float64)
    C0 = g.standard_normal((batch, M, N)).astype(np.float32).astype(np.float64)
    a, b = float(np.float32(1.1)), float(np.float32(0.1))
    got = h.gemm(A, B, C0, "f32", opA, opB, a, b, batched=True)
    assert oracle.rel_l2(got, oracle.gemm_batched(A, B, C0, opA, opB, a, b)) < 2e-6


@pytest.mark.parametrize("shape", [(64, 128, 1152), (100, 36, 68)])
def test_gemm_int8_is_exact(oracle, shape):
    g = h.rng(13)
    M, N, K = shape
    A = g.integers(-127, 128, (M, K), dtype=np.int8)
    B = g.integers(-127, 128, (N, K), dtype=np.int8)
    got = h.gemm(A, B, np.zeros((M, N), dtype=np.int32), "i8", False, True, None, None, c_dtype="i32")
    want = A.astype(np.int64) @ B.astype(np.int64).T
    np.testing.assert_array_equal(got, want.astype(np.int32))
    # beta = 1 accumulates; the (N, N) form goes through the fallback kernel
    C0 = g.integers(-1000, 1000, (M, N)).astype(np.int32)
    Bn = np.ascontiguousarray(B.T)
    if N % 4 == 0:
        got = h.gemm(A, Bn, C0, "i8", False, False, 1.0, 1.0, c_dtype="i32")
        np.testing.assert_array_equal(got, (want + C0).astype(np.int32))


def test_gemm_argument_errors(oracle):
    A = np.zeros((8, 12), dtype=np.int8)
    B = np.zeros((8, 12), dtype=np.int8)
    C0 = np.zeros((8, 8), dtype=np.int32)
    h.gemm(A, B, C0, "i8", False, True, 2.0, None, c_dtype="i32", expect=cb.STATUS_BAD_PARAM)          # alpha must be 0 or 1 (reference gemm.cpp:51)
    h.gemm(np.zeros((8, 10), dtype=np.int8), np.zeros((8, 10), dtype=np.int8), C0, "i8", False, True, None, None, c_dtype="i32",
           expect=cb.STATUS_BAD_PARAM)                                                                  # leading dimension % 4 (reference gemm.cpp:46)
    h.gemm(np.zeros((4, 5)), np.zeros((6, 7)), np.zeros((4, 7)), "f32", expect=cb.STATUS_BAD_PARAM)     # inner dimensions differ
    h.gemm(np.zeros((4, 5)), np.zeros((5, 7)), np.zeros((4, 7)), "f32", c_dtype="f16", expect=cb.STATUS_UNSUPPORTED_DATATYPE)
