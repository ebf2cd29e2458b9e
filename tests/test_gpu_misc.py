"""GPU tests of the helpers around the convolution path: add-bias, im2row, type conversion, memory and context entries."""
import ctypes as C

import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,tol", [("f16", 1e-3), ("bf16", 1e-2), ("f32", 1e-4), ("f64", 1e-4)])
def test_add_bias_reference_case(oracle, dtype, tol):
    """test/test_tensor_op.cpp:151-198: {23,45,67}, alpha1 1.1, alpha2 1.2, beta1 0.1, beta2 0.2, beta3 0.3, same tolerances."""
    g = h.rng(30)
    x = h.rounded(oracle, g.standard_normal((23, 45, 67)), dtype)
    z = h.rounded(oracle, g.standard_normal((23, 45, 67)), dtype)
    y0 = h.rounded(oracle, g.standard_normal((23, 45, 67)), dtype)
    b = g.standard_normal(67)
    b = b if dtype == "f64" else b.astype(np.float32).astype(np.float64)
    s = (lambda v: v) if dtype == "f64" else (lambda v: float(np.float32(v)))
    args = [s(1.1), s(1.2), s(0.1), s(0.2), s(0.3)]
    for act in (cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU, cb.ACTIVATION_SIGMOID, cb.ACTIVATION_TANH):
        got = h.add_bias(x, b, dtype, z, y0, *args, activation=act)
        want = oracle.add_bias(x, b, z, y0, *args, activation=act)
        assert oracle.rel_l2(got, want) < tol
    # vectorised path (last dimension a multiple of 4), no z, no y
    x4 = h.rounded(oracle, g.standard_normal((50, 128)), dtype)
    b4 = g.standard_normal(128).astype(np.float32).astype(np.float64)
    got = h.add_bias(x4, b4, dtype, activation=cb.ACTIVATION_RELU)
    assert oracle.rel_l2(got, oracle.add_bias(x4, b4, activation=oracle.RELU)) < tol


@pytest.mark.parametrize("R,pad,dtype", [(3, (-1, -1), "f32"), (5, (-2, -2), "f32"), (3, (-1, -1), "bf16"), (3, (-1, -1), "i8")])
@pytest.mark.parametrize("mode", [0, 1])
def test_im2row(oracle, R, pad, dtype, mode):
    """test/test_im2row.cpp:16-29: x {12,23,34,45}, 11 filters, 3x3 offset -1 and 5x5 offset -2 (batch reduced to 3)."""
    g = h.rng(31)
    shape = (3, 23, 34, 45)
    if dtype == "i8":
        x = g.integers(-127, 128, shape, dtype=np.int8)
    else:
        x = h.rounded(oracle, g.standard_normal(shape), dtype)
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(mode=mode, padding=pad)
        xt = c.tensor(x, dtype)
        wt = c.empty((11, R, R, 45), dtype)
        rows = c.empty((3 * 23 * 34, R * R * 45), dtype)
        cb.check(c.lib.cudaIm2Row(c.ctx.handle, conv.handle, wt.desc, xt.desc, xt.mem, rows.desc, rows.mem), "cudaIm2Row")
        c.finish()
        got = rows.download()
    want = oracle.im2row(np.asarray(x, dtype=np.float64), R, R, pad, mode)
    np.testing.assert_array_equal(np.asarray(got, dtype=np.float64), want)


@pytest.mark.parametrize("R,pad,stride,dilation", [(3, (-1, -1), (2, 2), (1, 1)), (3, (-2, -2), (1, 1), (2, 2)), (3, (-1, 0), (2, 1), (1, 2)), (5, (-2, -1), (3, 2), (1, 1))])
@pytest.mark.parametrize("dtype", ["f32", "bf16", "i8"])
def test_im2row_strides_and_dilations(oracle, R, pad, stride, dilation, dtype):
    """Strides, dilations and asymmetric offsets (the cases test/test_im2row.cpp:31-48 leaves commented out), bit-exact against
    the oracle; then rows x flattened filters through cudaGemm against the implicit-GEMM convolution of the same geometry."""
    g = h.rng(33)
    shape = (3, 23, 34, 16)
    K = 24
    if dtype == "i8":
        x = g.integers(-127, 128, shape, dtype=np.int8)
        w = g.integers(-127, 128, (K, R, R, shape[3]), dtype=np.int8)
    else:
        x = h.rounded(oracle, g.standard_normal(shape), dtype)
        w = h.rounded(oracle, g.standard_normal((K, R, R, shape[3])) * 0.2, dtype)
    Ho, Wo = oracle.conv_output_shape(shape[1], shape[2], R, R, pad, stride, dilation)
    out_dtype = "i32" if dtype == "i8" else dtype
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=pad, strides=stride, dilation=dilation, dtype=h.DT[dtype])
        xt, wt = c.tensor(x, dtype), c.tensor(w, dtype)
        rows = c.empty((3 * Ho * Wo, R * R * shape[3]), dtype)
        cb.check(c.lib.cudaIm2Row(c.ctx.handle, conv.handle, wt.desc, xt.desc, xt.mem, rows.desc, rows.mem), "cudaIm2Row")
        wflat = c.tensor(np.asarray(w).reshape(K, -1), dtype)
        prod = c.empty((3 * Ho * Wo, K), out_dtype)
        cb.check(c.lib.cudaGemm(c.ctx.handle, cb.GEMM_OPERATION_N, cb.GEMM_OPERATION_T, None, rows.desc, rows.mem, wflat.desc, wflat.mem, None, prod.desc, prod.mem),
                 "cudaGemm")
        y = c.empty((3, Ho, Wo, K), out_dtype)
        cb.check(c.lib.cudaConvolutionImplicitGemmForward(c.ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, 0, 0, None, 0, 0, None,
                                                          y.desc, y.mem, cb.ACTIVATION_LINEAR), "implicit GEMM")
        c.finish()
        got, explicit, implicit = rows.download(), prod.download(), y.download()
    want = oracle.im2row(np.asarray(x, dtype=np.float64), R, R, pad, 0, 0.0, stride, dilation)
    np.testing.assert_array_equal(np.asarray(got, dtype=np.float64), want)
    explicit = np.asarray(explicit, dtype=np.float64).reshape(3, Ho, Wo, K)
    implicit = np.asarray(implicit, dtype=np.float64)
    if dtype == "i8":
        np.testing.assert_array_equal(explicit, implicit)
        np.testing.assert_array_equal(implicit, oracle.conv2d_i8(x, w, pad=pad, stride=stride, dilation=dilation))
    else:
        assert oracle.rel_l2(explicit, implicit) < (1e-5 if dtype == "f32" else 4e-3)


def test_change_type(oracle):
    g = h.rng(32)
    v = np.concatenate([g.standard_normal(1000) * 50, [0.5, 1.5, 2.5, -0.5, -1.5, 127.5, 300.0, -300.0, 1e10, -1e10]]).astype(np.float32)
    import torch
    with h.Call() as c:
        src = c.tensor(v, "f32")
        n = v.size
        for dst_dtype, want in [
            (cb.DTYPE_FLOAT16, v.astype(np.float16).astype(np.float64)),
            (cb.DTYPE_BFLOAT16, torch.tensor(v).to(torch.bfloat16).to(torch.float64).numpy()),
            (cb.DTYPE_INT8, np.clip(np.rint(v.astype(np.float64)), -128, 127)),
            (cb.DTYPE_INT32, np.clip(np.rint(v.astype(np.float64)), -2 ** 31, 2 ** 31 - 1)),
            (cb.DTYPE_FLOAT64, v.astype(np.float64)),
        ]:
            dst = c.empty((n,), dst_dtype)
            cb.check(c.lib.cudaChangeType(c.ctx.handle, dst.mem, dst_dtype, src.mem, cb.DTYPE_FLOAT32, n), "cudaChangeType")
            c.finish()
            np.testing.assert_array_equal(np.asarray(dst.download(), dtype=np.float64), want)
        # and back up: bf16 / int8 -> fp32 are exact
        i8 = c.tensor(g.integers(-128, 128, 777, dtype=np.int8), "i8")
        f = c.empty((777,), "f32")
        cb.check(c.lib.cudaChangeType(c.ctx.handle, f.mem, cb.DTYPE_FLOAT32, i8.mem, cb.DTYPE_INT8, 777), "cudaChangeType")
        c.finish()
        np.testing.assert_array_equal(f.download(), i8.download().astype(np.float64))


def test_memory_entries():
    lib = cb.load_library()
    assert lib.cudaGetNumberOfDevices() >= 1
    name = C.create_string_buffer(256)
    cb.check(lib.cudaGetDeviceProperty(0, cb.DEVICE_NAME, name), "name")
    cus = C.c_int32(0)
    cb.check(lib.cudaGetDeviceProperty(0, cb.DEVICE_PROCESSOR_COUNT, C.byref(cus)), "cus")
    mem = C.c_int64(0)
    cb.check(lib.cudaGetDeviceProperty(0, cb.DEVICE_MEMORY, C.byref(mem)), "memory")
    print("device:", name.value.decode(), cus.value, "CUs", mem.value >> 30, "GiB")
    assert cus.value > 0 and mem.value > 0
    ctx = cb.Context(0)
    dflt = lib.cudaGetDefaultContext(0)
    m = C.c_int64(0)
    cb.check(lib.cudaCreateMemoryDescriptor(C.byref(m), 0, 4096), "alloc")
    # pattern fills of every width, checked on the host
    for width in (1, 2, 4, 8, 16):
        pattern = bytes(range(1, width + 1))
        cb.check(lib.cudaSetMemory(ctx.handle, m.value, 0, 4096, pattern, width), "set")
        ctx.synchronize()
        host = np.empty(4096, dtype=np.uint8)
        cb.check(lib.cudaCopyMemoryToHost(dflt, host.ctypes.data_as(C.c_void_p), m.value, 0, 4096), "d2h")
        np.testing.assert_array_equal(host, np.tile(np.frombuffer(pattern, dtype=np.uint8), 4096 // width))
    assert lib.cudaSetMemory(ctx.handle, m.value, 0, 4095, b"\1\2", 2) == cb.STATUS_BAD_PARAM          # size not a multiple of the pattern
    assert lib.cudaSetMemory(ctx.handle, m.value, 0, 8192, None, 0) == cb.STATUS_BAD_PARAM             # beyond the block
    cb.check(lib.cudaSetMemory(dflt, m.value, 100, 1000, None, 0), "zero")
    host = np.empty(4096, dtype=np.uint8)
    cb.check(lib.cudaCopyMemoryToHost(dflt, host.ctypes.data_as(C.c_void_p), m.value, 0, 4096), "d2h")
    assert host[100:1100].sum() == 0 and host[99] != 0 and host[1100] != 0
    # view + device-to-device copy
    v = C.c_int64(0)
    cb.check(lib.cudaCreateMemoryView(C.byref(v), m.value, 1024, 2048), "view")
    assert lib.cudaCreateMemoryView(C.byref(C.c_int64(0)), v.value, 16, 0) == cb.STATUS_BAD_PARAM        # views of views are refused
    assert lib.cudaCreateMemoryView(C.byref(C.c_int64(0)), m.value, 4096, 1) == cb.STATUS_BAD_PARAM
    src = np.arange(1024, dtype=np.uint8)
    cb.check(lib.cudaCopyMemoryFromHost(dflt, v.value, 0, src.ctypes.data_as(C.c_void_p), 1024), "h2d")
    cb.check(lib.cudaCopyMemory(ctx.handle, m.value, 0, v.value, 0, 1024), "d2d")
    ctx.synchronize()
    cb.check(lib.cudaCopyMemoryToHost(dflt, host.ctypes.data_as(C.c_void_p), m.value, 0, 4096), "d2h")
    np.testing.assert_array_equal(host[:1024], src)
    np.testing.assert_array_equal(host[2048:3072], src)
    ready = C.c_bool(False)
    cb.check(lib.cudaIsContextReady(ctx.handle, C.byref(ready)), "ready")
    assert ready.value
    assert lib.cudaCopyMemoryToHost(dflt, None, m.value, 0, 4) == cb.STATUS_BAD_PARAM
    cb.check(lib.cudaDestroyMemoryDescriptor(v.value), "free view")
    cb.check(lib.cudaDestroyMemoryDescriptor(m.value), "free")
    assert lib.cudaDestroyMemoryDescriptor(m.value) == cb.STATUS_BAD_PARAM
    assert lib.cudaDestroyContextDescriptor(dflt) == cb.STATUS_BAD_PARAM                                # the default context cannot be destroyed
    ctx.close()


@pytest.mark.parametrize("dtype,tol", [("f16", 1e-3), ("bf16", 1e-2), ("f32", 1e-6), ("f64", 1e-13)])
def test_affine_forward_and_batchnorm_inference(oracle, dtype, tol):
    """src/batchnorm.cu:28-69: y = alpha * act(x * s + t) + beta * y per channel; folded batch normalisation.  Ragged and
    vector-friendly channel counts, parameters spanning one or two trailing dimensions."""
    g = h.rng(60)
    sfun = (lambda v: v) if dtype == "f64" else (lambda v: float(np.float32(v)))
    par = (lambda a: a) if dtype == "f64" else (lambda a: a.astype(np.float32).astype(np.float64))
    for shape, pshape in (((3, 7, 5, 13), (13,)), ((4, 6, 6, 64), (64,)), ((5, 3, 8), (3, 8))):
        x = h.rounded(oracle, g.standard_normal(shape), dtype)
        y0 = h.rounded(oracle, g.standard_normal(shape), dtype)
        w, b, mean = par(g.standard_normal(pshape)), par(g.standard_normal(pshape)), par(g.standard_normal(pshape))
        var = par(g.uniform(0.2, 2.0, pshape))
        for act in (cb.ACTIVATION_LINEAR, cb.ACTIVATION_RELU, cb.ACTIVATION_SIGMOID):
            got = h.affine_forward(x, w, b, dtype, y0, sfun(1.1), sfun(0.3), activation=act)
            assert oracle.rel_l2(got, oracle.affine_forward(x, w, b, y0, sfun(1.1), sfun(0.3), activation=act)) < tol
            got = h.batchnorm_inference(x, w, b, mean, var, dtype, None, None, None, 1e-3, activation=act)
            assert oracle.rel_l2(got, oracle.batchnorm_inference(x, w, b, mean, var, epsilon=1e-3, activation=act)) < tol * 3
    x = np.zeros((2, 4, 8))
    h.affine_forward(x, np.zeros(5), np.zeros(5), "f32", expect=cb.STATUS_BAD_PARAM)  # 5 does not divide 64
    h.affine_forward(x.astype(np.int32), np.zeros(8), np.zeros(8), "i32", expect=cb.STATUS_UNSUPPORTED_DATATYPE)


def test_measurement_probes_run_and_validate_arguments():
    """The two measurement aids of the kernel layer: they launch, leave the device healthy and refuse nonsense."""
    import ctypes as C
    lib = cb.load_library()
    lib.avhip_mfma_rate_probe.restype = C.c_int
    lib.avhip_mfma_rate_probe.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    lib.avhip_stream_probe.restype = C.c_int
    lib.avhip_stream_probe.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int64]
    ctx = cb.Context(0)
    sink = cb.DeviceTensor((64 * 256,), cb.DTYPE_FLOAT32)
    for dtype in (cb.DTYPE_BFLOAT16, cb.DTYPE_FLOAT16, cb.DTYPE_INT8, cb.DTYPE_FLOAT32):
        for operands in (0, 1):
            assert lib.avhip_mfma_rate_probe(ctx.stream(), dtype, 64, 16, operands, sink.pointer()) == 0
    assert lib.avhip_mfma_rate_probe(ctx.stream(), cb.DTYPE_FLOAT64, 64, 16, 0, sink.pointer()) != 0
    assert lib.avhip_mfma_rate_probe(ctx.stream(), cb.DTYPE_BFLOAT16, 0, 16, 0, sink.pointer()) != 0
    assert lib.avhip_mfma_rate_probe(ctx.stream(), cb.DTYPE_BFLOAT16, 64, 16, 2, sink.pointer()) != 0
    n = 1 << 20
    a = cb.DeviceTensor.from_numpy(np.arange(n, dtype=np.int32), cb.DTYPE_INT32)
    b = cb.DeviceTensor((n,), cb.DTYPE_INT32)
    assert lib.avhip_stream_probe(ctx.stream(), 2, a.pointer(), b.pointer(), 4 * n) == 0
    assert lib.avhip_stream_probe(ctx.stream(), 0, a.pointer(), sink.pointer(), 4 * n) == 0
    assert lib.avhip_stream_probe(ctx.stream(), 1, None, sink.pointer(), 4 * 64 * 256) == 0
    assert lib.avhip_stream_probe(ctx.stream(), 3, a.pointer(), b.pointer(), 4 * n) != 0
    assert lib.avhip_stream_probe(ctx.stream(), 2, None, b.pointer(), 4 * n) != 0
    assert lib.avhip_stream_probe(ctx.stream(), 2, a.pointer(), b.pointer(), 64) != 0
    ctx.synchronize()
    got = b.download()
    # the copy moves everything but at most the last 16 KiB
    np.testing.assert_array_equal(got[:n - 4096], np.arange(n - 4096, dtype=np.int32))
    for t in (a, b, sink):
        t.close()
    ctx.close()

