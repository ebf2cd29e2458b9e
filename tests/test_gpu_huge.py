"""Tensors beyond 2 GiB: the kernels' 32-bit-offset fast paths must hand such problems to the instances with 64-bit indexing.
Every image of a batch is independent, so images are generated, uploaded and checked one at a time against the CPU oracle:
the first, a middle and the last image (whose bytes lie beyond the 2 GiB mark) through the C API."""
import ctypes as C

import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu


def image(seed, shape, kind):
    g = np.random.default_rng(1000 + seed)
    if kind == "i8":
        return g.integers(-127, 128, shape, dtype=np.int8)
    return g.standard_normal(shape, dtype=np.float32).astype(np.float16)


def upload_images(lib, ctx, tensor, n_images, shape, kind):
    per = int(np.prod(shape)) * (1 if kind == "i8" else 2)
    for i in range(n_images):
        raw = np.ascontiguousarray(image(i, shape, kind))
        cb.check(lib.cudaCopyMemoryFromHost(ctx, tensor.mem, i * per, raw.ctypes.data_as(C.c_void_p), per), "upload")


def download_image(lib, ctx, tensor, index, shape, np_dtype):
    out = np.empty(shape, dtype=np_dtype)
    cb.check(lib.cudaCopyMemoryToHost(ctx, out.ctypes.data_as(C.c_void_p), tensor.mem, index * out.nbytes, out.nbytes), "download")
    return out


def test_int8_pointwise_beyond_2gib_bit_exact(oracle):
    N, H, W, Cin, K = 36, 1024, 1024, 64, 16          # x 2.42 GB int8, y 2.42 GB int32
    lib = cb.load_library()
    ctx = lib.cudaGetDefaultContext(0)
    g = h.rng(70)
    w = g.integers(-127, 128, (K, 1, 1, Cin), dtype=np.int8)
    b = g.integers(-2 ** 15, 2 ** 15, K).astype(np.int32)
    x = cb.DeviceTensor((N, H, W, Cin), cb.DTYPE_INT8, zero=False)
    y = cb.DeviceTensor((N, H, W, K), cb.DTYPE_INT32, zero=False)
    assert x.nbytes > 2 ** 31 and y.nbytes > 2 ** 31
    wt, bt = cb.DeviceTensor.from_numpy(w, cb.DTYPE_INT8), cb.DeviceTensor.from_numpy(b, cb.DTYPE_INT32)
    upload_images(lib, ctx, x, N, (H, W, Cin), "i8")
    conv = cb.ConvolutionDescriptor(padding=(0, 0), dtype=cb.DTYPE_INT8)
    print("int8 1x1 beyond 2 GiB", flush=True)
    cb.check(lib.cudaConvolutionImplicitGemmForward(ctx, conv.handle, None, x.desc, x.mem, wt.desc, wt.mem, bt.desc, bt.mem, None, 0, 0, None,
                                                     y.desc, y.mem, cb.ACTIVATION_RELU), "conv")
    cb.check(lib.cudaSynchronizeWithContext(ctx), "sync")
    for i in (0, N // 2, N - 1):
        got = download_image(lib, ctx, y, i, (H, W, K), np.int32)
        want = oracle.conv2d_i8(image(i, (1, H, W, Cin), "i8"), w, b, pad=(0, 0), activation=oracle.RELU)[0]
        np.testing.assert_array_equal(got, want)
    for t in (x, y, wt, bt):
        t.close()


def test_fp16_3x3_beyond_2gib(oracle):
    N, H, W, Cin, K = 9, 2048, 2048, 32, 8            # x 2.42 GB fp16
    lib = cb.load_library()
    ctx = lib.cudaGetDefaultContext(0)
    g = h.rng(71)
    w = h.rounded(oracle, g.standard_normal((K, 3, 3, Cin)) * np.sqrt(2.0 / (9 * Cin)), "f16")
    b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    x = cb.DeviceTensor((N, H, W, Cin), cb.DTYPE_FLOAT16, zero=False)
    y = cb.DeviceTensor((N, H, W, K), cb.DTYPE_FLOAT16, zero=False)
    assert x.nbytes > 2 ** 31
    wt, bt = cb.DeviceTensor.from_numpy(w, cb.DTYPE_FLOAT16), cb.DeviceTensor.from_numpy(b, cb.DTYPE_FLOAT32)
    upload_images(lib, ctx, x, N, (H, W, Cin), "f16")
    conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=cb.DTYPE_FLOAT16)
    print("fp16 3x3 beyond 2 GiB", flush=True)
    cb.check(lib.cudaConvolutionImplicitGemmForward(ctx, conv.handle, None, x.desc, x.mem, wt.desc, wt.mem, bt.desc, bt.mem, None, 0, 0, None,
                                                     y.desc, y.mem, cb.ACTIVATION_RELU), "conv")
    cb.check(lib.cudaSynchronizeWithContext(ctx), "sync")
    for i in (0, N - 1):
        got = download_image(lib, ctx, y, i, (H, W, K), np.float16).astype(np.float64)
        want = oracle.conv2d(image(i, (1, H, W, Cin), "f16").astype(np.float64), w, b, activation=oracle.RELU)[0]
        err = oracle.rel_l2(got, want)
        print("image %d rel-L2 = %.3e" % (i, err))
        assert err < 2e-3
    for t in (x, y, wt, bt):
        t.close()
