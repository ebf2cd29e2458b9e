"""CPU-only checks of the boundary: the shared library loads without a GPU, exports every symbol the headers declare, and its
host-side descriptor logic and argument validation behave as the reference's C API documents."""
import ctypes as C
import os
import re

import pytest

import cudabackend_amd as cb

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b((?:cuda|avhip)[A-Za-z_0-9]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    lib = cb.load_library()
    api = declared_symbols("avocado_hip_backend.h")
    kernels = declared_symbols("avocado_hip_kernels.h")
    assert len(api) >= 40 and len(kernels) == 35
    for name in sorted(api | kernels):
        assert hasattr(lib, name), name
    # the Python binding covers the whole API header
    assert api == set(cb.api.PROTOTYPES)
    assert kernels == set(cb.api.KERNEL_LAYER_SYMBOLS)


def test_missing_library_is_an_error(tmp_path):
    with pytest.raises(FileNotFoundError):
        cb.load_library(str(tmp_path / "libavocado_hip.so"))


def test_tensor_descriptor_roundtrip():
    lib = cb.load_library()
    d = C.c_int64(0)
    cb.check(lib.cudaCreateTensorDescriptor(C.byref(d)))
    dims = (C.c_int * 4)(12, 13, 14, 135)
    cb.check(lib.cudaSetTensorDescriptor(d.value, cb.DTYPE_BFLOAT16, 4, dims))
    dtype, nb, out = C.c_int(0), C.c_int(0), (C.c_int * 8)()
    cb.check(lib.cudaGetTensorDescriptor(d.value, C.byref(dtype), C.byref(nb), out))
    assert dtype.value == cb.DTYPE_BFLOAT16 and nb.value == 4 and list(out)[:4] == [12, 13, 14, 135]
    assert lib.cudaSetTensorDescriptor(d.value, cb.DTYPE_FLOAT32, 9, dims) == cb.STATUS_BAD_PARAM      # more than 8 dimensions
    assert lib.cudaSetTensorDescriptor(d.value, cb.DTYPE_FLOAT32, 2, None) == cb.STATUS_BAD_PARAM
    cb.check(lib.cudaSetTensorDescriptor(d.value, cb.DTYPE_FLOAT32, 0, None))
    cb.check(lib.cudaDestroyTensorDescriptor(d.value))
    assert lib.cudaDestroyTensorDescriptor(d.value) == cb.STATUS_BAD_PARAM
    assert lib.cudaGetTensorDescriptor(d.value, None, None, None) == cb.STATUS_BAD_PARAM
    assert lib.cudaCreateTensorDescriptor(None) == cb.STATUS_BAD_PARAM


def test_convolution_descriptor_defaults_and_roundtrip():
    lib = cb.load_library()
    d = C.c_int64(0)
    cb.check(lib.cudaCreateConvolutionDescriptor(C.byref(d)))
    # null arrays mean padding 0, stride 1, dilation 1 (reference header :758-762)
    cb.check(lib.cudaSetConvolutionDescriptor(d.value, cb.CROSS_CORRELATION_MODE, 2, None, None, None, 1, None))
    mode, nb, groups = C.c_int(0), C.c_int(0), C.c_int(0)
    pad, st, dil = (C.c_int * 3)(9, 9, 9), (C.c_int * 3)(9, 9, 9), (C.c_int * 3)(9, 9, 9)
    pv = C.create_string_buffer(16)
    cb.check(lib.cudaGetConvolutionDescriptor(d.value, C.byref(mode), C.byref(nb), pad, st, dil, C.byref(groups), pv))
    assert (mode.value, nb.value, groups.value) == (cb.CROSS_CORRELATION_MODE, 2, 1)
    assert list(pad)[:2] == [0, 0] and list(st)[:2] == [1, 1] and list(dil)[:2] == [1, 1] and pv.raw == b"\0" * 16
    value = C.create_string_buffer(bytes(range(16)), 16)
    cb.check(lib.cudaSetConvolutionDescriptor(d.value, cb.CONVOLUTION_MODE, 2, (C.c_int * 2)(-1, -2), (C.c_int * 2)(2, 3), (C.c_int * 2)(1, 2), 1, value))
    cb.check(lib.cudaGetConvolutionDescriptor(d.value, C.byref(mode), C.byref(nb), pad, st, dil, C.byref(groups), pv))
    assert list(pad)[:2] == [-1, -2] and list(st)[:2] == [2, 3] and list(dil)[:2] == [1, 2] and pv.raw == bytes(range(16))
    assert lib.cudaSetConvolutionDescriptor(d.value, cb.CONVOLUTION_MODE, 4, None, None, None, 1, None) == cb.STATUS_BAD_PARAM
    assert lib.cudaSetConvolutionDescriptor(d.value, cb.CONVOLUTION_MODE, 2, None, None, None, 0, None) == cb.STATUS_BAD_PARAM
    cb.check(lib.cudaDestroyConvolutionDescriptor(d.value))
    assert lib.cudaDestroyConvolutionDescriptor(d.value) == cb.STATUS_BAD_PARAM


def test_handles_are_typed():
    lib = cb.load_library()
    t = C.c_int64(0)
    cb.check(lib.cudaCreateTensorDescriptor(C.byref(t)))
    assert lib.cudaDestroyConvolutionDescriptor(t.value) == cb.STATUS_BAD_PARAM
    assert lib.cudaDestroyMemoryDescriptor(t.value) == cb.STATUS_BAD_PARAM
    assert lib.cudaDestroyContextDescriptor(t.value) == cb.STATUS_BAD_PARAM
    assert lib.cudaSynchronizeWithContext(t.value) == cb.STATUS_BAD_PARAM
    cb.check(lib.cudaDestroyTensorDescriptor(t.value))


@pytest.mark.skipif(cb.load_library().cudaGetNumberOfDevices() > 0, reason="checks the no-GPU behaviour")
def test_no_device_paths_fail_with_status_codes():
    lib = cb.load_library()
    assert lib.cudaGetNumberOfDevices() == 0
    assert lib.cudaGetDefaultContext(0) == -1
    h = C.c_int64(0)
    assert lib.cudaCreateContextDescriptor(C.byref(h), 0) == cb.STATUS_BAD_PARAM
    assert lib.cudaCreateMemoryDescriptor(C.byref(h), 0, 16) == cb.STATUS_BAD_PARAM
    # a compute entry with an invalid context is refused before anything is launched
    assert lib.cudaGemm(-1, 0, 0, None, 0, 0, 0, 0, None, 0, 0) == cb.STATUS_BAD_PARAM
    assert lib.cudaConvolutionImplicitGemmForward(-1, 0, None, 0, 0, 0, 0, 0, 0, None, 0, 0, None, 0, 0, 0) == cb.STATUS_BAD_PARAM
    buf = C.create_string_buffer(256)
    assert lib.cudaGetDeviceProperty(0, cb.DEVICE_NAME, buf) == cb.STATUS_BAD_PARAM


def test_page_lock_is_reported_as_not_supported():
    lib = cb.load_library()
    buf = C.create_string_buffer(64)
    assert lib.cudaPageLock(None, 64) == cb.STATUS_BAD_PARAM
    assert lib.cudaPageLock(buf, 64) == cb.STATUS_NOT_SUPPORTED
    assert lib.cudaPageUnlock(buf) == cb.STATUS_NOT_SUPPORTED


def test_copy_possible_only_within_one_device():
    lib = cb.load_library()
    r = C.c_bool(False)
    cb.check(lib.cudaIsCopyPossible(0, 0, C.byref(r)))
    assert r.value
    cb.check(lib.cudaIsCopyPossible(0, 1, C.byref(r)))
    assert not r.value
    assert lib.cudaIsCopyPossible(0, 0, None) == cb.STATUS_BAD_PARAM


def test_headers_compile_as_c_and_cxx_and_link(tmp_path):
    """A front-end written in C or C++ includes <Avocado/cuda_backend.h> and links the shared library: the headers must be
    valid in both languages and every entry point must resolve at link time (the program only calls what works without a GPU)."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib_dir = os.path.join(root, "cudabackend_amd")
    if not os.path.exists(os.path.join(lib_dir, "libavocado_hip.so")):
        pytest.skip("library not built")
    c_src = tmp_path / "front_end.c"
    c_src.write_text('#include <stdio.h>\n#include "avocado_hip_backend.h"\n#include "avocado_hip_kernels.h"\n'
                     'int main(void) {\n'
                     '  avTensorDescriptor_t t; int dims[4] = {2, 3, 4, 5};\n'
                     '  if (cudaCreateTensorDescriptor(&t) != AVOCADO_STATUS_SUCCESS) return 1;\n'
                     '  if (cudaSetTensorDescriptor(t, AVOCADO_DTYPE_FLOAT32, 4, dims) != AVOCADO_STATUS_SUCCESS) return 2;\n'
                     '  if (cudaDestroyTensorDescriptor(t) != AVOCADO_STATUS_SUCCESS) return 3;\n'
                     '  printf("devices %d\\n", cudaGetNumberOfDevices());\n'
                     '  return avhip_conv2d_implicit_gemm(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1.0, 1.0, 0.0, 0, 0) == AVHIP_BAD_PARAM ? 0 : 4;\n}\n')
    cxx_src = tmp_path / "front_end.cpp"
    cxx_src.write_text('#include <Avocado/cuda_backend.h>\nusing namespace avocado::backend;\n'
                       'int main() { avConvolutionDescriptor_t c; if (cudaCreateConvolutionDescriptor(&c) != AVOCADO_STATUS_SUCCESS) return 1;\n'
                       '  return cudaDestroyConvolutionDescriptor(c) == AVOCADO_STATUS_SUCCESS ? 0 : 2; }\n')
    env = dict(os.environ, LD_LIBRARY_PATH=lib_dir + ":/opt/rocm/lib:" + os.environ.get("LD_LIBRARY_PATH", ""))
    for compiler, src, exe in (("gcc", c_src, tmp_path / "c_front"), ("g++", cxx_src, tmp_path / "cxx_front")):
        cmd = [compiler, "-Wall", "-Werror", "-I", os.path.join(root, "include"), str(src), "-o", str(exe), "-L", lib_dir, "-lavocado_hip",
               "-Wl,-rpath," + lib_dir, "-Wl,-rpath-link,/opt/rocm/lib"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stdout + r.stderr
        r = subprocess.run([str(exe)], capture_output=True, text=True, env=env)
        assert r.returncode == 0, "exit %d: %s%s" % (r.returncode, r.stdout, r.stderr)


def test_descriptor_tables_survive_concurrent_callers():
    """Eight host threads create, set, read back and destroy descriptors at once (ctypes releases the interpreter lock
    during a call): every handle is unique while it lives, every read-back returns what its own thread wrote, and a
    destroyed handle is refused.  Host logic only; no device is touched."""
    import threading
    lib = cb.load_library()
    live, lock, errors = set(), threading.Lock(), []

    def worker(seed):
        try:
            for i in range(400):
                t, c = C.c_int64(0), C.c_int64(0)
                cb.check(lib.cudaCreateTensorDescriptor(C.byref(t)))
                cb.check(lib.cudaCreateConvolutionDescriptor(C.byref(c)))
                with lock:
                    assert t.value not in live and c.value not in live and t.value != c.value
                    live.update((t.value, c.value))
                dims = (C.c_int * 4)(seed + 1, i + 1, 7, 9)
                cb.check(lib.cudaSetTensorDescriptor(t.value, cb.DTYPE_FLOAT16, 4, dims))
                pad = (C.c_int * 2)(-seed, -i)
                cb.check(lib.cudaSetConvolutionDescriptor(c.value, cb.CONVOLUTION_MODE, 2, pad, None, None, 1, None))
                dtype, nb, out = C.c_int(0), C.c_int(0), (C.c_int * 8)()
                cb.check(lib.cudaGetTensorDescriptor(t.value, C.byref(dtype), C.byref(nb), out))
                assert dtype.value == cb.DTYPE_FLOAT16 and nb.value == 4 and list(out)[:4] == [seed + 1, i + 1, 7, 9]
                with lock:
                    live.difference_update((t.value, c.value))
                cb.check(lib.cudaDestroyTensorDescriptor(t.value))
                cb.check(lib.cudaDestroyConvolutionDescriptor(c.value))
        except Exception as e:  # noqa: BLE001 - collected and re-raised in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors[0]


class ConvShape(C.Structure):
    """avhipConvShape of include/avocado_hip_kernels.h."""
    _fields_ = [(n, C.c_int) for n in ("N", "H", "W", "C", "K", "R", "S", "Ho", "Wo", "pad_h", "pad_w", "stride_h", "stride_w", "dil_h", "dil_w", "mode")]


def split_k_bytes(lib, dtype, N, H, Cin, K, R, stride=1):
    pad = -(R // 2)
    Ho = (H - 2 * pad - R) // stride + 1
    s = ConvShape(N, H, H, Cin, K, R, R, Ho, Ho, pad, pad, stride, stride, 1, 1, 0)
    out = C.c_int64(-1)
    lib.avhip_conv2d_split_k_workspace.argtypes = [C.c_int, C.POINTER(ConvShape), C.POINTER(C.c_int64)]
    assert lib.avhip_conv2d_split_k_workspace(dtype, C.byref(s), C.byref(out)) == 0
    return out.value, N * Ho * Ho * K * 4


def test_split_k_plan_is_for_few_pixels_and_a_long_k():
    """The host-side plan of the split-k implicit GEMM (no GPU involved): partial sums of two or more parts for the last stages
    of a deep network at a modest batch, nothing for layers that fill the chip, that are short in k, that the small-problem
    kernel takes, or whose tensors the branch-free loaders cannot read."""
    lib = cb.load_library()
    bf16, f32, i8 = cb.DTYPE_BFLOAT16, cb.DTYPE_FLOAT32, cb.DTYPE_INT8
    got, plane = split_k_bytes(lib, bf16, 32, 7, 512, 512, 3)           # 3x3 512->512 on 32 images of 7x7
    assert got >= 2 * plane and got % plane == 0
    got, plane = split_k_bytes(lib, bf16, 32, 14, 512, 512, 3, stride=2)
    assert got >= 2 * plane
    got, plane = split_k_bytes(lib, f32, 32, 14, 256, 256, 3)           # fp32: half the compute units would idle for 8x the MFMA time
    assert got >= 2 * plane
    assert split_k_bytes(lib, bf16, 256, 15, 128, 128, 3)[0] == 0       # BASELINE config 2: 900 tiles of 128 x 128
    assert split_k_bytes(lib, bf16, 32, 14, 256, 256, 3)[0] == 0        # the image-tile kernel's pace is hard to beat
    assert split_k_bytes(lib, bf16, 32, 14, 256, 1024, 1)[0] == 0       # four k-steps
    assert split_k_bytes(lib, f32, 8, 15, 64, 64, 3)[0] == 0            # BASELINE config 1: the small-problem kernel's
    assert split_k_bytes(lib, bf16, 4, 7, 512, 512, 3)[0] == 0          # tiny batch: the small-problem kernel's
    assert split_k_bytes(lib, i8, 32, 7, 512, 512, 3)[0] == 0           # floating types only
    assert split_k_bytes(lib, bf16, 32, 7, 500, 512, 3)[0] == 0         # 1000 bytes of channels: not whole 16-byte chunks
    assert split_k_bytes(lib, bf16, 32, 7, 512, 512, 7)[0] == 0         # 49 taps: beyond the loaders' tap mask
    s = ConvShape(0, 7, 7, 512, 512, 3, 3, 7, 7, -1, -1, 1, 1, 1, 1, 0)
    out = C.c_int64(0)
    assert lib.avhip_conv2d_split_k_workspace(bf16, C.byref(s), C.byref(out)) != 0      # N = 0
    assert lib.avhip_conv2d_split_k_workspace(bf16, None, C.byref(out)) != 0


def test_weight_cache_eviction_policy():
    """The rule by which the cache of transformed weights makes room, on made-up buffers (no device involved): least recently used
    first, never a buffer that a captured graph holds (flag 1) or that a call has looked up and not yet launched for (flag 2), and no
    more than needed."""
    import ctypes as C
    lib = cb.load_library()

    def probe(sizes, last_use, flags, budget, incoming):
        n = len(sizes)
        evicted = (C.c_int32 * n)()
        st = lib.avhipWeightCachePolicyProbe(n, (C.c_int64 * n)(*sizes), (C.c_int64 * n)(*last_use), (C.c_int32 * n)(*flags), budget, incoming, evicted)
        assert st == cb.STATUS_SUCCESS
        return list(evicted)
    # everything fits: nothing goes
    assert probe([10, 10, 10], [1, 2, 3], [0, 0, 0], 100, 10) == [0, 0, 0]
    # 10 more bytes need one buffer gone: the one used longest ago
    assert probe([10, 10, 10], [5, 2, 9], [0, 0, 0], 30, 10) == [0, 1, 0]
    # 25 more need all three
    assert probe([10, 10, 10], [5, 2, 9], [0, 0, 0], 30, 25) == [1, 1, 1]
    # the oldest is held by a graph, the next by a call in flight: the third goes although it is the most recent, and then the rule stops
    assert probe([10, 10, 10], [1, 2, 9], [1, 2, 0], 30, 25) == [0, 0, 1]
    # nothing can go: the rule leaves everything (the cache then exceeds its budget rather than free memory in use)
    assert probe([10, 10], [1, 2], [1, 3], 5, 100) == [0, 0]
    # a budget of zero empties the cache of what is free to go
    assert probe([10, 10, 10, 10], [4, 3, 2, 1], [0, 1, 0, 2], 0, 0) == [1, 0, 1, 0]
    assert lib.avhipWeightCachePolicyProbe(1, None, None, None, 1, 1, None) == cb.STATUS_BAD_PARAM


class _Shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("N", "H", "W", "C", "K", "R", "S", "Ho", "Wo", "pad_h", "pad_w", "stride_h", "stride_w", "dil_h", "dil_w",
                                       "mode")]


def _shape(x, w, pad, stride=1):
    Ho, Wo = (x[1] - 2 * pad - w[1]) // stride + 1, (x[2] - 2 * pad - w[2]) // stride + 1  # pad is the (negative) offset of the first tap
    return _Shape(x[0], x[1], x[2], x[3], w[0], w[1], w[2], Ho, Wo, pad, pad, stride, stride, 1, 1, 0)


def test_plans_of_the_one_kernel_convolutions():
    """What the dispatcher weighs for the three kernels that keep their pixel operand in LDS and take the filters from L2 — the
    number of workgroups and how many of a workgroup's GEMM rows are real — is host arithmetic: checked here on the BASELINE shapes
    and on what each kernel must decline."""
    lib = cb.load_library()
    bf16, f32 = cb.DTYPE_BFLOAT16, cb.DTYPE_FLOAT32
    groups, rows = C.c_int(0), C.c_int(0)

    def plan(fn, dtype, s):
        rc = fn(dtype, C.byref(s), C.byref(groups), C.byref(rows))
        return (groups.value, rows.value) if rc == 0 else rc

    rw = lib.avhip_conv2d_winograd_rows_plan
    assert plan(rw, bf16, _shape((256, 15, 15, 128), (128, 3, 3, 128), -1)) == (256, 120)  # config 2: one image per workgroup, 15 rows x 8 pairs
    assert plan(rw, bf16, _shape((64, 56, 56, 256), (256, 3, 3, 256), -1)) == (1792, 112)  # config 3: 7 bands x 2 segments x 2 filter blocks
    assert plan(rw, bf16, _shape((128, 20, 20, 128), (128, 3, 3, 128), -1))[1] >= 100      # config 4's shape in bf16
    assert plan(rw, f32, _shape((256, 15, 15, 128), (128, 3, 3, 128), -1)) == -1
    assert plan(rw, bf16, _shape((256, 15, 15, 128), (64, 3, 3, 128), -1)) == -1           # filters not a multiple of 128
    assert plan(rw, bf16, _shape((256, 15, 15, 96), (128, 3, 3, 96), -1)) == -1            # channels other than 64, 128, 256
    assert plan(rw, bf16, _shape((256, 15, 15, 128), (128, 3, 3, 128), -1, stride=2)) == -1

    st = lib.avhip_conv2d_strided_plan
    assert plan(st, bf16, _shape((64, 56, 56, 128), (256, 3, 3, 128), -1, stride=2)) == (256, 196)  # config 5: 7 x 28 output pixels per tile
    assert plan(st, bf16, _shape((64, 56, 56, 128), (256, 3, 3, 128), -1)) == -1
    assert plan(st, bf16, _shape((64, 56, 56, 128), (128, 3, 3, 128), -1, stride=2)) == -1          # filters not a multiple of 256

    pb = lib.avhip_conv2d_pointwise_block_plan
    assert plan(pb, bf16, _shape((64, 28, 28, 256), (512, 1, 1, 256), 0)) == (256, 196)    # config 5: 50176 pixels in 256 equal blocks
    assert plan(pb, bf16, _shape((8, 28, 28, 256), (1024, 1, 1, 256), 0)) == (242, 52)     # two filter blocks share the chip: 121 pixel blocks of 52
    assert plan(pb, bf16, _shape((64, 28, 28, 64), (512, 1, 1, 64), 0)) == -1
    assert plan(pb, bf16, _shape((64, 28, 28, 256), (512, 3, 3, 256), -1)) == -1
