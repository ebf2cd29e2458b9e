"""ctypes binding of the backend's C API, with the same names, argument order and status codes as the C header
(include/avocado_hip_backend.h, which mirrors include/Avocado/cuda_backend.h of the reference), plus small RAII helpers
in the spirit of the TensorWrapper / ContextWrapper of the reference's scratch driver (app/CudaBackend.cu:22-120)."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libavocado_hip.so")

# ---- enumerations (values of include/avocado_backend_defs.h) --------------------------------------------------------
(STATUS_SUCCESS, STATUS_ALLOC_FAILED, STATUS_FREE_FAILED, STATUS_BAD_ALLOC, STATUS_BAD_PARAM, STATUS_ARCH_MISMATCH, STATUS_INTERNAL_ERROR,
 STATUS_NOT_SUPPORTED, STATUS_UNSUPPORTED_DATATYPE, STATUS_EXECUTION_FAILED, STATUS_INSUFFICIENT_DRIVER, STATUS_DEVICE_TYPE_MISMATCH) = range(12)
STATUS_NAMES = ["SUCCESS", "ALLOC_FAILED", "FREE_FAILED", "BAD_ALLOC", "BAD_PARAM", "ARCH_MISMATCH", "INTERNAL_ERROR", "NOT_SUPPORTED",
                "UNSUPPORTED_DATATYPE", "EXECUTION_FAILED", "INSUFFICIENT_DRIVER", "DEVICE_TYPE_MISMATCH"]
(DTYPE_UNKNOWN, DTYPE_UINT8, DTYPE_INT8, DTYPE_INT16, DTYPE_INT32, DTYPE_INT64, DTYPE_FLOAT16, DTYPE_BFLOAT16, DTYPE_FLOAT32, DTYPE_FLOAT64,
 DTYPE_COMPLEX32, DTYPE_COMPLEX64) = range(12)
(ACTIVATION_LINEAR, ACTIVATION_SIGMOID, ACTIVATION_TANH, ACTIVATION_RELU, ACTIVATION_SELU, ACTIVATION_ELU, ACTIVATION_EXPONENTIAL,
 ACTIVATION_SOFTPLUS, ACTIVATION_SOFTSIGN) = range(9)
CONVOLUTION_MODE, CROSS_CORRELATION_MODE = 0, 1
GEMM_OPERATION_N, GEMM_OPERATION_T = 0, 1
(DEVICE_NAME, DEVICE_PROCESSOR_COUNT, DEVICE_MEMORY, DEVICE_SUPPORTS_HALF_PRECISION, DEVICE_SUPPORTS_BFLOAT16, DEVICE_SUPPORTS_SINGLE_PRECISION,
 DEVICE_SUPPORTS_DOUBLE_PRECISION, DEVICE_SUPPORTS_SSE, DEVICE_SUPPORTS_SSE2, DEVICE_SUPPORTS_SSE3, DEVICE_SUPPORTS_SSSE3, DEVICE_SUPPORTS_SSE41,
 DEVICE_SUPPORTS_SSE42, DEVICE_SUPPORTS_AVX, DEVICE_SUPPORTS_AVX2, DEVICE_SUPPORTS_AVX512_F, DEVICE_SUPPORTS_AVX512_VL_BW_DQ, DEVICE_SUPPORTS_DP4A,
 DEVICE_ARCH_MAJOR, DEVICE_ARCH_MINOR, DEVICE_SUPPORTS_TENSOR_CORES) = range(21)

DTYPE_SIZE = {DTYPE_UINT8: 1, DTYPE_INT8: 1, DTYPE_INT16: 2, DTYPE_INT32: 4, DTYPE_INT64: 8, DTYPE_FLOAT16: 2, DTYPE_BFLOAT16: 2, DTYPE_FLOAT32: 4,
              DTYPE_FLOAT64: 8}
# host representation of each device dtype (bf16 travels as uint16 bit patterns)
HOST_DTYPE = {DTYPE_UINT8: np.uint8, DTYPE_INT8: np.int8, DTYPE_INT16: np.int16, DTYPE_INT32: np.int32, DTYPE_INT64: np.int64,
              DTYPE_FLOAT16: np.float16, DTYPE_BFLOAT16: np.uint16, DTYPE_FLOAT32: np.float32, DTYPE_FLOAT64: np.float64}

i64, i32, vp = C.c_int64, C.c_int, C.c_void_p
ip = C.POINTER(C.c_int)

# name -> (restype, argtypes); mirrors include/avocado_hip_backend.h line by line
PROTOTYPES = {
    "cudaGetNumberOfDevices": (i32, []),
    "cudaGetDeviceProperty": (i32, [i32, i32, vp]),
    "cudaIsCopyPossible": (i32, [i32, i32, C.POINTER(C.c_bool)]),
    "cudaCreateContextDescriptor": (i32, [C.POINTER(i64), i32]),
    "cudaDestroyContextDescriptor": (i32, [i64]),
    "cudaGetDefaultContext": (i64, [i32]),
    "cudaSynchronizeWithContext": (i32, [i64]),
    "cudaIsContextReady": (i32, [i64, C.POINTER(C.c_bool)]),
    "cudaCreateMemoryDescriptor": (i32, [C.POINTER(i64), i32, i64]),
    "cudaCreateMemoryView": (i32, [C.POINTER(i64), i64, i64, i64]),
    "cudaDestroyMemoryDescriptor": (i32, [i64]),
    "cudaSetMemory": (i32, [i64, i64, i64, i64, vp, i64]),
    "cudaCopyMemory": (i32, [i64, i64, i64, i64, i64, i64]),
    "cudaCopyMemoryToHost": (i32, [i64, vp, i64, i64, i64]),
    "cudaCopyMemoryFromHost": (i32, [i64, i64, i64, vp, i64]),
    "cudaPageLock": (i32, [vp, i64]),
    "cudaPageUnlock": (i32, [vp]),
    "cudaCreateTensorDescriptor": (i32, [C.POINTER(i64)]),
    "cudaDestroyTensorDescriptor": (i32, [i64]),
    "cudaSetTensorDescriptor": (i32, [i64, i32, i32, ip]),
    "cudaGetTensorDescriptor": (i32, [i64, ip, ip, ip]),
    "cudaCreateConvolutionDescriptor": (i32, [C.POINTER(i64)]),
    "cudaDestroyConvolutionDescriptor": (i32, [i64]),
    "cudaSetConvolutionDescriptor": (i32, [i64, i32, i32, ip, ip, ip, i32, vp]),
    "cudaGetConvolutionDescriptor": (i32, [i64, ip, ip, ip, ip, ip, ip, vp]),
    "cudaChangeType": (i32, [i64, i64, i32, i64, i32, i64]),
    "cudaAffineForward": (i32, [i64, i32, i64, i64, i64, i64, vp, i64, i64, vp, i64, i64]),
    "cudaBatchNormInference": (i32, [i64, i32, vp, i64, i64, vp, i64, i64, i64, i64, i64, i64, i64, C.c_double]),
    "cudaAddBias": (i32, [i64, vp, vp, i64, i64, i64, i64, i64, i64, vp, vp, vp, i64, i32]),
    "cudaGemm": (i32, [i64, i32, i32, vp, i64, i64, i64, i64, vp, i64, i64]),
    "cudaGemmBatched": (i32, [i64, i32, i32, vp, i64, i64, i64, i64, vp, i64, i64]),
    "cudaIm2Row": (i32, [i64, i64, i64, i64, i64, i64, i64]),
    "cudaConvolutionImplicitGemmForward": (i32, [i64, i64, vp, i64, i64, i64, i64, i64, i64, vp, i64, i64, vp, i64, i64, i32]),
    "cudaConvolutionWinogradFusedForward": (i32, [i64, i64, vp, i64, i64, i64, i64, i64, i64, vp, i64, i64, vp, i64, i64, i32]),
    "avhipConvolutionWinogradFusedForwardNoAlloc": (i32, [i64, i64, vp, i64, i64, i64, i64, i64, i64, vp, i64, i64, vp, i64, i64, i32]),
    "cudaWinogradWeightTransform": (i32, [i64, i64, i32, i64, i64, i64, i64]),
    "cudaWinogradInputTransform": (i32, [i64, i64, i32, i64, i64, i64, i64, i64]),
    "cudaWinogradOutputTransform": (i32, [i64, i64, i32, i64, vp, i64, i64, i64, i64, i64, i64, vp, i64, i64, vp, i32]),
    "cudaWinogradGradientTransform": (i32, [i64, i64, i32, i64, i64, i64, i64, i64]),
    "cudaWinogradUpdateTransform": (i32, [i64, i64, i32, vp, i64, i64, vp, i64, i64]),
    "cudaGetConvolutionWorkspaceSize": (i32, [i64, i64, i64, i64, i64, C.POINTER(i64)]),
    "cudaConvolutionBiasActivationForward": (i32, [i64, i64, vp, i64, i64, i64, i64, i64, i64, vp, i64, i64, vp, i64, i64, i32, i64]),
    "cudaConvolutionForward": (i32, [i64, i64, vp, i64, i64, i64, i64, vp, i64, i64, i64]),
    "avhipConvolutionRequantForward": (i32, [i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i32]),
    "avhipGetContextStream": (i32, [i64, C.POINTER(vp)]),
    "avhipGetMemoryPointer": (i32, [i64, C.POINTER(vp)]),
    "avhipInvalidateCaches": (i32, []),
    "avhipGetWeightCacheState": (i32, [C.POINTER(i64), C.POINTER(i64), C.POINTER(i64)]),
    "avhipSetWeightCacheBudget": (i32, [i64, C.POINTER(i64)]),
    "avhipWeightCachePolicyProbe": (i32, [i32, C.POINTER(i64), C.POINTER(i64), C.POINTER(i32), i64, i64, C.POINTER(i32)]),
}
# the thin kernel layer of include/avocado_hip_kernels.h (exported, bound only for the symbol check)
KERNEL_LAYER_SYMBOLS = ["avhip_winograd_weight_transform", "avhip_winograd_input_transform", "avhip_winograd_output_transform",
                        "avhip_winograd_gradient_transform", "avhip_winograd_update_transform", "avhip_gemm_batched",
                        "avhip_conv2d_implicit_gemm", "avhip_conv2d_implicit_gemm_split_k", "avhip_conv2d_split_k_workspace", "avhip_conv2d_winograd_fused", "avhip_add_bias", "avhip_im2row", "avhip_change_type",
                        "avhip_set_memory", "avhip_mfma_rate_probe", "avhip_set_small_problem_threshold", "avhip_set_short_k_engine",
                        "avhip_affine_forward", "avhip_batchnorm_inference", "avhip_stream_probe", "avhip_conv2d_winograd_rows",
                        "avhip_winograd_rows_weight_transform", "avhip_winograd_rows_weight_bytes", "avhip_conv2d_winograd_rows_plan",
                        "avhip_set_winograd_rows", "avhip_conv2d_strided", "avhip_conv2d_strided_weight_layout", "avhip_conv2d_strided_weight_bytes",
                        "avhip_conv2d_strided_plan", "avhip_set_conv_strided", "avhip_conv2d_pointwise_block", "avhip_conv2d_pointwise_block_weight_layout",
                        "avhip_conv2d_pointwise_block_weight_bytes", "avhip_conv2d_pointwise_block_plan", "avhip_set_pointwise_block"]

_lib = None


class BackendError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        name = STATUS_NAMES[status] if 0 <= status < len(STATUS_NAMES) else str(status)
        super().__init__("%s returned AVOCADO_STATUS_%s" % (where, name))


def load_library(path=None):
    """Loads libavocado_hip.so and sets the prototypes.  Raises when the library has not been built: there is no fallback."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    path = path or LIBRARY_PATH
    if not os.path.exists(path):
        raise FileNotFoundError("%s is missing: build it with `python -m cudabackend_amd.build` (hipcc, gfx950)" % path)
    lib = C.CDLL(path)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    for name in KERNEL_LAYER_SYMBOLS:
        getattr(lib, name)
    _lib = lib
    return lib


def check(status, where="call"):
    if status != STATUS_SUCCESS:
        raise BackendError(status, where)


# ---- host-side conversions between numpy arrays and device element types ----------------------------------------------
def _f32_to_bf16_bits(a):
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    out = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    out[np.isnan(np.asarray(a, dtype=np.float32))] = 0x7FC0
    return out


def to_device_repr(a, dtype):
    """numpy values -> the host array whose bytes are the device representation (rounding to nearest even)."""
    if dtype == DTYPE_BFLOAT16:
        return _f32_to_bf16_bits(np.asarray(a, dtype=np.float32))
    if dtype == DTYPE_FLOAT16:
        return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16))
    return np.ascontiguousarray(a, dtype=HOST_DTYPE[dtype])


def from_device_repr(raw, dtype):
    """Inverse of to_device_repr: returns float64 for floating types, the integer array otherwise."""
    if dtype == DTYPE_BFLOAT16:
        return (raw.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    if dtype in (DTYPE_FLOAT16, DTYPE_FLOAT32, DTYPE_FLOAT64):
        return raw.astype(np.float64)
    return raw


def scalar(value, dtype):
    """Host scalar for alpha / beta arguments: fp64 for fp64 tensors, fp32 otherwise; None stays a null pointer."""
    if value is None:
        return None
    return C.byref(C.c_double(value)) if dtype == DTYPE_FLOAT64 else C.byref(C.c_float(value))


# ---- RAII helpers ----------------------------------------------------------------------------------------------------
class Context:
    """A context descriptor; Context(default=True) wraps the default (synchronous) context of the device."""

    def __init__(self, device=0, default=False):
        self.lib = load_library()
        self.device = device
        self.default = default
        if default:
            self.handle = self.lib.cudaGetDefaultContext(device)
            if self.handle == -1:
                raise BackendError(STATUS_BAD_PARAM, "cudaGetDefaultContext")
        else:
            h = i64(0)
            check(self.lib.cudaCreateContextDescriptor(C.byref(h), device), "cudaCreateContextDescriptor")
            self.handle = h.value

    def synchronize(self):
        check(self.lib.cudaSynchronizeWithContext(self.handle), "cudaSynchronizeWithContext")

    def stream(self):
        s = vp()
        check(self.lib.avhipGetContextStream(self.handle, C.byref(s)), "avhipGetContextStream")
        return s.value

    def close(self):
        if not self.default and self.handle:
            self.lib.cudaDestroyContextDescriptor(self.handle)
            self.handle = 0

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


class DeviceTensor:
    """Tensor descriptor + memory descriptor, app/CudaBackend.cu:29-101 of the reference."""

    def __init__(self, shape, dtype, device=0, zero=True):
        self.lib = load_library()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = dtype
        self.device = device
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * DTYPE_SIZE[dtype]
        d = i64(0)
        check(self.lib.cudaCreateTensorDescriptor(C.byref(d)), "cudaCreateTensorDescriptor")
        self.desc = d.value
        dims = (C.c_int * len(self.shape))(*self.shape)
        check(self.lib.cudaSetTensorDescriptor(self.desc, dtype, len(self.shape), dims), "cudaSetTensorDescriptor")
        m = i64(0)
        check(self.lib.cudaCreateMemoryDescriptor(C.byref(m), device, self.nbytes), "cudaCreateMemoryDescriptor")
        self.mem = m.value
        if zero and self.nbytes:
            check(self.lib.cudaSetMemory(self.lib.cudaGetDefaultContext(device), self.mem, 0, self.nbytes, None, 0), "cudaSetMemory")

    @classmethod
    def from_numpy(cls, values, dtype, device=0):
        values = np.asarray(values)
        t = cls(values.shape, dtype, device, zero=False)
        t.upload(values)
        return t

    def upload(self, values):
        raw = to_device_repr(np.asarray(values).reshape(self.shape), self.dtype)
        assert raw.nbytes == self.nbytes
        check(self.lib.cudaCopyMemoryFromHost(self.lib.cudaGetDefaultContext(self.device), self.mem, 0, raw.ctypes.data_as(vp), self.nbytes),
              "cudaCopyMemoryFromHost")

    def download_raw(self):
        raw = np.empty(self.shape, dtype=HOST_DTYPE[self.dtype])
        check(self.lib.cudaCopyMemoryToHost(self.lib.cudaGetDefaultContext(self.device), raw.ctypes.data_as(vp), self.mem, 0, self.nbytes),
              "cudaCopyMemoryToHost")
        return raw

    def download(self):
        """float64 values for floating tensors, the integer array otherwise."""
        return from_device_repr(self.download_raw(), self.dtype)

    def download_slice(self, first, count=1):
        """Entries first .. first + count - 1 along the leading dimension, as download() returns them."""
        assert 0 <= first and first + count <= self.shape[0]
        raw = np.empty((count,) + self.shape[1:], dtype=HOST_DTYPE[self.dtype])
        row = self.nbytes // self.shape[0]
        check(self.lib.cudaCopyMemoryToHost(self.lib.cudaGetDefaultContext(self.device), raw.ctypes.data_as(vp), self.mem, first * row, count * row),
              "cudaCopyMemoryToHost")
        return from_device_repr(raw, self.dtype)

    def pointer(self):
        p = vp()
        check(self.lib.avhipGetMemoryPointer(self.mem, C.byref(p)), "avhipGetMemoryPointer")
        return p.value

    def close(self):
        if self.mem:
            self.lib.cudaDestroyMemoryDescriptor(self.mem)
            self.mem = 0
        if self.desc:
            self.lib.cudaDestroyTensorDescriptor(self.desc)
            self.desc = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ConvolutionDescriptor:
    def __init__(self, mode=CONVOLUTION_MODE, padding=(-1, -1), strides=(1, 1), dilation=(1, 1), groups=1, padding_value=None, dtype=DTYPE_FLOAT32):
        self.lib = load_library()
        h = i64(0)
        check(self.lib.cudaCreateConvolutionDescriptor(C.byref(h)), "cudaCreateConvolutionDescriptor")
        self.handle = h.value
        n = len(padding)
        pv = None
        if padding_value is not None:
            raw = to_device_repr(np.array([padding_value]), dtype).tobytes()
            pv = C.create_string_buffer(raw + b"\0" * (16 - len(raw)), 16)
        check(self.lib.cudaSetConvolutionDescriptor(self.handle, mode, n, (C.c_int * n)(*padding), (C.c_int * n)(*strides), (C.c_int * n)(*dilation),
                                                    groups, pv), "cudaSetConvolutionDescriptor")

    def close(self):
        if self.handle:
            self.lib.cudaDestroyConvolutionDescriptor(self.handle)
            self.handle = 0

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
