"""ctypes front-end of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and bench.py's cpu_baseline leg may import this module; the product
package never does.  All floating-point checkers take and return float64 numpy arrays; callers round
inputs to the tensor dtype first (see ``round_to``).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")

LINEAR, SIGMOID, TANH, RELU, SELU, ELU, EXPONENTIAL, SOFTPLUS, SOFTSIGN = range(9)
CONVOLUTION, CROSS_CORRELATION = 0, 1


def build(force=False):
    """Compiles liboracle.so and libcpubaseline.so with the Makefile next to this file."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load(name):
    path = os.path.join(_BUILD, name)
    if not os.path.exists(path):
        build()
    return C.CDLL(path)


_lib = None
_base = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load("liboracle.so")
        _lib.orc_activation.restype = C.c_double
        _lib.orc_activation.argtypes = [C.c_int, C.c_double]
    return _lib


def baseline_lib():
    global _base
    if _base is None:
        _base = _load("libcpubaseline.so")
    return _base


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f64(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float64)


# --------------------------------------------------------------------------------------------
# dtype helpers shared by the tests (host-side rounding to the storage type of a tensor)
# --------------------------------------------------------------------------------------------
def f32_to_bf16_bits(a):
    """Round-to-nearest-even fp32 -> bf16, returned as uint16 bit patterns."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = np.isnan(np.asarray(a, dtype=np.float32))
    out = rounded.astype(np.uint16)
    out[nan] = 0x7FC0
    return out


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_to(a, dtype):
    """Rounds a float array to the storage dtype ('f64','f32','f16','bf16') and widens back to fp64."""
    a = np.asarray(a, dtype=np.float64)
    if dtype == "f64":
        return a.copy()
    if dtype == "f32":
        return a.astype(np.float32).astype(np.float64)
    if dtype == "f16":
        return a.astype(np.float32).astype(np.float16).astype(np.float64)
    if dtype == "bf16":
        return bf16_bits_to_f32(f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64)
    raise ValueError(dtype)


def conv_output_shape(H, W, R, S, pad, stride=(1, 1), dilation=(1, 1)):
    """Textbook output size with Avocado's signed offset padding (pad = -p)."""
    ph, pw = -pad[0], -pad[1]
    Ho = (H + 2 * ph - ((R - 1) * dilation[0] + 1)) // stride[0] + 1
    Wo = (W + 2 * pw - ((S - 1) * dilation[1] + 1)) // stride[1] + 1
    return Ho, Wo


# --------------------------------------------------------------------------------------------
# checkers
# --------------------------------------------------------------------------------------------
def conv2d(x, w, bias=None, z=None, y=None, pad=(-1, -1), stride=(1, 1), dilation=(1, 1), groups=1, mode=CONVOLUTION,
           padding_value=0.0, alpha1=1.0, alpha2=1.0, beta=0.0, activation=LINEAR, out_shape=None):
    x, w, bias, z = _f64(x), _f64(w), _f64(bias), _f64(z)
    N, H, W, Cin = x.shape
    K, R, S, _ = w.shape
    Ho, Wo = out_shape if out_shape is not None else conv_output_shape(H, W, R, S, pad, stride, dilation)
    if y is None:
        y = np.zeros((N, Ho, Wo, K), dtype=np.float64)
    else:
        y = np.array(y, dtype=np.float64).reshape(N, Ho, Wo, K)
    lib().orc_conv2d_f64(_p(x), _p(w), _p(bias), _p(z), _p(y), N, H, W, Cin, K, R, S, Ho, Wo, pad[0], pad[1], stride[0], stride[1],
                         dilation[0], dilation[1], groups, mode, C.c_double(padding_value), C.c_double(alpha1), C.c_double(alpha2),
                         C.c_double(beta), activation)
    return y


def conv2d_i8(x, w, bias=None, pad=(-1, -1), stride=(1, 1), dilation=(1, 1), mode=CONVOLUTION, padding_value=0, activation=LINEAR):
    x = np.ascontiguousarray(x, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    N, H, W, Cin = x.shape
    K, R, S, _ = w.shape
    Ho, Wo = conv_output_shape(H, W, R, S, pad, stride, dilation)
    y = np.zeros((N, Ho, Wo, K), dtype=np.int32)
    lib().orc_conv2d_i8(_p(x), _p(w), _p(bias), _p(y), N, H, W, Cin, K, R, S, Ho, Wo, pad[0], pad[1], stride[0], stride[1], dilation[0],
                        dilation[1], mode, int(padding_value), activation)
    return y


def requant_i8(acc, scale):
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    scale = np.ascontiguousarray(scale, dtype=np.float32)
    K = acc.shape[-1]
    q = np.zeros(acc.shape, dtype=np.int8)
    lib().orc_requant_i8(_p(acc), _p(scale), _p(q), C.c_int64(acc.size // K), K)
    return q


_OUT_KIND = {np.dtype(np.int32): 0, np.dtype(np.int8): 1, np.dtype(np.float32): 2}


def conv2d_i8_float_epilogue(acc, bias, z, y, alpha1, alpha2, beta, activation):
    """acc: raw int32 sums; y (int32 / int8 / fp32 array) is updated in place and returned."""
    acc = np.ascontiguousarray(acc, dtype=np.int32)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    kind = _OUT_KIND[y.dtype]
    z = None if z is None else np.ascontiguousarray(z, dtype=y.dtype)
    y = np.ascontiguousarray(y)
    K = acc.shape[-1]
    lib().orc_conv2d_i8_float_epilogue(_p(acc), _p(bias), _p(z), _p(y), C.c_int64(acc.size // K), K, C.c_float(alpha1), C.c_float(alpha2),
                                       C.c_float(beta), activation, kind)
    return y


def winograd_table(m, r, which):
    t = m + r - 1
    shape = {0: (t, r), 1: (t, t), 2: (m, t), 3: (t, m), 4: (r, t)}[which]
    out = np.zeros(shape, dtype=np.float64)
    n = lib().orc_winograd_table(m, r, which, _p(out))
    if n != out.size:
        raise ValueError("unsupported (m, r) = (%d, %d)" % (m, r))
    return out


def winograd_weight_transform(w, m, invert=False):
    w = _f64(w)
    K, r, _, Cin = w.shape
    t = m + r - 1
    U = np.zeros((t * t, K, Cin), dtype=np.float64)
    if lib().orc_winograd_weight_transform(_p(w), _p(U), K, Cin, m, r, int(bool(invert))) != 0:
        raise ValueError("unsupported transform")
    return U


def winograd_input_transform(x, m, r, pad=(-1, -1), padding_value=0.0):
    x = _f64(x)
    N, H, W, Cin = x.shape
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    V = np.zeros((t * t, tiles, Cin), dtype=np.float64)
    if lib().orc_winograd_input_transform(_p(x), _p(V), N, H, W, Cin, m, r, pad[0], pad[1], C.c_double(padding_value)) != 0:
        raise ValueError("unsupported transform")
    return V


def winograd_output_transform(M, shape, m, r, bias=None, z=None, y=None, alpha1=1.0, alpha2=1.0, beta=0.0, activation=LINEAR):
    M, bias, z = _f64(M), _f64(bias), _f64(z)
    N, H, W, K = shape
    y = np.zeros(shape, dtype=np.float64) if y is None else np.array(y, dtype=np.float64).reshape(shape)
    if lib().orc_winograd_output_transform(_p(M), _p(y), _p(bias), _p(z), N, H, W, K, m, r, C.c_double(alpha1), C.c_double(alpha2),
                                           C.c_double(beta), activation) != 0:
        raise ValueError("unsupported transform")
    return y


def winograd_gradient_transform(dy, m, r):
    dy = _f64(dy)
    N, H, W, K = dy.shape
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    M = np.zeros((t * t, tiles, K), dtype=np.float64)
    if lib().orc_winograd_gradient_transform(_p(dy), _p(M), N, H, W, K, m, r) != 0:
        raise ValueError("unsupported transform")
    return M


def winograd_update_transform(M, m, r, dw=None, alpha=1.0, beta=0.0):
    M = _f64(M)
    t = m + r - 1
    assert M.shape[0] == t * t
    _, K, Cin = M.shape
    dw = np.zeros((K, r, r, Cin), dtype=np.float64) if dw is None else np.array(dw, dtype=np.float64).reshape(K, r, r, Cin)
    if lib().orc_winograd_update_transform(_p(M), _p(dw), K, Cin, m, r, C.c_double(alpha), C.c_double(beta)) != 0:
        raise ValueError("unsupported transform")
    return dw


def gemm_batched(A, B, Cm=None, opA=False, opB=False, alpha=1.0, beta=0.0):
    A, B = _f64(A), _f64(B)
    if A.ndim == 2:
        A, B = A[None], B[None]
        squeeze = True
    else:
        squeeze = False
    batch = A.shape[0]
    M, K = (A.shape[2], A.shape[1]) if opA else (A.shape[1], A.shape[2])
    N = B.shape[1] if opB else B.shape[2]
    out = np.zeros((batch, M, N), dtype=np.float64) if Cm is None else np.array(Cm, dtype=np.float64).reshape(batch, M, N)
    lib().orc_gemm_batched(_p(A), _p(B), _p(out), batch, M, N, K, int(opA), int(opB), C.c_double(alpha), C.c_double(beta))
    return out[0] if squeeze else out


def add_bias(x, b, z=None, y=None, alpha1=1.0, alpha2=1.0, beta1=0.0, beta2=0.0, beta3=0.0, activation=LINEAR):
    x, b, z = _f64(x), _f64(b), _f64(z)
    last = x.shape[-1]
    out = np.zeros(x.shape, dtype=np.float64) if y is None else np.array(y, dtype=np.float64).reshape(x.shape)
    lib().orc_add_bias(_p(x), _p(b), _p(z), _p(out), C.c_int64(x.size // last), last, C.c_double(alpha1), C.c_double(alpha2),
                       C.c_double(beta1), C.c_double(beta2), C.c_double(beta3), activation)
    return out


def affine_forward(x, weight, bias, y=None, alpha=1.0, beta=0.0, activation=LINEAR):
    """y = alpha * act(x * weight + bias) + beta * y, weight and bias spanning the trailing dimensions of x."""
    x, weight, bias = _f64(x), _f64(weight), _f64(bias)
    last = weight.size
    out = np.zeros(x.shape, dtype=np.float64) if y is None else np.array(y, dtype=np.float64).reshape(x.shape)
    lib().orc_affine_forward(_p(x), _p(weight), _p(bias), _p(out), C.c_int64(x.size // last), C.c_int64(last), C.c_double(alpha), C.c_double(beta),
                             activation)
    return out


def batchnorm_inference(x, scale, bias, mean, variance, y=None, alpha=1.0, beta=0.0, epsilon=1e-5, activation=LINEAR):
    x, scale, bias, mean, variance = _f64(x), _f64(scale), _f64(bias), _f64(mean), _f64(variance)
    last = scale.size
    out = np.zeros(x.shape, dtype=np.float64) if y is None else np.array(y, dtype=np.float64).reshape(x.shape)
    lib().orc_batchnorm_inference(_p(x), _p(scale), _p(bias), _p(mean), _p(variance), _p(out), C.c_int64(x.size // last), C.c_int64(last),
                                  C.c_double(alpha), C.c_double(beta), C.c_double(epsilon), activation)
    return out


def im2row(x, R, S, pad, mode=CONVOLUTION, padding_value=0.0, stride=(1, 1), dilation=(1, 1)):
    x = _f64(x)
    N, H, W, Cin = x.shape
    Ho, Wo = conv_output_shape(H, W, R, S, pad, stride, dilation)
    rows = np.zeros((N * Ho * Wo, R * S * Cin), dtype=np.float64)
    lib().orc_im2row(_p(x), _p(rows), N, H, W, Cin, R, S, Ho, Wo, pad[0], pad[1], stride[0], stride[1], dilation[0], dilation[1], mode,
                     C.c_double(padding_value))
    return rows


def activation(act, v):
    return np.vectorize(lambda t: lib().orc_activation(act, float(t)))(np.asarray(v, dtype=np.float64))


def rel_l2(got, want):
    got = np.asarray(got, dtype=np.float64).ravel()
    want = np.asarray(want, dtype=np.float64).ravel()
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (den if den > 0 else 1.0))


# --------------------------------------------------------------------------------------------
# timed CPU baseline (bench.py only)
# --------------------------------------------------------------------------------------------
def baseline_conv2d_f32(x, w, bias, pad=(-1, -1), stride=(1, 1), relu=True):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    N, H, W, Cin = x.shape
    K, R, S, _ = w.shape
    Ho, Wo = conv_output_shape(H, W, R, S, pad, stride)
    y = np.empty((N, Ho, Wo, K), dtype=np.float32)
    rc = baseline_lib().orc_conv2d_f32_omp(_p(x), _p(w), _p(bias), _p(y), N, H, W, Cin, K, R, S, Ho, Wo, pad[0], pad[1], stride[0], stride[1],
                                           int(bool(relu)))
    if rc != 0:
        raise MemoryError("cpu baseline scratch allocation failed")
    return y


def baseline_conv2d_i8(x, w, bias, pad=(-1, -1), stride=(1, 1)):
    x = np.ascontiguousarray(x, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.int32)
    N, H, W, Cin = x.shape
    K, R, S, _ = w.shape
    Ho, Wo = conv_output_shape(H, W, R, S, pad, stride)
    y = np.empty((N, Ho, Wo, K), dtype=np.int32)
    rc = baseline_lib().orc_conv2d_i8_omp(_p(x), _p(w), _p(bias), _p(y), N, H, W, Cin, K, R, S, Ho, Wo, pad[0], pad[1], stride[0], stride[1])
    if rc != 0:
        raise MemoryError("cpu baseline scratch allocation failed")
    return y


def baseline_threads():
    return int(baseline_lib().orc_num_threads())
