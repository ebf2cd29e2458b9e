"""Shared plumbing of the GPU parity tests: seeded inputs rounded to the tensor dtype, and thin callers that push numpy
arrays through the backend's C API (ctypes) and bring the result back.  No compute happens here."""
import ctypes as C

import numpy as np

import cudabackend_amd as cb

DT = {"f16": cb.DTYPE_FLOAT16, "bf16": cb.DTYPE_BFLOAT16, "f32": cb.DTYPE_FLOAT32, "f64": cb.DTYPE_FLOAT64, "i8": cb.DTYPE_INT8,
      "i32": cb.DTYPE_INT32}
SEED = 0xA70CAD0


def short_k_engine_fixture(request):
    """Body of a parametrised autouse fixture: runs a test once per engine of the short-k products (1x1 convolutions, Winograd's
    batched GEMM): B operand resident in registers (the default) and both operands through LDS."""
    lib = cb.load_library()
    lib.avhip_set_short_k_engine.restype = int
    previous = lib.avhip_set_short_k_engine(1 if request.param == "both_through_lds" else 0)
    yield
    lib.avhip_set_short_k_engine(previous)


def rng(offset=0):
    return np.random.default_rng(SEED + offset)


def rounded(orc, a, dtype):
    """Values representable in `dtype` (what the GPU will see), as float64."""
    return orc.round_to(a, dtype)


def null():
    return 0


class Call:
    """Keeps device tensors alive for the duration of one backend call and frees them afterwards."""

    def __init__(self, default_context=False):
        self.lib = cb.load_library()
        self.ctx = cb.Context(0, default=default_context)
        self.keep = []

    def tensor(self, values, dtype):
        if values is None:
            return None
        t = cb.DeviceTensor.from_numpy(values, DT[dtype] if isinstance(dtype, str) else dtype)
        self.keep.append(t)
        return t

    def empty(self, shape, dtype):
        t = cb.DeviceTensor(shape, DT[dtype] if isinstance(dtype, str) else dtype)
        self.keep.append(t)
        return t

    def finish(self):
        self.ctx.synchronize()

    def close(self):
        for t in self.keep:
            t.close()
        self.keep = []
        self.ctx.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _d(t):
    return t.desc if t is not None else 0


def _m(t):
    return t.mem if t is not None else 0


def winograd_weight_transform(w, dtype, m, mode=0, mat_dtype=None, expect=cb.STATUS_SUCCESS):
    mat_dtype = mat_dtype or dtype
    K, r, _, Cin = w.shape
    t = m + r - 1
    with Call() as c:
        conv = cb.ConvolutionDescriptor(mode=mode, padding=(-(r // 2), -(r // 2)))
        wt = c.tensor(w, dtype)
        U = c.empty((t * t, K, Cin), mat_dtype)
        st = c.lib.cudaWinogradWeightTransform(c.ctx.handle, conv.handle, m, wt.desc, wt.mem, U.desc, U.mem)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return U.download() if st == cb.STATUS_SUCCESS else None


def winograd_input_transform(x, wshape, dtype, m, pad, padding_value=None, mat_dtype=None, expect=cb.STATUS_SUCCESS):
    mat_dtype = mat_dtype or dtype
    N, H, W, Cin = x.shape
    r = wshape[1]
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    with Call() as c:
        conv = cb.ConvolutionDescriptor(padding=pad, padding_value=padding_value, dtype=DT[dtype])
        xt = c.tensor(x, dtype)
        wt = c.empty(wshape, dtype)
        V = c.empty((t * t, tiles, Cin), mat_dtype)
        st = c.lib.cudaWinogradInputTransform(c.ctx.handle, conv.handle, m, wt.desc, xt.desc, xt.mem, V.desc, V.mem)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return V.download() if st == cb.STATUS_SUCCESS else None


def winograd_output_transform(M, yshape, wshape, dtype, m, bias=None, z=None, y0=None, alpha1=None, alpha2=None, beta=None, activation=0,
                              mat_dtype=None, expect=cb.STATUS_SUCCESS):
    mat_dtype = mat_dtype or dtype
    bias_dtype = "f64" if dtype == "f64" else "f32"
    with Call() as c:
        conv = cb.ConvolutionDescriptor()
        Mt = c.tensor(M, mat_dtype)
        wt = c.empty(wshape, dtype)
        y = c.tensor(y0, dtype) if y0 is not None else c.empty(yshape, dtype)
        b = c.tensor(bias, bias_dtype)
        zt = c.tensor(z, dtype)
        d = DT[dtype]
        st = c.lib.cudaWinogradOutputTransform(c.ctx.handle, conv.handle, m, wt.desc, cb.scalar(alpha1, d), Mt.desc, Mt.mem, y.desc, y.mem, _d(b), _m(b),
                                               cb.scalar(alpha2, d), _d(zt), _m(zt), cb.scalar(beta, d), activation)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return y.download() if st == cb.STATUS_SUCCESS else None


def winograd_gradient_transform(dy, wshape, dtype, m, mat_dtype=None, expect=cb.STATUS_SUCCESS):
    mat_dtype = mat_dtype or dtype
    N, H, W, K = dy.shape
    r = wshape[1]
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    with Call() as c:
        conv = cb.ConvolutionDescriptor()
        dyt = c.tensor(dy, dtype)
        wt = c.empty(wshape, dtype)
        M = c.empty((t * t, tiles, K), mat_dtype)
        st = c.lib.cudaWinogradGradientTransform(c.ctx.handle, conv.handle, m, wt.desc, dyt.desc, dyt.mem, M.desc, M.mem)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return M.download() if st == cb.STATUS_SUCCESS else None


def winograd_update_transform(M, wshape, dtype, m, dw0=None, alpha=None, beta=None, mat_dtype=None, expect=cb.STATUS_SUCCESS):
    mat_dtype = mat_dtype or dtype
    with Call() as c:
        conv = cb.ConvolutionDescriptor()
        Mt = c.tensor(M, mat_dtype)
        dw = c.tensor(dw0, dtype) if dw0 is not None else c.empty(wshape, dtype)
        d = DT[dtype]
        st = c.lib.cudaWinogradUpdateTransform(c.ctx.handle, conv.handle, m, cb.scalar(alpha, d), Mt.desc, Mt.mem, cb.scalar(beta, d), dw.desc, dw.mem)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return dw.download() if st == cb.STATUS_SUCCESS else None


def gemm(A, B, C0, dtype, opA=False, opB=False, alpha=None, beta=None, c_dtype=None, batched=False, expect=cb.STATUS_SUCCESS):
    c_dtype = c_dtype or dtype
    with Call() as c:
        a = c.tensor(A, dtype)
        b = c.tensor(B, dtype)
        ct = c.tensor(C0, c_dtype)
        fn = c.lib.cudaGemmBatched if batched else c.lib.cudaGemm
        d = DT[c_dtype]
        st = fn(c.ctx.handle, int(opA), int(opB), cb.scalar(alpha, d), a.desc, a.mem, b.desc, b.mem, cb.scalar(beta, d), ct.desc, ct.mem)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return ct.download() if st == cb.STATUS_SUCCESS else None


def conv_forward(entry, x, w, yshape, dtype, y_dtype=None, bias=None, bias_dtype=None, z=None, y0=None, alpha1=None, alpha2=None, beta=None,
                 activation=0, pad=(-1, -1), stride=(1, 1), dilation=(1, 1), mode=0, padding_value=None, groups=1, workspace_bytes=None,
                 expect=cb.STATUS_SUCCESS, scale=None):
    """entry: 'implicit_gemm' | 'winograd_fused' | 'dispatch' | 'requant'."""
    y_dtype = y_dtype or dtype
    bias_dtype = bias_dtype or ("f64" if dtype == "f64" else "f32")
    with Call() as c:
        conv = cb.ConvolutionDescriptor(mode=mode, padding=pad, strides=stride, dilation=dilation, groups=groups, padding_value=padding_value,
                                        dtype=DT[dtype])
        xt = c.tensor(x, dtype)
        wt = c.tensor(w, dtype)
        y = c.tensor(y0, y_dtype) if y0 is not None else c.empty(yshape, y_dtype)
        b = c.tensor(bias, bias_dtype)
        zt = c.tensor(z, y_dtype)
        d = DT[y_dtype]
        a1, a2, be = cb.scalar(alpha1, d), cb.scalar(alpha2, d), cb.scalar(beta, d)
        if entry == "implicit_gemm":
            st = c.lib.cudaConvolutionImplicitGemmForward(c.ctx.handle, conv.handle, a1, xt.desc, xt.mem, wt.desc, wt.mem, _d(b), _m(b), a2, _d(zt), _m(zt),
                                                          be, y.desc, y.mem, activation)
        elif entry == "winograd_fused":
            st = c.lib.cudaConvolutionWinogradFusedForward(c.ctx.handle, conv.handle, a1, xt.desc, xt.mem, wt.desc, wt.mem, _d(b), _m(b), a2, _d(zt),
                                                           _m(zt), be, y.desc, y.mem, activation)
        elif entry == "requant":
            sc = c.tensor(scale, "f32")
            st = c.lib.avhipConvolutionRequantForward(c.ctx.handle, conv.handle, xt.desc, xt.mem, wt.desc, wt.mem, _d(b), _m(b), sc.desc, sc.mem, y.desc,
                                                      y.mem, activation)
        elif entry == "dispatch":
            need = C.c_int64(0)
            cb.check(c.lib.cudaGetConvolutionWorkspaceSize(c.ctx.handle, conv.handle, xt.desc, wt.desc, _d(b), C.byref(need)), "workspace size")
            nbytes = need.value if workspace_bytes is None else workspace_bytes
            ws = c.empty((max(nbytes, 1),), cb.DTYPE_UINT8) if nbytes > 0 else None
            st = c.lib.cudaConvolutionBiasActivationForward(c.ctx.handle, conv.handle, a1, xt.desc, xt.mem, wt.desc, wt.mem, _d(b), _m(b), a2, _d(zt),
                                                            _m(zt), be, y.desc, y.mem, activation, _m(ws))
        else:
            raise ValueError(entry)
        assert st == expect, "%s returned %s" % (entry, cb.STATUS_NAMES[st])
        c.finish()
        return y.download() if st == cb.STATUS_SUCCESS else None


def add_bias(x, b, dtype, z=None, y0=None, alpha1=None, alpha2=None, beta1=None, beta2=None, beta3=None, activation=0, expect=cb.STATUS_SUCCESS):
    bias_dtype = "f64" if dtype == "f64" else "f32"
    with Call() as c:
        xt = c.tensor(x, dtype)
        bt = c.tensor(b, bias_dtype)
        y = c.tensor(y0, dtype) if y0 is not None else c.empty(x.shape, dtype)
        zt = c.tensor(z, dtype)
        d = DT[dtype]
        st = c.lib.cudaAddBias(c.ctx.handle, cb.scalar(alpha1, d), cb.scalar(alpha2, d), xt.desc, xt.mem, bt.desc, bt.mem, y.desc, y.mem,
                               cb.scalar(beta1, d), cb.scalar(beta2, d), cb.scalar(beta3, d), _m(zt), activation)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return y.download() if st == cb.STATUS_SUCCESS else None


def affine_forward(x, w, b, dtype, y0=None, alpha=None, beta=None, activation=0, expect=cb.STATUS_SUCCESS):
    pdt = "f64" if dtype == "f64" else "f32"
    with Call() as c:
        xt, wt, bt = c.tensor(x, dtype), c.tensor(w, pdt), c.tensor(b, pdt)
        y = c.tensor(y0, dtype) if y0 is not None else c.empty(x.shape, dtype)
        d = DT[dtype]
        st = c.lib.cudaAffineForward(c.ctx.handle, activation, wt.desc, wt.mem, bt.desc, bt.mem, cb.scalar(alpha, d), xt.desc, xt.mem, cb.scalar(beta, d),
                                     y.desc, y.mem)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return y.download() if st == cb.STATUS_SUCCESS else None


def batchnorm_inference(x, scale, bias, mean, var, dtype, y0=None, alpha=None, beta=None, epsilon=1e-5, activation=0, expect=cb.STATUS_SUCCESS):
    pdt = "f64" if dtype == "f64" else "f32"
    with Call() as c:
        xt = c.tensor(x, dtype)
        ps = [c.tensor(p, pdt) for p in (scale, bias, mean, var)]
        y = c.tensor(y0, dtype) if y0 is not None else c.empty(x.shape, dtype)
        d = DT[dtype]
        st = c.lib.cudaBatchNormInference(c.ctx.handle, activation, cb.scalar(alpha, d), xt.desc, xt.mem, cb.scalar(beta, d), y.desc, y.mem, ps[0].desc,
                                          ps[0].mem, ps[1].mem, ps[2].mem, ps[3].mem, epsilon)
        assert st == expect, cb.STATUS_NAMES[st]
        c.finish()
        return y.download() if st == cb.STATUS_SUCCESS else None


def winograd_nonfused(x, w, dtype, m, mat_dtype, acc_dtype, bias=None, z=None, activation=0, pad=(-1, -1), mode=0):
    """The four-call non-fused Winograd sequence with the matrices staying on the device, as a front-end runs it
    (src/winograd_nonfused.cu:881,906,932 and src/gemm.cpp:126 of the reference): weight transform, input transform, batched GEMM
    M = V U^T, output transform with the fused epilogue.  mat_dtype: dtype of U and V, acc_dtype: dtype of M."""
    N, H, W, Cin = x.shape
    K, r = w.shape[0], w.shape[1]
    t = m + r - 1
    tiles = N * ((H + m - 1) // m) * ((W + m - 1) // m)
    with Call() as c:
        conv = cb.ConvolutionDescriptor(mode=mode, padding=pad, dtype=DT[dtype])
        xt, wt = c.tensor(x, dtype), c.tensor(w, dtype)
        b, zt = c.tensor(bias, "f32"), c.tensor(z, dtype)
        U, V, M = c.empty((t * t, K, Cin), mat_dtype), c.empty((t * t, tiles, Cin), mat_dtype), c.empty((t * t, tiles, K), acc_dtype)
        y = c.empty((N, H, W, K), dtype)
        hdl = c.ctx.handle
        cb.check(c.lib.cudaWinogradWeightTransform(hdl, conv.handle, m, wt.desc, wt.mem, U.desc, U.mem), "weight transform")
        cb.check(c.lib.cudaWinogradInputTransform(hdl, conv.handle, m, wt.desc, xt.desc, xt.mem, V.desc, V.mem), "input transform")
        cb.check(c.lib.cudaGemmBatched(hdl, 0, 1, None, V.desc, V.mem, U.desc, U.mem, None, M.desc, M.mem), "batched GEMM")
        cb.check(c.lib.cudaWinogradOutputTransform(hdl, conv.handle, m, wt.desc, None, M.desc, M.mem, y.desc, y.mem, _d(b), _m(b), None, _d(zt), _m(zt), None,
                                                   activation), "output transform")
        c.finish()
        return y.download()
