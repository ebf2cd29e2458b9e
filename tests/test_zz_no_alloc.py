"""The entry point that allocates nothing, avhipConvolutionWinogradFusedForwardNoAlloc, against the entry point it is a
variant of (cudaConvolutionWinogradFusedForward) and against the CPU oracle, through the C API.  Two calls in a row on one
context, the second on a smaller problem, so that what the first call left in the library's fixed scratch array would show."""
import ctypes as C

import numpy as np
import pytest

import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu

TOL = {"f32": 1e-4, "f16": 2e-3, "bf16": 2e-3}  # fused Winograd bars: fp32 1e-4, 16-bit 2e-3 (rel-L2 against the fp64 oracle)


def _fused(c, entry, conv, xt, wt, bt, zt, yt, a1, a2, be, act):
    fn = getattr(c.lib, entry)
    d = xt.dtype
    st = fn(c.ctx.handle, conv.handle, cb.scalar(a1, d), xt.desc, xt.mem, wt.desc, wt.mem, bt.desc, bt.mem, cb.scalar(a2, d), zt.desc, zt.mem,
            cb.scalar(be, d), yt.desc, yt.mem, act)
    assert st == cb.STATUS_SUCCESS, "%s returned %s" % (entry, cb.STATUS_NAMES[st])


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
def test_no_alloc_entry_matches_fused_entry_twice(oracle, dtype):
    g = h.rng(71)
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=h.DT[dtype])
        # first a larger problem, then a smaller one with other weights: the scratch array still holds the first call's matrices
        for (N, H, W, Cin, K) in ((3, 15, 15, 128, 128), (2, 9, 11, 32, 64)):
            x = oracle.round_to(g.standard_normal((N, H, W, Cin)), dtype)
            w = oracle.round_to(g.standard_normal((K, 3, 3, Cin)) * np.sqrt(2.0 / (9 * Cin)), dtype)
            b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
            z = oracle.round_to(g.standard_normal((N, H, W, K)), dtype)
            y0 = oracle.round_to(g.standard_normal((N, H, W, K)), dtype)
            xt, wt, bt, zt = c.tensor(x, dtype), c.tensor(w, dtype), c.tensor(b, "f32"), c.tensor(z, dtype)
            print("no-alloc case", dtype, (N, H, W, Cin, K), flush=True)
            want = oracle.conv2d(x, w, b, z, y0, alpha1=1.1, alpha2=1.2, beta=0.1, activation=oracle.RELU)
            outs = {}
            for entry in ("cudaConvolutionWinogradFusedForward", "avhipConvolutionWinogradFusedForwardNoAlloc"):
                yt = c.tensor(y0, dtype)
                _fused(c, entry, conv, xt, wt, bt, zt, yt, 1.1, 1.2, 0.1, cb.ACTIVATION_RELU)
                c.finish()
                outs[entry] = yt.download()
                assert oracle.rel_l2(outs[entry], want) < TOL[dtype]
            # the same kernels on the same matrices: identical bits
            np.testing.assert_array_equal(outs["avhipConvolutionWinogradFusedForwardNoAlloc"], outs["cudaConvolutionWinogradFusedForward"])


def test_no_alloc_entry_rejects_what_does_not_fit():
    """16 * K * C fp32 matrix elements beyond the fixed array: a status, no launch."""
    with h.Call() as c:
        conv = cb.ConvolutionDescriptor(padding=(-1, -1))
        K = Cin = 512  # 16 * 512 * 512 * 4 = 16 MiB > 4 MiB
        xt, wt = c.empty((1, 8, 8, Cin), "f32"), c.empty((K, 3, 3, Cin), "f32")
        yt = c.empty((1, 8, 8, K), "f32")
        st = c.lib.avhipConvolutionWinogradFusedForwardNoAlloc(c.ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, 0, 0, None, 0, 0, None,
                                                               yt.desc, yt.mem, 0)
        assert st == cb.STATUS_NOT_SUPPORTED
        # the largest that fits: 16 * 256 * 256 * 4 = 4 MiB exactly
        K = Cin = 256
        xt, wt = c.empty((1, 8, 8, Cin), "f32"), c.empty((K, 3, 3, Cin), "f32")
        yt = c.empty((1, 8, 8, K), "f32")
        st = c.lib.avhipConvolutionWinogradFusedForwardNoAlloc(c.ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, 0, 0, None, 0, 0, None,
                                                               yt.desc, yt.mem, 0)
        assert st == cb.STATUS_SUCCESS
        c.finish()
        assert not np.any(yt.download())  # zero weights and inputs
