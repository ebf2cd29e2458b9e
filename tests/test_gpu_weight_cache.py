"""The library's cache of Winograd-transformed weights under the uses that could break it: one weight tensor shared by two
contexts (two streams), weights rewritten between calls on different contexts, weight tensors that are views into an arena that
is also written elsewhere, stream capture with a cold cache, and a captured graph replayed after a weight update.  Results are
checked against the CPU oracle (fp32 fused / non-fused Winograd bar 1e-4, rel-L2).  The ownership contract is that of
include/Avocado/cuda_backend.h:154-165 of the reference (views into an owning block)."""
import ctypes as C

import numpy as np
import pytest

import bench
import cudabackend_amd as cb
import helpers as h

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _state(lib):
    e, b, t = C.c_int64(0), C.c_int64(0), C.c_int64(0)
    cb.check(lib.avhipGetWeightCacheState(C.byref(e), C.byref(b), C.byref(t)), "avhipGetWeightCacheState")
    return e.value, b.value, t.value


def _fused(lib, ctx, conv, x, w, b, y, expect=cb.STATUS_SUCCESS):
    st = lib.cudaConvolutionWinogradFusedForward(ctx.handle, conv.handle, None, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, None, 0, 0, None, y.desc, y.mem,
                                                 cb.ACTIVATION_RELU)
    assert st == expect, cb.STATUS_NAMES[st]


def _problem(oracle, g, N=6, HW=15, Cin=64, K=64):
    x = oracle.round_to(g.standard_normal((N, HW, HW, Cin)), "f32")
    w = oracle.round_to(g.standard_normal((K, 3, 3, Cin)) * np.sqrt(2.0 / (9 * Cin)), "f32")
    b = g.uniform(-0.1, 0.1, K).astype(np.float32).astype(np.float64)
    return x, w, b


def test_two_contexts_share_one_weight_tensor(oracle):
    lib = cb.load_library()
    cb.check(lib.avhipInvalidateCaches(), "avhipInvalidateCaches")
    g = h.rng(91)
    x, w, b = _problem(oracle, g, N=64, Cin=128, K=128)
    want = oracle.conv2d(x, w, b, activation=oracle.RELU)
    conv = cb.ConvolutionDescriptor(padding=(-1, -1))
    c1, c2 = cb.Context(0), cb.Context(0)
    xt, wt, bt = cb.DeviceTensor.from_numpy(x, cb.DTYPE_FLOAT32), cb.DeviceTensor.from_numpy(w, cb.DTYPE_FLOAT32), cb.DeviceTensor.from_numpy(b, cb.DTYPE_FLOAT32)
    y1, y2 = cb.DeviceTensor(want.shape, cb.DTYPE_FLOAT32), cb.DeviceTensor(want.shape, cb.DTYPE_FLOAT32)
    t0 = _state(lib)[2]
    # back to back, no synchronisation in between: the second context must wait for the transform the first one enqueued
    _fused(lib, c1, conv, xt, wt, bt, y1)
    _fused(lib, c2, conv, xt, wt, bt, y2)
    c1.synchronize()
    c2.synchronize()
    assert _state(lib)[2] == t0 + 1, "one weight tensor, one transform"
    assert oracle.rel_l2(y1.download(), want) < TOL
    assert oracle.rel_l2(y2.download(), want) < TOL
    # weights rewritten through the API on the second context, then used by the first: transformed again, into the same buffer
    entries, nbytes, _ = _state(lib)
    w2 = oracle.round_to(g.standard_normal(w.shape) * np.sqrt(2.0 / (9 * w.shape[3])), "f32")
    raw = np.ascontiguousarray(w2, dtype=np.float32)
    cb.check(lib.cudaCopyMemoryFromHost(c2.handle, wt.mem, 0, raw.ctypes.data, raw.nbytes), "cudaCopyMemoryFromHost")
    c2.synchronize()  # the caller's own ordering between the write and other streams that read the weights
    _fused(lib, c1, conv, xt, wt, bt, y1)
    _fused(lib, c2, conv, xt, wt, bt, y2)
    c1.synchronize()
    c2.synchronize()
    want2 = oracle.conv2d(x, w2, b, activation=oracle.RELU)
    assert oracle.rel_l2(y1.download(), want2) < TOL
    assert oracle.rel_l2(y2.download(), want2) < TOL
    assert _state(lib) == (entries, nbytes, t0 + 2), "re-transformed once, in place: no new buffer"
    for t in (xt, wt, bt, y1, y2):
        t.close()
    c1.close()
    c2.close()


def test_weights_in_an_arena_survive_writes_elsewhere_in_it(oracle):
    """Weights, input and output are views into one owning block.  Writing the output view (every call does) or the input view must
    not invalidate the cached matrices of the weight view; writing the weight view must."""
    lib = cb.load_library()
    g = h.rng(92)
    x, w, b = _problem(oracle, g)
    want = oracle.conv2d(x, w, b, activation=oracle.RELU)
    conv = cb.ConvolutionDescriptor(padding=(-1, -1))
    sizes = [a.size * 4 for a in (w, x, want)]
    offs = np.cumsum([0] + [(s + 255) // 256 * 256 for s in sizes])
    arena = C.c_int64(0)
    cb.check(lib.cudaCreateMemoryDescriptor(C.byref(arena), 0, int(offs[-1])), "arena")
    views = []
    for off, size in zip(offs[:-1], sizes):
        v = C.c_int64(0)
        cb.check(lib.cudaCreateMemoryView(C.byref(v), arena.value, size, int(off)), "view")
        views.append(v.value)
    wv, xv, yv = views
    descs = {}
    for name, arr in (("w", w), ("x", x), ("y", want)):
        d = C.c_int64(0)
        cb.check(lib.cudaCreateTensorDescriptor(C.byref(d)), "desc")
        cb.check(lib.cudaSetTensorDescriptor(d.value, cb.DTYPE_FLOAT32, 4, (C.c_int * 4)(*arr.shape)), "set desc")
        descs[name] = d.value
    bt = cb.DeviceTensor.from_numpy(b, cb.DTYPE_FLOAT32)
    with cb.Context(0) as ctx:
        def upload(view, arr):
            raw = np.ascontiguousarray(arr, dtype=np.float32)
            cb.check(lib.cudaCopyMemoryFromHost(ctx.handle, view, 0, raw.ctypes.data, raw.nbytes), "upload")

        def run():
            st = lib.cudaConvolutionWinogradFusedForward(ctx.handle, conv.handle, None, descs["x"], xv, descs["w"], wv, bt.desc, bt.mem, None, 0, 0, None,
                                                         descs["y"], yv, cb.ACTIVATION_RELU)
            assert st == cb.STATUS_SUCCESS, cb.STATUS_NAMES[st]
            ctx.synchronize()
            out = np.empty(want.shape, dtype=np.float32)
            cb.check(lib.cudaCopyMemoryToHost(ctx.handle, out.ctypes.data, yv, 0, out.nbytes), "download")
            ctx.synchronize()
            return out.astype(np.float64)
        upload(wv, w)
        upload(xv, x)
        t0 = _state(lib)[2]
        assert oracle.rel_l2(run(), want) < TOL
        assert _state(lib)[2] == t0 + 1
        for _ in range(3):  # every call writes the output view of the same block
            assert oracle.rel_l2(run(), want) < TOL
        x2 = oracle.round_to(g.standard_normal(x.shape), "f32")
        upload(xv, x2)
        assert oracle.rel_l2(run(), oracle.conv2d(x2, w, b, activation=oracle.RELU)) < TOL
        assert _state(lib)[2] == t0 + 1, "writes to other views of the block left the cached matrices alone"
        w2 = oracle.round_to(w[::-1] * 0.5, "f32")
        upload(wv, w2)
        assert oracle.rel_l2(run(), oracle.conv2d(x2, w2, b, activation=oracle.RELU)) < TOL
        assert _state(lib)[2] == t0 + 2
        # a write through the owning block's handle that covers the weight bytes counts as well
        raw = np.ascontiguousarray(w, dtype=np.float32)
        cb.check(lib.cudaCopyMemoryFromHost(ctx.handle, arena.value, int(offs[0]), raw.ctypes.data, raw.nbytes), "upload through the owner")
        assert oracle.rel_l2(run(), oracle.conv2d(x2, w, b, activation=oracle.RELU)) < TOL
        assert _state(lib)[2] == t0 + 3
        # many more writes of the same few ranges than the write log has slots (what a deep network does to an arena: every layer
        # writes one of two or three activation buffers): a range that is written again renews its slot, the weights stay cached
        for i in range(200):
            upload(xv, x2)
            upload(yv, want)
        assert oracle.rel_l2(run(), oracle.conv2d(x2, w, b, activation=oracle.RELU)) < TOL
        assert _state(lib)[2] == t0 + 3, "repeated writes of the same ranges must not push the weight's history out of the log"
        # more DISTINCT ranges written elsewhere than the log holds: the lookup turns conservative (transforms again), results stay right
        piece = np.ascontiguousarray(x2.reshape(-1)[:4], dtype=np.float32)
        for i in range(70):
            cb.check(lib.cudaCopyMemoryFromHost(ctx.handle, xv, 16 * i, piece.ctypes.data, piece.nbytes), "upload of a piece")
        x3 = x2.copy()
        x3.reshape(-1)[:4 * 70] = np.tile(piece.astype(np.float64), 70)
        assert oracle.rel_l2(run(), oracle.conv2d(x3, w, b, activation=oracle.RELU)) < TOL
        assert _state(lib)[2] == t0 + 4
    for v in views:
        lib.cudaDestroyMemoryDescriptor(v)
    # destroying the block drops its cached matrices
    entries = _state(lib)[0]
    lib.cudaDestroyMemoryDescriptor(arena.value)
    assert _state(lib)[0] == entries - 1
    for d in descs.values():
        lib.cudaDestroyTensorDescriptor(d)
    bt.close()


def test_view_of_a_destroyed_block_is_not_resolved_to_a_recycled_slot():
    lib = cb.load_library()
    a, v, b2 = C.c_int64(0), C.c_int64(0), C.c_int64(0)
    cb.check(lib.cudaCreateMemoryDescriptor(C.byref(a), 0, 4096), "block")
    cb.check(lib.cudaCreateMemoryView(C.byref(v), a.value, 1024, 1024), "view")
    cb.check(lib.cudaDestroyMemoryDescriptor(a.value), "destroy block")
    cb.check(lib.cudaCreateMemoryDescriptor(C.byref(b2), 0, 8192), "block in the recycled slot")
    # a view cannot be made of a view, and the orphaned view must not count as a view of the new block: writing through it
    # (a fill of its own 1 KiB) is harmless to the library's bookkeeping, which is all that can be checked from outside
    w = C.c_int64(0)
    assert lib.cudaCreateMemoryView(C.byref(w), v.value, 16, 0) == cb.STATUS_BAD_PARAM
    lib.cudaDestroyMemoryDescriptor(v.value)
    lib.cudaDestroyMemoryDescriptor(b2.value)


def test_capture_with_a_cold_cache_allocates_nothing(oracle):
    """Under stream capture a Winograd entry with uncached weights reports BAD_ALLOC and launches nothing; the dispatcher falls
    back to implicit GEMM inside the same capture; after one call outside capture both capture and replay the Winograd plan."""
    lib = cb.load_library()
    hip = bench.Hip()
    g = h.rng(93)
    x, w, b = _problem(oracle, g, N=64, Cin=128, K=128)  # large enough for the dispatcher to pick a Winograd plan
    want = oracle.conv2d(x, w, b, activation=oracle.RELU)
    conv = cb.ConvolutionDescriptor(padding=(-1, -1))
    xt, wt, bt = cb.DeviceTensor.from_numpy(x, cb.DTYPE_FLOAT32), cb.DeviceTensor.from_numpy(w, cb.DTYPE_FLOAT32), cb.DeviceTensor.from_numpy(b, cb.DTYPE_FLOAT32)
    y = cb.DeviceTensor(want.shape, cb.DTYPE_FLOAT32)
    need = C.c_int64(0)
    with cb.Context(0) as ctx:
        cb.check(lib.cudaGetConvolutionWorkspaceSize(ctx.handle, conv.handle, xt.desc, wt.desc, bt.desc, C.byref(need)), "workspace size")
        ws = cb.DeviceTensor((max(need.value, 256),), cb.DTYPE_UINT8)

        def dispatch():
            cb.check(lib.cudaConvolutionBiasActivationForward(ctx.handle, conv.handle, None, xt.desc, xt.mem, wt.desc, wt.mem, bt.desc, bt.mem, None, 0, 0,
                                                              None, y.desc, y.mem, cb.ACTIVATION_RELU, ws.mem), "dispatch")
        before = _state(lib)
        exe = hip.capture(ctx.stream(), lambda: (_fused(lib, ctx, conv, xt, wt, bt, y, expect=cb.STATUS_BAD_ALLOC), dispatch()))
        assert _state(lib) == before, "nothing allocated or transformed during capture"
        for _ in range(2):
            cb.check(lib.cudaSetMemory(ctx.handle, y.mem, 0, y.nbytes, None, 0), "clear y")
            hip.launch(exe, ctx.stream())
            ctx.synchronize()
            assert oracle.rel_l2(y.download(), want) < 1e-5  # the implicit-GEMM plan (fp32 bar 1e-5)
        hip.rt.hipGraphExecDestroy(exe)
        # warm the cache outside capture, then capture the Winograd plans themselves
        dispatch()
        _fused(lib, ctx, conv, xt, wt, bt, y)
        ctx.synchronize()
        warm = _state(lib)
        assert warm[2] > before[2]
        exe = hip.capture(ctx.stream(), lambda: (_fused(lib, ctx, conv, xt, wt, bt, y), dispatch()))
        assert _state(lib) == warm
        for _ in range(3):
            cb.check(lib.cudaSetMemory(ctx.handle, y.mem, 0, y.nbytes, None, 0), "clear y")
            hip.launch(exe, ctx.stream())
            ctx.synchronize()
            assert oracle.rel_l2(y.download(), want) < TOL
        # weights rewritten, one eager call (re-transforms in place), and the old graph replays on valid memory with the new matrices
        w2 = oracle.round_to(w * 0.25, "f32")
        wt.upload(w2)
        dispatch()
        _fused(lib, ctx, conv, xt, wt, bt, y)
        ctx.synchronize()
        assert _state(lib)[:2] == warm[:2]
        cb.check(lib.cudaSetMemory(ctx.handle, y.mem, 0, y.nbytes, None, 0), "clear y")
        hip.launch(exe, ctx.stream())
        ctx.synchronize()
        assert oracle.rel_l2(y.download(), oracle.conv2d(x, w2, b, activation=oracle.RELU)) < TOL
        hip.rt.hipGraphExecDestroy(exe)
        ws.close()
    for t in (xt, wt, bt, y):
        t.close()


def test_budget_never_frees_what_a_graph_holds(oracle):
    """With a budget that every insertion exceeds, the cache frees the least recently used matrices, but never those a captured graph
    was handed: the graph replays on valid memory after other weight tensors have gone through the cache."""
    lib = cb.load_library()
    hip = bench.Hip()
    cb.check(lib.avhipInvalidateCaches(), "avhipInvalidateCaches")
    previous = C.c_int64(0)
    cb.check(lib.avhipSetWeightCacheBudget(1, C.byref(previous)), "avhipSetWeightCacheBudget")
    g = h.rng(95)
    x, w, b = _problem(oracle, g)
    want = oracle.conv2d(x, w, b, activation=oracle.RELU)
    conv = cb.ConvolutionDescriptor(padding=(-1, -1))
    xt, wt, bt = cb.DeviceTensor.from_numpy(x, cb.DTYPE_FLOAT32), cb.DeviceTensor.from_numpy(w, cb.DTYPE_FLOAT32), cb.DeviceTensor.from_numpy(b, cb.DTYPE_FLOAT32)
    y = cb.DeviceTensor(want.shape, cb.DTYPE_FLOAT32)
    others = [cb.DeviceTensor.from_numpy(oracle.round_to(g.standard_normal(w.shape) * 0.05, "f32"), cb.DTYPE_FLOAT32) for _ in range(3)]
    y2 = cb.DeviceTensor(want.shape, cb.DTYPE_FLOAT32)
    try:
        with cb.Context(0) as ctx:
            _fused(lib, ctx, conv, xt, wt, bt, y)  # warm: the matrices of w are in the cache
            ctx.synchronize()
            assert _state(lib)[0] == 1
            exe = hip.capture(ctx.stream(), lambda: _fused(lib, ctx, conv, xt, wt, bt, y))
            per_entry = _state(lib)[1]
            for i, other in enumerate(others):  # every insertion is over the budget: the previous `other` goes, the graph's entry stays
                _fused(lib, ctx, conv, xt, other, bt, y2)
                ctx.synchronize()
                assert _state(lib)[:2] == (2, 2 * per_entry), "one pinned entry and the newest one"
            cb.check(lib.cudaSetMemory(ctx.handle, y.mem, 0, y.nbytes, None, 0), "clear y")
            hip.launch(exe, ctx.stream())
            ctx.synchronize()
            assert oracle.rel_l2(y.download(), want) < TOL
            hip.rt.hipGraphExecDestroy(exe)
    finally:
        cb.check(lib.avhipSetWeightCacheBudget(previous.value, None), "avhipSetWeightCacheBudget")
        cb.check(lib.avhipInvalidateCaches(), "avhipInvalidateCaches")
    for t in [xt, wt, bt, y, y2] + others:
        t.close()
