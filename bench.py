#!/usr/bin/env python3
"""Benchmark of the convolution hot path on one MI355X.

Workload (BASELINE config 2): residual tower, NHWC, N=256, 15x15, 128 channels: stem 3x3 conv 4->128, then 10 blocks of
[3x3 conv + bias + ReLU, 3x3 conv + bias + residual + ReLU] = 21 convolutions per step, every one a call of
cudaConvolutionBiasActivationForward.  Synthetic seeded data: inputs are 4 planes of Bernoulli(0.15) ones, weights He-normal,
biases U(-0.1, 0.1).  All tensors are resident in HBM before the timed region; the timed region is bracketed by HIP events on
the context's stream and by device synchronisation.

Prints ONE JSON line.  `value` is direct-convolution-equivalent TFLOP/s (2*N*Ho*Wo*K*C*R*S per convolution) of the whole tower
in the headline dtype (bf16).  `roofline` is for the dominant kernel (the 128->128 body convolution), its duration measured
with HIP events over the timed region ((pass - stem) / 20); `ms_per_step` is the median of five timings of `--steps` passes each.  `cpu_baseline` is the restated CPU direct convolution
(oracle/cpu_baseline.c, "port") timed on the host cores on a batch slice of the same body convolution.  `detail` carries the
other dtypes and the per-stage figures of the non-fused Winograd path.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import cudabackend_amd as cb  # noqa: E402

PEAK = {"hbm_GBs": 8000.0, "bf16": 2500.0, "f16": 2500.0, "i8": 5000.0, "f32": 157.3}
DT = {"bf16": cb.DTYPE_BFLOAT16, "f16": cb.DTYPE_FLOAT16, "f32": cb.DTYPE_FLOAT32, "i8": cb.DTYPE_INT8}
SEED = 0xA70CAD0
# HBM bytes per launch of the body convolution kernel (read + written, average over the residual and non-residual launches of a
# pass), from the FETCH_SIZE / WRITE_SIZE counter runs summarised in profiles/winograd_rows_bf16_cfg2_hbm_traffic.md.  Counters
# cannot be read from inside this process, so the figure is a CONSTANT carried here, not a measurement of this run; it is only
# reported for the dtype it was taken on.
COUNTED_TRAFFIC_BYTES = {"bf16": 40.22e6}
LONG_CALL_REPLAYS = 4  # graph replays per timing for side-leg calls of 50 us and more (time_calls)


class Hip:
    """The few HIP runtime calls the harness needs itself: events on a given stream."""

    def __init__(self):
        # symbols are looked up through the backend library, i.e. in the HIP runtime IT is linked against: a process may hold a
        # second copy of the runtime (PyTorch ships its own), and a stream of one copy means nothing to the other
        self.rt = cb.load_library()
        for name in ("hipEventCreate", "hipEventRecord", "hipEventSynchronize", "hipEventElapsedTime", "hipEventDestroy", "hipStreamBeginCapture",
                     "hipStreamEndCapture", "hipGraphInstantiate", "hipGraphLaunch", "hipGraphExecDestroy", "hipGraphDestroy", "hipDeviceSynchronize",
                     "hipStreamWaitEvent"):
            getattr(self.rt, name).restype = C.c_int
        self.rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipEventSynchronize.argtypes = [C.c_void_p]
        self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.rt.hipEventDestroy.argtypes = [C.c_void_p]
        self.rt.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        self.rt.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        self.rt.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        self.rt.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipGraphExecDestroy.argtypes = [C.c_void_p]
        self.rt.hipGraphDestroy.argtypes = [C.c_void_p]
        self.rt.hipStreamSynchronize.argtypes = [C.c_void_p]

    def event(self):
        e = C.c_void_p()
        assert self.rt.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.rt.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, a, b):
        assert self.rt.hipEventSynchronize(b) == 0
        ms = C.c_float(0)
        assert self.rt.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)

    def sync(self):
        assert self.rt.hipDeviceSynchronize() == 0

    def capture(self, stream, enqueue):
        """Records what `enqueue()` launches on `stream` into a HIP graph and returns the executable graph.  The library
        launches plain kernels only (no memset nodes, no allocation once its weight cache is warm), so a step of the tower
        is a chain of 21 kernel nodes that replays without any host work between the kernels."""
        rc = self.rt.hipStreamBeginCapture(stream, 0)  # hipStreamCaptureModeGlobal
        assert rc == 0, "hipStreamBeginCapture: error %d" % rc
        enqueue()
        graph = C.c_void_p()
        rc = self.rt.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0, "hipStreamEndCapture: error %d" % rc
        exe = C.c_void_p()
        rc = self.rt.hipGraphInstantiate(C.byref(exe), graph, None, None, 0)
        assert rc == 0, "hipGraphInstantiate: error %d" % rc
        self.rt.hipGraphDestroy(graph)
        return exe

    def launch(self, exe, stream):
        assert self.rt.hipGraphLaunch(exe, stream) == 0

    def time_graph(self, exe, stream, replays, warmup=2):
        for _ in range(warmup):
            self.launch(exe, stream)
        assert self.rt.hipStreamSynchronize(stream) == 0  # the timed replays start on an idle stream
        e0, e1 = self.event(), self.event()
        self.record(e0, stream)
        for _ in range(replays):
            self.launch(exe, stream)
        self.record(e1, stream)
        ms = self.elapsed_ms(e0, e1)
        self.rt.hipEventDestroy(e0)
        self.rt.hipEventDestroy(e1)
        return ms / replays

    def time_graph_groups(self, exe, stream, replays, warmup=2, groups=5):
        """`groups` timings of `replays` replays each, every one between its own pair of events on an idle stream.  Returns the
        per-replay durations of the groups, sorted: one group of 20 passes is 7-9 ms and the clocks of a box drift by several
        per cent over such spans, so a single sample would carry that drift straight into the reported figure."""
        return sorted(self.time_graph(exe, stream, replays, warmup if g == 0 else 1) for g in range(groups))


def conv_flops(N, Ho, Wo, K, Cin, R, S):
    return 2.0 * N * Ho * Wo * K * Cin * R * S


class Tower:
    """Config 2.  Holds every tensor on the device; step() enqueues the 21 convolutions of one forward pass."""

    def __init__(self, ctx, dtype, N=256, HW=15, ch=128, blocks=10, planes=4):
        self.ctx, self.lib, self.dtype = ctx, cb.load_library(), dtype
        self.N, self.HW, self.ch, self.blocks, self.planes = N, HW, ch, blocks, planes
        g = np.random.default_rng(SEED + 2)
        d = DT[dtype]
        x0 = (g.random((N, HW, HW, planes)) < 0.15).astype(np.float32)
        self.x0 = cb.DeviceTensor.from_numpy(x0, d)
        self.conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=d)
        self.layers = []
        self.host_layers = []  # the same weights and biases on the host, for the self-check
        cin = planes
        for _ in range(1 + 2 * blocks):
            w = g.standard_normal((ch, 3, 3, cin)).astype(np.float32) * np.float32(np.sqrt(2.0 / (9 * cin)))
            b = g.uniform(-0.1, 0.1, ch).astype(np.float32)
            self.layers.append((cb.DeviceTensor.from_numpy(w, d), cb.DeviceTensor.from_numpy(b, cb.DTYPE_FLOAT32)))
            self.host_layers.append((w, b))
            cin = ch
        self.act = [cb.DeviceTensor((N, HW, HW, ch), d) for _ in range(3)]
        need = C.c_int64(0)
        cb.check(self.lib.cudaGetConvolutionWorkspaceSize(ctx.handle, self.conv.handle, self.act[0].desc, self.layers[1][0].desc, self.layers[1][1].desc,
                                                          C.byref(need)), "cudaGetConvolutionWorkspaceSize")
        self.workspace = cb.DeviceTensor((max(int(need.value), 256),), cb.DTYPE_UINT8)
        self.workspace_bytes = int(need.value)
        self.flops_body = conv_flops(N, HW, HW, ch, ch, 3, 3)
        self.flops_step = conv_flops(N, HW, HW, ch, planes, 3, 3) + 2 * blocks * self.flops_body

    def _conv(self, x, layer, z, y):
        w, b = self.layers[layer]
        st = self.lib.cudaConvolutionBiasActivationForward(self.ctx.handle, self.conv.handle, None, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, None,
                                                           z.desc if z is not None else 0, z.mem if z is not None else 0, None, y.desc, y.mem,
                                                           cb.ACTIVATION_RELU, self.workspace.mem)
        cb.check(st, "cudaConvolutionBiasActivationForward")

    def stem(self):
        self._conv(self.x0, 0, None, self.act[0])

    def step(self, after=None):
        """One forward pass: stem, then per block [conv -> t, conv + residual -> b] with the three activation buffers rotating.
        after(layer, x, z, y), when given, is called behind each enqueued convolution with its input, residual and output tensors."""
        after = after or (lambda *args: None)
        a, t, b = self.act
        self._conv(self.x0, 0, None, a)
        after(0, self.x0, None, a)
        layer = 1
        for _ in range(self.blocks):
            self._conv(a, layer, None, t)
            after(layer, a, None, t)
            self._conv(t, layer + 1, a, b)
            after(layer + 1, t, a, b)
            layer += 2
            a, b = b, a
        return a

    def set_weights(self, layer, w):
        """Rewrites the weights of one layer through the API (the library tracks the write and re-transforms what it cached)."""
        self.layers[layer][0].upload(w)
        self.host_layers[layer] = (np.asarray(w, dtype=np.float32), self.host_layers[layer][1])

    def close(self):
        for t in [self.x0, self.workspace] + self.act + [t for pair in self.layers for t in pair]:
            t.close()


def time_tower(hip, ctx, dtype, steps, warmup, check=True):
    """Times `steps` forward passes of the tower.  One pass is captured into a HIP graph and replayed, so the timed region
    holds 21 * steps kernels back to back on the context's stream, bracketed by HIP events on that stream.  The duration of
    the dominant kernel (the 20 identical 128->128 body convolutions of a pass) is (pass - stem) / 20 with the stem
    convolution timed the same way; the rocprofv3 kernel trace of this command gives the same figure per launch."""
    tower = Tower(ctx, dtype)
    stream = ctx.stream()
    for _ in range(max(1, warmup)):
        tower.step()  # also fills the library's transformed-weight cache, so that nothing allocates during capture
    ctx.synchronize()
    final = []
    full = hip.capture(stream, lambda: final.append(tower.step()))
    stem = hip.capture(stream, lambda: [tower.stem() for _ in range(10)])
    hip.sync()
    groups = hip.time_graph_groups(full, stream, steps, warmup)  # five timings of exactly `steps` passes each
    ms_step = groups[len(groups) // 2]
    ctx.synchronize()
    checked = self_check(tower, final[0]) if check else {"checked": False}  # what the timed replays left behind, against the CPU oracle
    t0 = time.perf_counter()
    for _ in range(steps):
        tower.step()  # the same pass as 21 eager calls: launch and host cost of the API included
    ctx.synchronize()
    ms_eager = (time.perf_counter() - t0) * 1e3 / steps
    # host time of one call (descriptor checks, dispatch, launch) on an idle stream: a loop that only enqueues soon runs into the
    # back-pressure of the queue and then measures the kernels, not the host
    host = []

    def one_call_at_a_time(layer, x, z, y):
        host.append(time.perf_counter())
        ctx.synchronize()
        host.append(time.perf_counter())
    host.append(time.perf_counter())
    tower.step(after=one_call_at_a_time)
    calls = 1 + 2 * tower.blocks
    host_us_per_call = sorted((host[2 * i + 1] - host[2 * i]) * 1e6 for i in range(calls))[calls // 2]
    ctx.synchronize()
    ms_stem = hip.time_graph_groups(stem, stream, max(steps, 10), warmup, groups=3)[1] / 10
    ctx.synchronize()
    body_us = (ms_step - ms_stem) * 1e3 / (2 * tower.blocks)
    out = {"ms_per_step": ms_step, "ms_per_step_groups": {"timings": len(groups), "passes_each": steps, "min": groups[0], "max": groups[-1]},
           "tflops": tower.flops_step / (ms_step * 1e-3) / 1e12, "stem_conv_us": ms_stem * 1e3,
           "body_conv_us": body_us, "body_conv_tflops": tower.flops_body / (body_us * 1e-6) / 1e12, "workspace_bytes": tower.workspace_bytes,
           "ms_per_step_eager_calls": ms_eager, "host_us_per_call": host_us_per_call, "self_check": checked}
    hip.rt.hipGraphExecDestroy(full)
    hip.rt.hipGraphExecDestroy(stem)
    tower.close()
    return out


def two_half_batch_chains(hip, dtype, steps):
    """NOT the headline: what a caller gains by driving the same 256 images as two independent towers of 128 on two contexts
    (two streams).  In one chain every convolution is one round of lock-stepped workgroups, so nothing overlaps the first
    loads, the epilogue and the gap between dependent launches of a kernel; two chains fill those with each other's MFMAs.
    Timed from an event on the first stream to an event the first stream records after waiting for the second."""
    hip.rt.hipStreamWaitEvent.argtypes = [C.c_void_p, C.c_void_p, C.c_uint]
    ctxs = [cb.Context(0), cb.Context(0)]
    towers, graphs = [], []
    for c in ctxs:
        t = Tower(c, dtype, N=128)
        t.step()
        c.synchronize()
        towers.append(t)
        graphs.append(hip.capture(c.stream(), t.step))
    s0, s1 = ctxs[0].stream(), ctxs[1].stream()

    def run(passes):
        for _ in range(passes):
            hip.launch(graphs[0], s0)
            hip.launch(graphs[1], s1)
    run(3)
    for c in ctxs:
        c.synchronize()
    e0, e1, joined = hip.event(), hip.event(), hip.event()
    hip.record(e0, s0)
    assert hip.rt.hipStreamWaitEvent(s1, e0, 0) == 0  # the second chain starts no earlier than the clock
    run(steps)
    hip.record(joined, s1)
    assert hip.rt.hipStreamWaitEvent(s0, joined, 0) == 0
    hip.record(e1, s0)
    ms = hip.elapsed_ms(e0, e1) / steps
    flops = 2 * towers[0].flops_step
    for g in graphs:
        hip.rt.hipGraphExecDestroy(g)
    for t in towers:
        t.close()
    for c in ctxs:
        c.close()
    return {"ms_per_pass_of_256_images": ms, "tflops": flops / (ms * 1e-3) / 1e12}


def time_calls(hip, ctx, fn, iters, warmup=3):
    """Duration of one call of fn: ten calls are captured into a graph, the graph is replayed; median of three timings."""
    stream = ctx.stream()
    for _ in range(warmup):
        fn()
    ctx.synchronize()
    exe = hip.capture(stream, lambda: [fn() for _ in range(10)])
    # the median of three timings: single layers of 10-20 us scatter by 10 % from one timing to the next (clocks), and the
    # ratios the detail reports (int8 over bf16) are quotients of two of them
    replays = max(2, iters // 2)
    if hip.time_graph(exe, stream, 1, warmup=1) > 0.5:
        # calls of 50 us and more: four replays of the ten calls (40 calls per timing) are plenty.  The cap is also what keeps
        # this script runnable under rocprofv3's kernel trace, which ended in a segmentation fault inside hipGraphLaunch, in the
        # tracer's own frames, with ten replays of the 0.1-0.25 ms stages of config 3 queued at once; untraced runs never failed.
        replays = min(replays, LONG_CALL_REPLAYS)
    ms = sorted(hip.time_graph(exe, stream, replays) / 10 for _ in range(3))[1]
    ctx.synchronize()
    hip.rt.hipGraphExecDestroy(exe)
    return ms


def int8_leg(hip, ctx, iters, shape=(128, 20, 20, 128), filters=((3, -1), (1, 0))):
    """Config 4: N=128, 20x20, 128->128, 3x3 offset -1 and 1x1: int8 x int8 -> int32 (bit-exact path), int8 -> int8
    requantised by a per-filter fp32 scale, and the same shapes in bf16 for the throughput ratio on equal work: through the same
    entry point (cudaConvolutionImplicitGemmForward: the direct kernels for both types) and, as `bf16_dispatcher`, through
    cudaConvolutionBiasActivationForward, which may pick a Winograd plan that int8 cannot have."""
    lib = cb.load_library()
    g = np.random.default_rng(SEED + 4)
    out = {}
    ch = shape[3]
    x = cb.DeviceTensor.from_numpy(g.integers(-127, 128, shape, dtype=np.int8), cb.DTYPE_INT8)
    b = cb.DeviceTensor.from_numpy(g.integers(-2 ** 15, 2 ** 15, ch).astype(np.int32), cb.DTYPE_INT32)
    scale = cb.DeviceTensor.from_numpy(g.uniform(1e-4, 1e-3, ch).astype(np.float32), cb.DTYPE_FLOAT32)
    y = cb.DeviceTensor(shape, cb.DTYPE_INT32)
    q = cb.DeviceTensor(shape, cb.DTYPE_INT8)
    xb = cb.DeviceTensor.from_numpy(g.standard_normal(shape).astype(np.float32), cb.DTYPE_BFLOAT16)
    bb = cb.DeviceTensor.from_numpy(g.uniform(-0.1, 0.1, ch).astype(np.float32), cb.DTYPE_FLOAT32)
    yb = cb.DeviceTensor(shape, cb.DTYPE_BFLOAT16)
    for r, pad in filters:
        w = cb.DeviceTensor.from_numpy(g.integers(-127, 128, (ch, r, r, ch), dtype=np.int8), cb.DTYPE_INT8)
        wb = cb.DeviceTensor.from_numpy((g.standard_normal((ch, r, r, ch)) * np.sqrt(2.0 / (r * r * ch))).astype(np.float32), cb.DTYPE_BFLOAT16)
        conv = cb.ConvolutionDescriptor(padding=(pad, pad), dtype=cb.DTYPE_INT8)
        convb = cb.ConvolutionDescriptor(padding=(pad, pad), dtype=cb.DTYPE_BFLOAT16)

        def exact():
            cb.check(lib.cudaConvolutionImplicitGemmForward(ctx.handle, conv.handle, None, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, None, 0, 0, None,
                                                            y.desc, y.mem, cb.ACTIVATION_LINEAR), "int8 conv")

        def requant():
            cb.check(lib.avhipConvolutionRequantForward(ctx.handle, conv.handle, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, scale.desc, scale.mem,
                                                        q.desc, q.mem, cb.ACTIVATION_RELU), "int8 requant conv")

        def bf16():
            cb.check(lib.cudaConvolutionImplicitGemmForward(ctx.handle, convb.handle, None, xb.desc, xb.mem, wb.desc, wb.mem, bb.desc, bb.mem, None, 0, 0,
                                                            None, yb.desc, yb.mem, cb.ACTIVATION_RELU), "bf16 conv")

        def bf16_dispatcher():
            cb.check(lib.cudaConvolutionBiasActivationForward(ctx.handle, convb.handle, None, xb.desc, xb.mem, wb.desc, wb.mem, bb.desc, bb.mem, None, 0, 0,
                                                              None, yb.desc, yb.mem, cb.ACTIVATION_RELU, 0), "bf16 conv, dispatcher")
        ops = conv_flops(shape[0], shape[1], shape[2], ch, ch, r, r)
        rec = {}
        for name, fn in (("int32_out", exact), ("int8_requant_out", requant), ("bf16_same_shape", bf16), ("bf16_dispatcher", bf16_dispatcher)):
            ms = time_calls(hip, ctx, fn, iters)
            rec[name] = {"us": ms * 1e3, "tops": ops / (ms * 1e-3) / 1e12}
        rec["int8_over_bf16"] = {"int32_out": rec["bf16_same_shape"]["us"] / rec["int32_out"]["us"],
                                 "int8_requant_out": rec["bf16_same_shape"]["us"] / rec["int8_requant_out"]["us"]}
        rec["int8_over_bf16_dispatcher"] = {"int32_out": rec["bf16_dispatcher"]["us"] / rec["int32_out"]["us"],
                                            "int8_requant_out": rec["bf16_dispatcher"]["us"] / rec["int8_requant_out"]["us"]}
        out["%dx%d" % (r, r)] = rec
        w.close()
        wb.close()
    for t in (x, b, scale, y, q, xb, bb, yb):
        t.close()
    return out


def nonfused_stages(hip, ctx, dtype, mat_dtype, m, iters, shape=(256, 15, 128), acc_dtype="f32", rates=None):
    """The four-call non-fused Winograd sequence F(m x m, 3x3) on one layer, one timing per stage.  shape = (N, H = W, C = K):
    the body convolution of config 2 by default, (64, 56, 256) for config 3.  mat_dtype: U and V, acc_dtype: M.
    Algorithmic bytes per stage: input x + V; GEMM V + U + M; output M + y + bias (weight transform w + U).  The GEMM stage is
    reported against the MFMA peak and against min(MFMA peak, arithmetic intensity x 8 TB/s), the roof a product that streams V
    and M through HBM has."""
    lib = cb.load_library()
    g = np.random.default_rng(SEED + 5)
    N, HW, ch = shape
    d, md, ad = DT[dtype], DT[mat_dtype], DT[acc_dtype]
    t = m + 2
    tiles = N * ((HW + m - 1) // m) ** 2
    esz, msz, asz = cb.DTYPE_SIZE[d], cb.DTYPE_SIZE[md], cb.DTYPE_SIZE[ad]
    x = cb.DeviceTensor.from_numpy(g.standard_normal((N, HW, HW, ch)).astype(np.float32), d)
    w = cb.DeviceTensor.from_numpy((g.standard_normal((ch, 3, 3, ch)) * np.sqrt(2.0 / (9 * ch))).astype(np.float32), d)
    b = cb.DeviceTensor.from_numpy(g.uniform(-0.1, 0.1, ch).astype(np.float32), cb.DTYPE_FLOAT32)
    U = cb.DeviceTensor((t * t, ch, ch), md)
    V = cb.DeviceTensor((t * t, tiles, ch), md)
    Mx = cb.DeviceTensor((t * t, tiles, ch), ad)
    y = cb.DeviceTensor((N, HW, HW, ch), d)
    conv = cb.ConvolutionDescriptor(padding=(-1, -1), dtype=d)
    h = ctx.handle
    calls = {
        "weight_transform": lambda: cb.check(lib.cudaWinogradWeightTransform(h, conv.handle, m, w.desc, w.mem, U.desc, U.mem), "weight"),
        "input_transform": lambda: cb.check(lib.cudaWinogradInputTransform(h, conv.handle, m, w.desc, x.desc, x.mem, V.desc, V.mem), "input"),
        "gemm": lambda: cb.check(lib.cudaGemmBatched(h, 0, 1, None, V.desc, V.mem, U.desc, U.mem, None, Mx.desc, Mx.mem), "gemm"),
        "output_transform": lambda: cb.check(lib.cudaWinogradOutputTransform(h, conv.handle, m, w.desc, None, Mx.desc, Mx.mem, y.desc, y.mem, b.desc, b.mem,
                                                                          None, 0, 0, None, cb.ACTIVATION_RELU), "output"),
    }
    xbytes = N * HW * HW * ch * esz
    alg_bytes = {"weight_transform": ch * 9 * ch * esz + t * t * ch * ch * msz, "input_transform": xbytes + t * t * tiles * ch * msz,
                 "gemm": t * t * tiles * ch * msz + t * t * ch * ch * msz + t * t * tiles * ch * asz,
                 "output_transform": t * t * tiles * ch * asz + xbytes + 4 * ch}
    written = {"weight_transform": t * t * ch * ch * msz, "input_transform": t * t * tiles * ch * msz, "gemm": t * t * tiles * ch * asz,
               "output_transform": xbytes}
    gemm_flops = 2.0 * t * t * tiles * ch * ch
    out = {"shape": {"N": N, "HW": HW, "channels": ch, "tiles": tiles}, "matrices": mat_dtype, "M": acc_dtype}
    total = 0.0
    for name, fn in calls.items():
        ms = time_calls(hip, ctx, fn, iters)
        rec = {"us": ms * 1e3, "MB": alg_bytes[name] / 1e6, "GBs": alg_bytes[name] / (ms * 1e-3) / 1e9,
               "hbm_frac": alg_bytes[name] / (ms * 1e-3) / 1e9 / PEAK["hbm_GBs"]}
        if rates is not None:
            # the time a kernel that streams the same bytes at the read-only and write-only rates measured on this box in this run
            # (avhip_stream_probe, 1 GiB) would take, reads and writes one after the other, over the stage's time
            floor_ms = ((alg_bytes[name] - written[name]) / rates["read"] + written[name] / rates["write"]) / 1e6
            rec["frac_of_measured_stream_rates"] = floor_ms / ms
        if name == "gemm":
            rec["gflop"] = gemm_flops / 1e9
            rec["tflops"] = gemm_flops / (ms * 1e-3) / 1e12
            rec["mfma_frac"] = rec["tflops"] / PEAK[mat_dtype]
            intensity = gemm_flops / alg_bytes[name]
            roof = min(PEAK[mat_dtype], intensity * PEAK["hbm_GBs"] / 1e3)
            rec["flop_per_byte"] = intensity
            rec["roof_min_mfma_hbm_tflops"] = roof
            rec["frac_of_that_roof"] = rec["tflops"] / roof
        out[name] = rec
        if name != "weight_transform":
            total += ms
    out["conv_tflops_direct_equivalent"] = conv_flops(N, HW, HW, ch, ch, 3, 3) / (total * 1e-3) / 1e12
    for tns in (x, w, b, U, V, Mx, y):
        tns.close()
    return out


def copy_bandwidth(hip, ctx, iters=10):
    lib = cb.load_library()
    nbytes = 1 << 30
    a, b = cb.DeviceTensor((nbytes,), cb.DTYPE_UINT8), cb.DeviceTensor((nbytes,), cb.DTYPE_UINT8)
    ms = time_calls(hip, ctx, lambda: cb.check(lib.cudaCopyMemory(ctx.handle, b.mem, 0, a.mem, 0, nbytes), "copy"), iters)
    a.close()
    b.close()
    return 2.0 * nbytes / (ms * 1e-3) / 1e9


def stream_rates(hip, ctx, iters=10):
    """Read-only, write-only and copy rates of streaming kernels with 16-byte accesses (avhip_stream_probe) over 1 GiB, GB/s:
    the ceilings an HBM-bound kernel of this library can reach on this box, next to the nominal 8 TB/s."""
    lib = cb.load_library()
    lib.avhip_stream_probe.restype = C.c_int
    lib.avhip_stream_probe.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int64]
    nbytes = 1 << 30
    a, b = cb.DeviceTensor((nbytes,), cb.DTYPE_UINT8), cb.DeviceTensor((nbytes,), cb.DTYPE_UINT8)
    out = {}
    for kind, name, moved in ((0, "read", 1.0), (1, "write", 1.0), (2, "copy", 2.0)):
        def call():
            assert lib.avhip_stream_probe(ctx.stream(), kind, a.pointer(), b.pointer(), nbytes) == 0
        ms = time_calls(hip, ctx, call, iters)
        out[name] = moved * nbytes / (ms * 1e-3) / 1e9
    a.close()
    b.close()
    return out


def mfma_rates(hip, ctx):
    """What the matrix cores sustain with register-resident operands and no memory traffic (avhip_mfma_rate_probe), per
    dtype, in T(FL)OP/s: with nearly all-zero operand bits (clock near boost) and with random finite operands, whose
    switching activity lowers the clock the power management allows; the datasheet peak assumes the boost clock."""
    lib = cb.load_library()
    lib.avhip_mfma_rate_probe.restype = C.c_int
    lib.avhip_mfma_rate_probe.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    workgroups, iterations = 256 * 8, 4096
    sink = cb.DeviceTensor((workgroups * 256,), cb.DTYPE_FLOAT32)
    out = {"quiet_operands": {}, "random_operands": {}}
    for operands, key in ((0, "quiet_operands"), (1, "random_operands")):
        for name, k, per_call in (("bf16", 16, 1), ("f16", 16, 1), ("i8", 32, 1), ("f32", 2, 4)):
            def call():
                assert lib.avhip_mfma_rate_probe(ctx.stream(), DT[name], workgroups, iterations, operands, sink.pointer()) == 0
            ms = time_calls(hip, ctx, call, 4, warmup=1)
            ops = workgroups * 4.0 * iterations * 8 * per_call * 2 * 32 * 32 * k
            out[key][name] = ops / (ms * 1e-3) / 1e12
    sink.close()
    return out


BASELINE_LAYERS = [("cfg1_f32_3x3_15x15_64", "f32", (8, 15, 15, 64), (64, 3, 3, 64), -1, 1),
                   ("cfg3_bf16_3x3_56x56_256", "bf16", (64, 56, 56, 256), (256, 3, 3, 256), -1, 1),
                   ("cfg3_f16_3x3_56x56_256", "f16", (64, 56, 56, 256), (256, 3, 3, 256), -1, 1),
                   ("cfg5_bf16_3x3_stride2_128_256", "bf16", (64, 56, 56, 128), (256, 3, 3, 128), -1, 2),
                   ("cfg5_bf16_1x1_256_512", "bf16", (64, 28, 28, 256), (512, 1, 1, 256), 0, 1),
                   ("cfg5_bf16_5x5_64_64", "bf16", (64, 32, 32, 64), (64, 5, 5, 64), -2, 1)]
# not BASELINE configs: first layers over image planes, the shapes of the thin-channel kernel
FIRST_LAYERS = [("bf16_7x7_stride2_3_64_224x224_N32", "bf16", (32, 224, 224, 3), (64, 7, 7, 3), -3, 2),
                ("bf16_5x5_3_32_128x128_N32", "bf16", (32, 128, 128, 3), (32, 5, 5, 3), -2, 1),
                ("f32_3x3_3_64_64x64_N64", "f32", (64, 64, 64, 3), (64, 3, 3, 3), -1, 1)]


def other_configs(hip, ctx, iters, cases=BASELINE_LAYERS):
    """Single layers through the dispatcher (bias + ReLU fused), one timing each: BASELINE configs 1, 3 and 5 by default."""
    lib = cb.load_library()
    g = np.random.default_rng(SEED + 7)
    out = {}
    for name, dtype, xs, ws, pad, stride in cases:
        d = DT[dtype]
        N, H, W, Cin = xs
        K, R, S, _ = ws
        Ho = (H - 2 * pad - R) // stride + 1
        x = cb.DeviceTensor.from_numpy(g.standard_normal(xs).astype(np.float32), d)
        w = cb.DeviceTensor.from_numpy((g.standard_normal(ws) * np.sqrt(2.0 / (R * S * Cin))).astype(np.float32), d)
        b = cb.DeviceTensor.from_numpy(g.uniform(-0.1, 0.1, K).astype(np.float32), cb.DTYPE_FLOAT32)
        y = cb.DeviceTensor((N, Ho, Ho, K), d)
        conv = cb.ConvolutionDescriptor(padding=(pad, pad), strides=(stride, stride), dtype=d)
        need = C.c_int64(0)
        cb.check(lib.cudaGetConvolutionWorkspaceSize(ctx.handle, conv.handle, x.desc, w.desc, b.desc, C.byref(need)), "workspace size")
        ws_mem = cb.DeviceTensor((max(int(need.value), 256),), cb.DTYPE_UINT8)

        def call():
            cb.check(lib.cudaConvolutionBiasActivationForward(ctx.handle, conv.handle, None, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, None, 0, 0, None,
                                                              y.desc, y.mem, cb.ACTIVATION_RELU, ws_mem.mem), "conv")
        ms = time_calls(hip, ctx, call, iters)
        out[name] = {"us": ms * 1e3, "tflops": conv_flops(N, Ho, Ho, K, Cin, R, S) / (ms * 1e-3) / 1e12}
        for t in (x, w, b, y, ws_mem):
            t.close()
    return out


def counter_calibration(ctx, launches=3):
    """Launches a plain streaming kernel of known traffic (fp32 -> fp16 conversion of 2^26 elements: 256 MiB read, 128 MiB
    written).  Under `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` its reading fixes the factor between the counter and bytes."""
    lib = cb.load_library()
    n = 1 << 26
    a, b = cb.DeviceTensor((n,), cb.DTYPE_FLOAT32), cb.DeviceTensor((n,), cb.DTYPE_FLOAT16)
    for _ in range(launches):
        cb.check(lib.cudaChangeType(ctx.handle, b.mem, cb.DTYPE_FLOAT16, a.mem, cb.DTYPE_FLOAT32, n), "cudaChangeType")
    ctx.synchronize()
    a.close()
    b.close()


# ---- CPU legs: the oracle as checker of the timed region's output, and the timed CPU baseline ------------------------------------
LAYER_BAR = {"bf16": 2e-3, "f16": 2e-3, "f32": 1e-4}   # one convolution against the oracle on the same inputs (rel-L2)
# 21 chained convolutions against the oracle chained the same way: output roundings that fall the other way propagate through
# the layers (measured 7e-3 / 1e-3 / 2e-6), while a layer that used wrong weights or a wrong buffer gives an error of order one
CHAIN_BAR = {"bf16": 2e-2, "f16": 4e-3, "f32": 2e-4}


def check_layer(orc, tower, layer, x, z, y, images):
    """One convolution of the tower against the oracle on the GPU's own input (and residual) of that layer, for some images.
    Returns the largest rel-L2 error over the images."""
    w, b = tower.host_layers[layer]
    wr = orc.round_to(w, tower.dtype)
    worst = 0.0
    for n in images:
        xin = x.download_slice(n)
        zin = z.download_slice(n) if z is not None else None
        want = orc.conv2d(xin, wr, b.astype(np.float64), zin, activation=orc.RELU)
        worst = max(worst, orc.rel_l2(y.download_slice(n), want))
    return worst


def check_chain(orc, tower, out, images):
    """The whole pass for some images: the oracle chained through all 21 layers with the tower's buffer rotation restated on the host
    (each layer's output rounded to the tensor dtype, as the device stores it), against the final activation `out`."""
    worst = 0.0
    for n in images:
        a = tower.x0.download_slice(n)
        layer = 0
        w, b = tower.host_layers[0]
        a = orc.round_to(orc.conv2d(a, orc.round_to(w, tower.dtype), b.astype(np.float64), activation=orc.RELU), tower.dtype)
        layer = 1
        for _ in range(tower.blocks):
            w, b = tower.host_layers[layer]
            t = orc.round_to(orc.conv2d(a, orc.round_to(w, tower.dtype), b.astype(np.float64), activation=orc.RELU), tower.dtype)
            w, b = tower.host_layers[layer + 1]
            a = orc.round_to(orc.conv2d(t, orc.round_to(w, tower.dtype), b.astype(np.float64), a, activation=orc.RELU), tower.dtype)
            layer += 2
        worst = max(worst, orc.rel_l2(out.download_slice(n), a))
    return worst


def self_check(tower, out, images=(0,)):
    """Checks what the timed region left in the tower's buffers: the last convolution teacher-forced on the device's own
    inputs, and the whole chain of 21.  Raises when either misses its bar, so that no figure is reported for wrong results."""
    from oracle import oracle as orc
    a, t, b = tower.act
    last = 2 * tower.blocks
    residual = [buf for buf in tower.act if buf is not out and buf is not t][0]
    e_layer = check_layer(orc, tower, last, t, residual, out, images)
    e_chain = check_chain(orc, tower, out, images)
    if not (e_layer < LAYER_BAR[tower.dtype] and e_chain < CHAIN_BAR[tower.dtype]):
        raise AssertionError("tower self-check failed (%s): last layer rel-L2 %.3e (bar %.0e), chain of 21 rel-L2 %.3e (bar %.0e)"
                             % (tower.dtype, e_layer, LAYER_BAR[tower.dtype], e_chain, CHAIN_BAR[tower.dtype]))
    return {"checked": True, "images": list(images), "last_layer_rel_l2": e_layer, "chain_rel_l2": e_chain}


def cpu_baseline(seconds=12.0):
    """fp32 direct convolution of the body layer (128->128, 15x15, 3x3) on a batch slice, all host cores."""
    from oracle import oracle as orc
    g = np.random.default_rng(SEED + 6)
    n = 32
    x = g.standard_normal((n, 15, 15, 128)).astype(np.float32)
    w = (g.standard_normal((128, 3, 3, 128)) * np.sqrt(2.0 / (9 * 128))).astype(np.float32)
    b = g.uniform(-0.1, 0.1, 128).astype(np.float32)
    orc.baseline_conv2d_f32(x, w, b)  # warm the threads and the caches
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < seconds:
        orc.baseline_conv2d_f32(x, w, b)
        reps += 1
    dt = time.perf_counter() - t0
    flops = conv_flops(n, 15, 15, 128, 128, 3, 3) * reps
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": orc.baseline_threads(), "kind": "port",
            "sample": "fp32 3x3 conv 128->128 15x15, batch slice N=%d of 256, %d repetitions in %.1f s (restated CPU reference, not AvocadoML/CpuBackend)"
                      % (n, reps, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32"])
    ap.add_argument("--quick", action="store_true", help="headline tower only (no side legs, no CPU baseline)")
    ap.add_argument("--calibrate", action="store_true", help="also launch a streaming kernel of known traffic (for counter runs)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU legs: the baseline and the oracle check of the towers' outputs (for counter runs, where only the GPU side matters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards over the batch with no collectives)." % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    lib = cb.load_library()
    if lib.cudaGetNumberOfDevices() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    hip = Hip()
    ctx = cb.Context(0)
    head = time_tower(hip, ctx, args.dtype, args.steps, args.warmup, check=not args.no_cpu)
    detail = {"headline": head}
    cpu = None
    if args.calibrate:
        counter_calibration(ctx)
    if not args.quick:
        it = max(5, args.steps)
        for other in ("f32", "bf16", "f16"):
            if other != args.dtype:
                detail["tower_" + other] = time_tower(hip, ctx, other, max(3, args.steps // 2), 2, check=not args.no_cpu)
        detail["caller_level_two_chains_of_128"] = two_half_batch_chains(hip, args.dtype, args.steps)
        detail["int8_config4"] = int8_leg(hip, ctx, it)
        # the same comparison on a layer large enough for the k loop to dominate the fixed cost of a launch (the shape of config 3)
        detail["int8_at_config3_shape"] = int8_leg(hip, ctx, it, shape=(64, 56, 56, 256), filters=((3, -1),))
        detail["copy_GBs_measured"] = copy_bandwidth(hip, ctx)
        rates = detail["stream_GBs_measured"] = stream_rates(hip, ctx)
        detail["nonfused_winograd_f32_F4"] = nonfused_stages(hip, ctx, "f32", "f32", 4, it, rates=rates)
        detail["nonfused_winograd_bf16_F2_fp16mat"] = nonfused_stages(hip, ctx, "bf16", "f16", 2, it, rates=rates)
        detail["nonfused_winograd_f16_F2_fp16mat_fp16M"] = nonfused_stages(hip, ctx, "f16", "f16", 2, it, acc_dtype="f16", rates=rates)
        detail["nonfused_winograd_bf16_F2_fp16mat_fp16M"] = nonfused_stages(hip, ctx, "bf16", "f16", 2, it, acc_dtype="f16", rates=rates)
        cfg3 = (64, 56, 256)
        detail["config3_nonfused_winograd"] = {
            "bf16_F2_fp16mat": nonfused_stages(hip, ctx, "bf16", "f16", 2, it, shape=cfg3, rates=rates),
            "f16_F2_fp16mat_fp16M": nonfused_stages(hip, ctx, "f16", "f16", 2, it, shape=cfg3, acc_dtype="f16", rates=rates),
            "bf16_F2_fp16mat_fp16M": nonfused_stages(hip, ctx, "bf16", "f16", 2, it, shape=cfg3, acc_dtype="f16", rates=rates),
            "bf16_F4_fp32mat": nonfused_stages(hip, ctx, "bf16", "f32", 4, it, shape=cfg3, rates=rates),
            "f16_F4_fp32mat": nonfused_stages(hip, ctx, "f16", "f32", 4, it, shape=cfg3, rates=rates),
        }
        detail["mfma_rate_measured"] = mfma_rates(hip, ctx)
        detail["other_configs"] = other_configs(hip, ctx, it)
        detail["first_layers_beyond_baseline"] = other_configs(hip, ctx, it, FIRST_LAYERS)
        cpu = None if args.no_cpu else cpu_baseline()
    ctx.close()
    peak = PEAK[args.dtype]
    line = {
        "metric": "3x3 conv TFLOP/s + % MFMA/HBM roofline at N=256,15x15,128ch; int8 TOPS",
        "value": head["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "BASELINE config 2: residual tower N=256 15x15 128ch, stem 4->128 + 10 blocks (21 3x3 convs), NHWC, bias+ReLU+residual fused",
                   "global_batch": 256, "entry": "cudaConvolutionBiasActivationForward"},
        "roofline": {"bound": "mfma", "achieved": head["body_conv_tflops"], "peak": peak, "unit": "TFLOP/s", "frac": head["body_conv_tflops"] / peak,
                     "traffic": COUNTED_TRAFFIC_BYTES.get(args.dtype),
                     "traffic_source": "constant from the committed FETCH_SIZE / WRITE_SIZE counter runs (profiles/), not measured in this run",
                     "kernel": "body 3x3 conv 128->128 (k_winograd_rows for 16-bit tensors: F(2,3) along rows, 12.885 GFLOP issued to the matrix cores "
                               "for the 16.987 GFLOP of the direct form): direct-equivalent flops / ((graph-replayed pass - stem) / 20) by HIP events"},
        "cpu_baseline": cpu,
        "detail": detail,
    }
    # the same fraction by the flops the kernel really issues (the row-wise Winograd form needs 2/3 of the direct form's multiplies)
    if args.dtype != "f32":
        line["roofline"]["frac_of_peak_by_issued_flops"] = line["roofline"]["frac"] * 12.885 / 16.987
    detail["timing"] = ("towers: median of 5 timings of `steps` graph replays each (min and max in ms_per_step_groups); single layers and stages: "
                        "median of 3 timings of a graph of 10 calls, replayed max(2, steps // 2) times, %d times when a call takes 50 us or more"
                        % LONG_CALL_REPLAYS)
    rates = detail.get("mfma_rate_measured")
    if rates is not None:
        # the same fraction against what the matrix cores of THIS box sustain on random operands with nothing else running
        key = {"bf16": "bf16", "f16": "f16", "f32": "f32"}[args.dtype]
        line["roofline"]["frac_of_measured_mfma_rate"] = head["body_conv_tflops"] / rates["random_operands"][key]
    print(json.dumps(line))


if __name__ == "__main__":
    main()
