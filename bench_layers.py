"""Times every convolution shape of a 50-layer residual network (the layer list of ResNet-50 v1.5, NHWC, bias + ReLU fused), one
call per shape, on one MI355X.  Not a BASELINE config: a check of how the launcher's choice of kernel holds up over the layers a
front-end really sends (first layer over three image planes, 1x1 and 3x3 layers from 56x56 down to 7x7, strided ones).

    python bench_layers.py --batch 32 --dtype bf16            # through cudaConvolutionBiasActivationForward with its workspace
    python bench_layers.py --batch 32 --dtype bf16 --entry implicit_gemm
    python bench_layers.py --batch 256 --dtype i8             # int8 in, int8 out (requantised)

Prints one line per shape (count in the network, microseconds per call, rate) and the sum over the network.  Durations are HIP
events around replays of a ten-call graph, as in bench.py."""
import argparse
import ctypes as C

import numpy as np

import bench
import cudabackend_amd as cb

# (name, count in the network, input height = width, input channels, filters, filter size, stride)
LAYERS = [("conv1 7x7/2 3->64", 1, 224, 3, 64, 7, 2),
          ("stage1 1x1 64->64", 1, 56, 64, 64, 1, 1), ("stage1 3x3 64->64", 3, 56, 64, 64, 3, 1), ("stage1 1x1 64->256", 4, 56, 64, 256, 1, 1),
          ("stage1 1x1 256->64", 2, 56, 256, 64, 1, 1),
          ("stage2 1x1 256->128", 1, 56, 256, 128, 1, 1), ("stage2 3x3/2 128->128", 1, 56, 128, 128, 3, 2), ("stage2 1x1 128->512", 4, 28, 128, 512, 1, 1),
          ("stage2 1x1/2 256->512", 1, 56, 256, 512, 1, 2), ("stage2 1x1 512->128", 3, 28, 512, 128, 1, 1), ("stage2 3x3 128->128", 3, 28, 128, 128, 3, 1),
          ("stage3 1x1 512->256", 1, 28, 512, 256, 1, 1), ("stage3 3x3/2 256->256", 1, 28, 256, 256, 3, 2), ("stage3 1x1 256->1024", 6, 14, 256, 1024, 1, 1),
          ("stage3 1x1/2 512->1024", 1, 28, 512, 1024, 1, 2), ("stage3 1x1 1024->256", 5, 14, 1024, 256, 1, 1), ("stage3 3x3 256->256", 5, 14, 256, 256, 3, 1),
          ("stage4 1x1 1024->512", 1, 14, 1024, 512, 1, 1), ("stage4 3x3/2 512->512", 1, 14, 512, 512, 3, 2), ("stage4 1x1 512->2048", 3, 7, 512, 2048, 1, 1),
          ("stage4 1x1/2 1024->2048", 1, 14, 1024, 2048, 1, 2), ("stage4 1x1 2048->512", 2, 7, 2048, 512, 1, 1), ("stage4 3x3 512->512", 2, 7, 512, 512, 3, 1)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f16", "f32", "i8"])
    ap.add_argument("--entry", default="dispatch", choices=["dispatch", "implicit_gemm"], help="floating types only; int8 goes through avhipConvolutionRequantForward")
    args = ap.parse_args()
    lib = cb.load_library()
    hip, ctx = bench.Hip(), cb.Context(0)
    g = np.random.default_rng(bench.SEED + 11)
    d = bench.DT[args.dtype] if args.dtype != "i8" else cb.DTYPE_INT8
    N = args.batch
    total_us, total_flops = 0.0, 0.0
    for name, count, H, Cin, K, R, stride in LAYERS:
        pad = -(R // 2)
        Ho = (H - 2 * pad - R) // stride + 1
        conv = cb.ConvolutionDescriptor(padding=(pad, pad), strides=(stride, stride), dtype=d)
        held = []
        if args.dtype == "i8":
            x = cb.DeviceTensor.from_numpy(g.integers(-127, 128, (N, H, H, Cin), dtype=np.int8), d)
            w = cb.DeviceTensor.from_numpy(g.integers(-127, 128, (K, R, R, Cin), dtype=np.int8), d)
            b = cb.DeviceTensor.from_numpy(g.integers(-100, 100, K).astype(np.int32), cb.DTYPE_INT32)
            scale = cb.DeviceTensor.from_numpy(g.uniform(1e-4, 1e-3, K).astype(np.float32), cb.DTYPE_FLOAT32)
            y = cb.DeviceTensor((N, Ho, Ho, K), d)
            held = [scale]

            def call():
                cb.check(lib.avhipConvolutionRequantForward(ctx.handle, conv.handle, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, scale.desc, scale.mem,
                                                            y.desc, y.mem, cb.ACTIVATION_RELU), "requant")
        else:
            x = cb.DeviceTensor.from_numpy(g.standard_normal((N, H, H, Cin)).astype(np.float32), d)
            w = cb.DeviceTensor.from_numpy((g.standard_normal((K, R, R, Cin)) * np.sqrt(2.0 / (R * R * Cin))).astype(np.float32), d)
            b = cb.DeviceTensor.from_numpy(g.uniform(-0.1, 0.1, K).astype(np.float32), cb.DTYPE_FLOAT32)
            y = cb.DeviceTensor((N, Ho, Ho, K), d)
            need = C.c_int64(0)
            cb.check(lib.cudaGetConvolutionWorkspaceSize(ctx.handle, conv.handle, x.desc, w.desc, b.desc, C.byref(need)), "workspace size")
            ws = cb.DeviceTensor((max(int(need.value), 256),), cb.DTYPE_UINT8)
            held = [ws]
            if args.entry == "dispatch":
                def call():
                    cb.check(lib.cudaConvolutionBiasActivationForward(ctx.handle, conv.handle, None, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, None, 0, 0,
                                                                      None, y.desc, y.mem, cb.ACTIVATION_RELU, ws.mem), "dispatch")
            else:
                def call():
                    cb.check(lib.cudaConvolutionImplicitGemmForward(ctx.handle, conv.handle, None, x.desc, x.mem, w.desc, w.mem, b.desc, b.mem, None, 0, 0,
                                                                    None, y.desc, y.mem, cb.ACTIVATION_RELU), "implicit gemm")
        us = bench.time_calls(hip, ctx, call, 6) * 1e3
        flops = bench.conv_flops(N, Ho, Ho, K, Cin, R, R)
        print("%-26s x%d %9.1f us %8.1f TFLOP/s" % (name, count, us, flops / us / 1e6), flush=True)
        total_us += count * us
        total_flops += count * flops
        for t in [x, w, b, y] + held:
            t.close()
    ctx.close()
    print("batch %d %s: the network's %d convolutions %.1f us, %.1f TFLOP/s" % (N, args.dtype, sum(l[1] for l in LAYERS), total_us, total_flops / total_us / 1e6))


if __name__ == "__main__":
    main()
