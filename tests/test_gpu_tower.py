"""The residual tower of BASELINE config 2 as the benchmark drives it (bench.Tower: 21 calls of cudaConvolutionBiasActivationForward,
three activation buffers rotating, the residual taken from two layers back; call sequence after app/CudaBackend.cu:401-420 of the
reference, entry src/convolution.cu:36-44), chained on the device and checked against the CPU oracle layer by layer: every
convolution is compared on the device's own input of that layer, so the single-convolution bars apply to each of the 21
(fp32 through the Winograd plans 1e-4, 16-bit 2e-3, rel-L2), and the whole chain is compared with the oracle chained the same way.
Then the same pass as a replayed HIP graph, and after one layer's weights were rewritten through the API."""
import numpy as np
import pytest

import bench
import cudabackend_amd as cb

pytestmark = pytest.mark.gpu

IMAGES = (0, 77)


def _eager_pass_checked(oracle, tower, ctx):
    errors = []

    def after(layer, x, z, y):
        ctx.synchronize()
        errors.append(bench.check_layer(oracle, tower, layer, x, z, y, IMAGES))
    out = tower.step(after)
    ctx.synchronize()
    assert len(errors) == 21
    worst = max(errors)
    print("tower %s: worst layer rel-L2 %.3e at layer %d" % (tower.dtype, worst, int(np.argmax(errors))), flush=True)
    assert worst < bench.LAYER_BAR[tower.dtype], errors
    chain = bench.check_chain(oracle, tower, out, IMAGES)
    print("tower %s: chain of 21 rel-L2 %.3e" % (tower.dtype, chain), flush=True)
    assert chain < bench.CHAIN_BAR[tower.dtype]
    return out


def _buffers(tower):
    return [t.download_raw().copy() for t in tower.act]


def _scribble(tower, ctx):
    """Eager work between graph replays: every activation buffer is overwritten, so a replay cannot pass on stale contents."""
    pattern = np.array([0x7F7F7F7F], dtype=np.uint32)
    for t in tower.act:
        cb.check(tower.lib.cudaSetMemory(ctx.handle, t.mem, 0, t.nbytes, pattern.ctypes.data, 4), "cudaSetMemory")
    ctx.synchronize()


@pytest.mark.parametrize("dtype", ["bf16", "f32", "f16"])
def test_tower_chain_eager_graph_and_rewritten_weights(oracle, dtype):
    hip = bench.Hip()
    with cb.Context(0) as ctx:
        tower = bench.Tower(ctx, dtype, N=128)
        try:
            # 1. 21 eager calls, each layer checked on the device's own inputs, then the chain
            out = _eager_pass_checked(oracle, tower, ctx)
            eager = _buffers(tower)
            # 2. the same pass captured once and replayed, with eager work and synchronisation between the replays
            final = []
            exe = hip.capture(ctx.stream(), lambda: final.append(tower.step()))
            assert final[0] is out
            for replay in range(3):
                _scribble(tower, ctx)
                hip.launch(exe, ctx.stream())
                ctx.synchronize()
                for got, want in zip(_buffers(tower), eager):
                    np.testing.assert_array_equal(got, want, err_msg="graph replay %d differs from the eager pass" % replay)
            hip.rt.hipGraphExecDestroy(exe)
            # 3. one layer's weights rewritten through the API: the next pass must use them (the Winograd plans cache transformed weights)
            g = np.random.default_rng(5)
            for layer in (7, 20):
                w_old = tower.host_layers[layer][0]
                tower.set_weights(layer, (g.standard_normal(w_old.shape) * np.sqrt(2.0 / (9 * tower.ch))).astype(np.float32))
            out2 = _eager_pass_checked(oracle, tower, ctx)
            assert not np.array_equal(out2.download_raw(), eager[tower.act.index(out)])
            # and a graph captured after the rewrite replays the new pass
            after_rewrite = _buffers(tower)
            exe = hip.capture(ctx.stream(), lambda: tower.step())
            for replay in range(2):
                _scribble(tower, ctx)
                hip.launch(exe, ctx.stream())
                ctx.synchronize()
                for got, want in zip(_buffers(tower), after_rewrite):
                    np.testing.assert_array_equal(got, want)
            hip.rt.hipGraphExecDestroy(exe)
        finally:
            tower.close()


def test_bench_self_check_catches_a_wrong_layer(oracle):
    """The checker bench.py runs after its timed region must fail when a layer computed something else: here the last layer's
    host copy of the weights is changed behind the device's back."""
    with cb.Context(0) as ctx:
        tower = bench.Tower(ctx, "bf16", N=4)
        try:
            out = tower.step()
            ctx.synchronize()
            rec = bench.self_check(tower, out)
            assert rec["checked"] and rec["last_layer_rel_l2"] < 2e-3
            w, b = tower.host_layers[11]
            tower.host_layers[11] = (w[::-1].copy(), b)  # filters in another order: only the chain check can see it
            with pytest.raises(AssertionError):
                bench.self_check(tower, out)
            tower.host_layers[11] = (w, b)
            w, b = tower.host_layers[20]
            tower.host_layers[20] = (w * np.float32(1.01), b)
            with pytest.raises(AssertionError):
                bench.self_check(tower, out)
        finally:
            tower.close()
