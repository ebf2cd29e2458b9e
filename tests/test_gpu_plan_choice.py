"""The dispatcher's choice among the one-kernel plans, held against the clock on the layers of the BASELINE configurations: the plan
it takes by itself must not be slower than what it would run with that plan switched off.  (Parity of every plan is tested
elsewhere; this pins that the thresholds of `rows_winograd_pays`, `strided_kernel_pays` and `pointwise_block_pays` point the
right way where it matters.)  Times are HIP events around graph replays, the same helper bench.py uses; the margin of 10 % is far
inside the differences measured (30-55 %), so the box-to-box spread of the clocks does not decide the outcome."""
import pytest

import cudabackend_amd as cb

pytestmark = pytest.mark.gpu

# name, dtype, x, w, padding, stride; the switch of the plan the dispatcher is expected to take
LAYERS = [
    (("config 2 body 3x3 128->128", "bf16", (256, 15, 15, 128), (128, 3, 3, 128), -1, 1), "avhip_set_winograd_rows"),
    (("config 3 3x3 256->256", "bf16", (64, 56, 56, 256), (256, 3, 3, 256), -1, 1), "avhip_set_winograd_rows"),
    (("config 5 3x3 stride 2 128->256", "bf16", (64, 56, 56, 128), (256, 3, 3, 128), -1, 2), "avhip_set_conv_strided"),
    (("config 5 1x1 256->512", "bf16", (64, 28, 28, 256), (512, 1, 1, 256), 0, 1), "avhip_set_pointwise_block"),
]


@pytest.mark.parametrize("case", range(len(LAYERS)))
def test_the_plan_taken_is_not_the_slower_one(case):
    import bench
    layer, switch = LAYERS[case]
    lib = cb.load_library()
    setter = getattr(lib, switch)
    setter.restype = int
    hip, ctx = bench.Hip(), cb.Context(0)
    times = {}
    previous = setter(1)
    try:
        for mode in (1, 0, 1, 0):
            setter(mode)
            us = bench.other_configs(hip, ctx, 10, [layer])[layer[0]]["us"]
            times[mode] = min(times.get(mode, us), us)
    finally:
        setter(previous)
        ctx.close()
    print("%s: %.1f us with the plan, %.1f us without" % (layer[0], times[1], times[0]))
    assert times[1] <= 1.10 * times[0]
