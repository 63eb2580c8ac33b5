"""The algorithm an automatic int8 handle picks must not lose much against the best forced one: the nine
distinct pointwise shapes of MobileNetV1-1.0 (int8 -> int8, relu, 90 % zeros) at 1, 4, 16 and 64 images per
launch, every algorithm the shape allows timed in the same process on the same buffers
(helpers.algo_times: parity-checked handles, interleaved runs, best of three).  A cell fails when the
automatic handle is more than 15 % (plus 0.3 us of timer resolution on these 4 to 17 us launches) slower than
the best forced algorithm."""
import pytest

from helpers import algo_times, workloads

pytestmark = pytest.mark.gpu

SHAPES = [(32, 64, 112), (64, 128, 56), (128, 128, 56), (128, 256, 28), (256, 256, 28), (256, 512, 14), (512, 512, 14), (512, 1024, 7), (1024, 1024, 7)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "%dx%d_%d" % s)
def test_auto_is_within_15_percent_of_the_best_forced_algorithm(shape):
    print("auto choice", shape, flush=True)
    index = workloads.MOBILENET_V1_POINTWISE.index(shape)
    slow = []
    for batch in (1, 4, 16, 64):
        case = workloads.config5_layer(index, batch=batch)
        times, picked = algo_times(case, warm=100, steps=400)
        best_name, best = min(((k, v) for k, v in times.items() if k != "auto"), key=lambda kv: kv[1])
        if times["auto"] > 1.15 * best + 0.3:
            # once more before failing: a burst on the box can land on one handle's runs
            times, picked = algo_times(case, warm=200, steps=800, repeats=5)
            best_name, best = min(((k, v) for k, v in times.items() if k != "auto"), key=lambda kv: kv[1])
            if times["auto"] > 1.15 * best + 0.3:
                slow.append("batch %d: auto (%s) %.2f us, %s %.2f us" % (batch, picked, times["auto"], best_name, best))
    assert not slow, "; ".join(slow)
