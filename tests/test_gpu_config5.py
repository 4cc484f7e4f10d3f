"""ResNet-152, batch 128, 3x224x224, fp32, under a 16 GiB device budget.

The reference's swap-capable executor exists to run this workload
(tests/ResNet152_test.py:92-149 builds the [3, 8, 36, 3] bottleneck network;
pycode/tinyflow/autodiff.py:90-139, 2631-2836 is the swap protocol).  The test runs
it at its real size: first unswapped (288 GB of HBM hold it), then under the
budget with swapping + recomputation, then one swap-only step, and checks that

  * every step's loss under the budget has the bits of the unswapped step's loss,
    and the updated parameters after the last step are bit-identical too;
  * the allocator's high-water mark stays within the budget;
  * what was offloaded was prefetched back (nothing fetched on demand after the
    warm-up steps, offloaded bytes == prefetched bytes).
"""
import gc

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

BUDGET = 16 << 30
STEPS = 5
WARMUP = 2     # steps the executor may use to settle its plan


def _fingerprint(arrays):
    """Bits of a few parameters spread over the network (first, middle, last, some biases)."""
    picks = sorted(set([0, 1, len(arrays) // 3, len(arrays) // 2, (2 * len(arrays)) // 3, len(arrays) - 2,
                        len(arrays) - 1]))
    return [arrays[i].asnumpy().tobytes() for i in picks]


def test_resnet152_b128_under_16gib_matches_the_unswapped_run():
    from tinyflow_amd import gpu_op, models
    from tinyflow_amd.SwapExecute import SwapExecutor
    from tinyflow_amd.TrainExecute import TrainExecutor

    gpu_op.set_device_memory_limit(0)
    model, X, y = models.build("resnet152", batch=128)
    assert X.shape == (128, 3, 224, 224) and len(model.variables) == 157   # 155 convolutions + the classifier's W, b
    ex = TrainExecutor(model.loss, 0.01)
    ex.init_Variable(dict(model.variables))
    feed = {model.X: X, model.y_: y}
    plain_loss = []
    out = None
    for step in range(STEPS):
        out = ex.run(feed if step == 0 else {})
        plain_loss.append(out[0].asnumpy().tobytes())
    plain_params = _fingerprint(out[1:])
    losses = [float(np.frombuffer(b, np.float32)[0]) for b in plain_loss]
    assert all(np.isfinite(losses)) and losses[0] > 0
    ex.close()
    del ex, out
    gc.collect()

    try:
        gpu_op.set_device_memory_limit(BUDGET)
        for recompute, steps in ((True, STEPS), (False, 1)):
            model, X, y = models.build("resnet152", batch=128)
            gpu_op.device_memory_stats(reset_peak=True)
            ex = SwapExecutor(model.loss, 0.01, swap=True, memory_budget=BUDGET, prefetch_distance=12,
                              recompute=recompute)
            ex.init_Variable(dict(model.variables))
            feed = {model.X: X, model.y_: y}
            reports = [ex.swap_report()]
            for step in range(steps):
                out = ex.run(feed if step == 0 else {})
                assert out[0].asnumpy().tobytes() == plain_loss[step], \
                    "step %d (recompute=%s): loss differs from the unswapped run" % (step, recompute)
                reports.append(ex.swap_report())
            reserved, in_use, peak = gpu_op.device_memory_stats()
            assert peak <= BUDGET, "peak in use %d bytes exceeds the budget" % peak
            final = reports[-1]
            assert final["offload_bytes"] > (1 << 30), "nothing substantial was swapped: %r" % final
            assert (final["recomputed"] > 0) == recompute
            if recompute:
                assert _fingerprint(out[1:]) == plain_params
                settled = reports[WARMUP]
                assert final["passive_swap_in"] == settled["passive_swap_in"], \
                    "values were fetched on demand after the warm-up steps: %r" % final
                assert (final["offload_bytes"] - settled["offload_bytes"]
                        == final["prefetch_bytes"] - settled["prefetch_bytes"]
                        + final.get("passive_bytes", 0) - settled.get("passive_bytes", 0))
                assert final.get("passive_bytes", 0) == settled.get("passive_bytes", 0)
            else:
                # every offloaded byte came back, by prefetch or on demand
                assert final["offload_bytes"] == final["prefetch_bytes"] + final.get("passive_bytes", 0)
            print("recompute=%s: peak %.2f GiB, offloaded %.2f GB per step, %d recomputations, "
                  "passive swap-ins %d" % (recompute, peak / 2.0**30, final["offload_bytes"] / 1e9 / steps,
                                           final["recomputed"], final["passive_swap_in"]))
            ex.close()
            del ex, out
            gc.collect()
    finally:
        gpu_op.set_device_memory_limit(0)
