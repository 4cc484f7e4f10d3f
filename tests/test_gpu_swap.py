"""Swap path: activations moved to pinned host memory on a side stream and back.

Checks (i) byte-exact round trips device -> pinned host -> device on a side
stream while the compute stream is busy, (ii) that a training step executed with
releases + swapping is bit-identical to the plain executor's step, (iii) that the
swapping executor fits a device budget the plain executor does not fit, and that
the budget convention of DLArrayAlloc (report the size, return no array) holds.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _no_garbage_from_earlier_tests():
    """These tests read the allocator's in-use and peak counters: device arrays of an
    earlier test that are still waiting for the garbage collector would be freed at
    some point in the middle of a measurement."""
    import gc
    gc.collect()
    yield


def _shallow_resnet(batch=16, image=64, width=8):
    from tinyflow_amd import models
    rng = np.random.RandomState(9)
    X, y = models.synthetic_batch(rng, (batch, 3, image, image), 10, "normal")
    model = models.resnet(rng, [2, 1, 1, 1], batch, image=image, n_class=10, bn_mode="pre_activation", width=width)
    return model, X, y


def test_round_trip_on_side_stream_is_byte_exact(rt):
    from tinyflow_amd import gpu_op, ndarray
    side = gpu_op.create_cudaStream()
    rng = np.random.RandomState(30)
    arrays = [rng.normal(0, 1, s).astype(np.float32) for s in [(64, 64, 56, 56), (3, 5, 7), (1,), (1 << 20,)]]
    busy_a = ndarray.array(rng.normal(0, 1, (2048, 2048)).astype(np.float32), rt.ctx)
    busy_c = ndarray.empty((2048, 2048), rt.ctx)
    for x in arrays:
        dev = ndarray.array(x, rt.ctx)
        for _ in range(4):   # keep the compute stream busy while the copies run
            gpu_op.matrix_multiply(busy_a, False, busy_a, False, busy_c, rt.cublas, rt.stream)
        host = ndarray.empty(x.shape, ndarray.cpu(0))
        dev.copyto(host, side)
        dev.free_gpu()
        back = host.copyto(rt.ctx, side)
        assert back.asnumpy().tobytes() == x.tobytes()
    gpu_op.destroy_cudaStream(side)


def test_pcie_probe_runs():
    from tinyflow_amd import gpu_op
    gpu_op.testPcie()


def test_swapped_step_is_bit_identical_to_plain_step():
    from tinyflow_amd.SwapExecute import SwapExecutor
    from tinyflow_amd.TrainExecute import TrainExecutor
    results, moved = [], {}
    for kind in ("plain", "release", "swap", "recompute"):
        model, X, y = _shallow_resnet()
        if kind == "plain":
            ex = TrainExecutor(model.loss, 0.01)
        else:
            ex = SwapExecutor(model.loss, 0.01, swap=(kind != "release"), min_swap_bytes=1 << 12, prefetch_distance=4,
                              recompute=(kind == "recompute"))
            ex.keep_values = set(ex.Variable_node_grad_list)
        ex.init_Variable(dict(model.variables))
        feed = {model.X: X, model.y_: y}
        steps = []
        for _ in range(3):
            out = ex.run(feed)
            grads = [ex.value_of(g).asnumpy() for g in ex.Variable_node_grad_list]
            steps.append(([o.asnumpy() for o in out], grads))
        if kind in ("swap", "recompute"):
            rep = ex.swap_report()
            assert rep["offload_bytes"] > 0 and rep["prefetch_bytes"] == rep["offload_bytes"]
            assert rep["passive_swap_in"] == 0
            assert (rep["recomputed"] > 0) == (kind == "recompute")
            moved[kind] = rep["offload_bytes"]
        if kind != "plain":
            ex.close()
        results.append(steps)
    assert moved["recompute"] < 0.7 * moved["swap"]   # normalisation / activation outputs no longer travel
    for other in results[1:]:
        for (out_a, g_a), (out_b, g_b) in zip(results[0], other):
            for a, b in zip(out_a + g_a, out_b + g_b):
                assert a.tobytes() == b.tobytes()


def test_swapping_fits_a_budget_the_plain_executor_does_not():
    from tinyflow_amd import gpu_op, ndarray
    from tinyflow_amd.SwapExecute import SwapExecutor
    from tinyflow_amd.TrainExecute import TrainExecutor
    gpu_op.set_device_memory_limit(0)
    peaks = {}
    try:
        for kind in ("plain", "release", "swap"):
            model, X, y = _shallow_resnet(batch=32, image=96, width=16)
            base = gpu_op.device_memory_stats(reset_peak=True)[1]
            if kind == "plain":
                ex = TrainExecutor(model.loss, 0.01)
            else:
                ex = SwapExecutor(model.loss, 0.01, swap=(kind == "swap"), min_swap_bytes=1 << 16,
                                  prefetch_distance=4)
            ex.init_Variable(dict(model.variables))
            loss = None
            for _ in range(2):
                loss = ex.run({model.X: X, model.y_: y})[0].asnumpy()
            peaks[kind] = (gpu_op.device_memory_stats()[2] - base, float(loss[0]))
            if kind != "plain":
                ex.close()
            del ex
        assert peaks["release"][0] < 0.7 * peaks["plain"][0]
        assert peaks["swap"][0] < 0.9 * peaks["release"][0]
        assert peaks["plain"][1] == peaks["release"][1] == peaks["swap"][1]
        # a budget between the two: the swapping executor runs, a plain allocation of the rest does not
        base = gpu_op.device_memory_stats()[1]
        budget = base + int(peaks["swap"][0] * 1.15)
        gpu_op.set_device_memory_limit(budget)
        model, X, y = _shallow_resnet(batch=32, image=96, width=16)
        ex = SwapExecutor(model.loss, 0.01, swap=True, min_swap_bytes=1 << 16, prefetch_distance=4)
        ex.init_Variable(dict(model.variables))
        for _ in range(2):
            loss = ex.run({model.X: X, model.y_: y})[0].asnumpy()
        assert float(loss[0]) == peaks["swap"][1]
        assert gpu_op.device_memory_stats()[2] <= budget
        ex.close()
        # the allocation convention under the budget: an int (bytes wanted), no array
        too_big = ndarray.empty((budget // 4 + 1024,), ndarray.gpu(0))
        assert isinstance(too_big, int)
    finally:
        gpu_op.set_device_memory_limit(0)


def test_budget_arena_never_overlaps_and_coalesces():
    """Random allocate / free traffic under a budget: live arrays never overlap,
    their contents survive their neighbours' churn, and once everything is freed
    one array of nearly the whole budget fits again (free ranges were merged)."""
    import ctypes
    from tinyflow_amd import gpu_op, ndarray
    ctx = ndarray.gpu(0)
    base = gpu_op.device_memory_stats()[1]
    budget = 64 << 20
    gpu_op.set_device_memory_limit(base + budget)
    try:
        rng = np.random.RandomState(5)
        live = {}
        refused = 0
        for step in range(400):
            if live and (rng.rand() < 0.45 or len(live) > 40):
                key = list(live)[rng.randint(len(live))]
                arr, value = live.pop(key)
                assert np.all(arr.asnumpy() == value)
                arr.free_gpu()
            else:
                n = int(rng.choice([64, 1000, 4096, 70000, 300000, 1 << 20, 3 << 20]))
                arr = ndarray.empty((n,), ctx)
                if isinstance(arr, int):
                    refused += 1
                    assert arr == 4 * n
                    continue
                value = np.float32(step)
                gpu_op.array_set(arr, float(value), None)
                live[step] = (arr, value)
            spans = sorted((ctypes.cast(a.handle.contents.data, ctypes.c_void_p).value, 4 * a.shape[0])
                           for a, _ in live.values())
            for (p0, l0), (p1, _) in zip(spans, spans[1:]):
                assert p0 + l0 <= p1
            assert gpu_op.device_memory_stats()[1] - base <= budget
        for arr, value in live.values():
            assert np.all(arr.asnumpy() == value)
            arr.free_gpu()
        assert gpu_op.device_memory_stats()[1] == base
        whole = ndarray.empty(((budget - (1 << 20)) // 4,), ctx)
        assert not isinstance(whole, int)
        whole.free_gpu()
    finally:
        gpu_op.set_device_memory_limit(0)


def test_a_new_budget_counts_arrays_that_outlive_the_previous_one():
    """Changing the budget while arrays of the old budget are alive: those arrays count
    against the new budget until they are freed."""
    from tinyflow_amd import gpu_op, ndarray
    ctx = ndarray.gpu(0)
    base = gpu_op.device_memory_stats()[1]
    mib = 1 << 20
    gpu_op.set_device_memory_limit(base + 8 * mib)
    try:
        a = ndarray.empty((mib,), ctx)                     # 4 MiB under the first budget
        assert not isinstance(a, int)
        gpu_op.array_set(a, 3.0, None)
        gpu_op.set_device_memory_limit(base + 6 * mib)
        assert isinstance(ndarray.empty((mib,), ctx), int)  # 4 + 4 MiB do not fit 6
        small = ndarray.empty((mib // 4,), ctx)            # 4 + 1 MiB do
        assert not isinstance(small, int)
        assert gpu_op.device_memory_stats()[1] - base <= 6 * mib
        assert np.all(a.asnumpy() == 3.0)
        a.free_gpu()
        b = ndarray.empty((mib,), ctx)                     # now 1 + 4 MiB
        assert not isinstance(b, int)
        assert gpu_op.device_memory_stats()[1] - base <= 6 * mib
        b.free_gpu()
        small.free_gpu()
        assert gpu_op.device_memory_stats()[1] == base
    finally:
        gpu_op.set_device_memory_limit(0)


def test_planner_lists_drive_the_step_bit_identically():
    """A schedule handed over in the planner's wire format (swap list, release
    list, recomputation list) gives the same bits as the plain executor: the
    built-in schedule is exported, every ReLU output is additionally released
    right after its forward use and listed for recomputation before its first
    backward use."""
    from tinyflow_amd.SwapExecute import SwapExecutor, schedule_to_wire
    from tinyflow_amd.TrainExecute import TrainExecutor
    model, X, y = _shallow_resnet()
    plain = TrainExecutor(model.loss, 0.01)
    plain.init_Variable(dict(model.variables))
    want = [[o.asnumpy() for o in plain.run({model.X: X, model.y_: y})] for _ in range(2)]

    model, X, y = _shallow_resnet()
    ex = SwapExecutor(model.loss, 0.01, swap=True, min_swap_bytes=1 << 19, prefetch_distance=4)
    ex.init_Variable(dict(model.variables))
    ex.run({model.X: X, model.y_: y})            # builds the built-in schedule (and is step 1)
    pos = {n: i for i, n in enumerate(ex.topo_order)}
    as_ids = lambda table: {t: [pos[n] for n in ns] for t, ns in table.items()}
    swap_out, swap_in, release = as_ids(ex.swap_out_at), as_ids(ex.swap_in_at), as_ids(ex.release_at)
    moved = {i for ids in swap_out.values() for i in ids}
    recompute = []
    first_backward = min(pos[n] for n in ex.topo_order if n not in ex.forward_nodes and n.isw not in (1, 2))
    for n in ex.topo_order:
        uses = ex.uses[n]
        if type(n.op).__name__ == "ActivationForwardOp" and n in ex.forward_nodes and pos[n] not in moved:
            fwd = [u for u in uses if u < first_backward]
            bwd = [u for u in uses if u >= first_backward]
            if fwd and bwd and n not in ex.keep:
                release.setdefault(fwd[-1], []).append(pos[n])
                recompute.append((bwd[0], pos[n], False))
    swaps, releases = schedule_to_wire(swap_out, swap_in, release)
    # a fresh executor fed only with the lists
    model, X, y = _shallow_resnet()
    ex2 = SwapExecutor(model.loss, 0.01, swap=True)
    ex2.init_Variable(dict(model.variables))
    ex2.set_schedule(swaps, releases, recompute)
    got = [[o.asnumpy() for o in ex2.run({model.X: X, model.y_: y})] for _ in range(2)]
    rep = ex2.swap_report()
    assert rep["offload_bytes"] > 0 and rep["passive_swap_in"] == 0
    assert recompute and rep["recomputed"] >= len(recompute)
    for a_step, b_step in zip(want, got):
        for a, b in zip(a_step, b_step):
            assert a.tobytes() == b.tobytes()
    ex.close()
    ex2.close()


def test_planner_message_carries_measured_runtimes():
    """The executor -> planner report after a measured step: every computed node has a
    positive runtime, the convolutions' runtimes dominate, sizes match the arrays, and
    the measuring step itself still gives the plain executor's bits."""
    from tinyflow_amd.SwapExecute import SwapExecutor
    from tinyflow_amd.TrainExecute import TrainExecutor
    pmodel, pX, py = _shallow_resnet()
    plain = TrainExecutor(pmodel.loss, 0.01)
    plain.init_Variable(dict(pmodel.variables))
    want = [o.asnumpy() for o in plain.run({pmodel.X: pX, pmodel.y_: py})]

    model, X, y = _shallow_resnet()
    ex = SwapExecutor(model.loss, 0.01, swap=False)
    ex.init_Variable(dict(model.variables))
    ex.measure_runtimes = True
    got = [o.asnumpy() for o in ex.run({model.X: X, model.y_: y})]
    ex.measure_runtimes = False
    for a, b in zip(want, got):
        assert a.tobytes() == b.tobytes()
    msg = ex.planner_message()
    assert len(msg) == len(ex.topo_order)
    # the measured times can also place the prefetches of the built-in schedule
    ex.replan()
    again = [o.asnumpy() for o in ex.run({model.X: X, model.y_: y})]
    second = [o.asnumpy() for o in plain.run({pmodel.X: pX, pmodel.y_: py})]
    for a, b in zip(second, again):
        assert a.tobytes() == b.tobytes()
    by_kind = {}
    for node, (tensors, inputs, name, op_id, flag, _, runtime) in zip(ex.topo_order, msg):
        if node.isw in (1, 2):
            assert runtime == 1e-8            # fed, not computed
            continue
        assert 1e-8 <= runtime < 0.5, (name, runtime)
        by_kind[type(node.op).__name__] = by_kind.get(type(node.op).__name__, 0.0) + runtime
        if not node.issgd:
            assert tensors[0][1] == 4 * int(np.prod(ex.tensors[node].shape))
    conv = sum(v for k, v in by_kind.items() if k.startswith("Convolution"))
    assert conv > 0 and conv >= 0.2 * sum(by_kind.values()), by_kind
    ex.close()


def test_swapping_adam_executor_is_bit_identical_to_the_plain_adam_executor():
    """The swap-capable executor with the reference's optimizer (Adam): three steps with
    swapping and recomputation give the bits of TrainExecuteAdam's plain executor."""
    from tinyflow_amd.SwapExecute import SwapExecutor
    from tinyflow_amd.TrainExecuteAdam import TrainExecutor
    model, X, y = _shallow_resnet()
    plain = TrainExecutor(model.loss, 0.001)
    plain.init_Variable(dict(model.variables))
    want = [[o.asnumpy() for o in plain.run({model.X: X, model.y_: y})] for _ in range(3)]

    model, X, y = _shallow_resnet()
    ex = SwapExecutor(model.loss, 0.001, swap=True, min_swap_bytes=1 << 19, prefetch_distance=4, recompute=True,
                      optimizer="adam")
    ex.init_Variable(dict(model.variables))
    got = [[o.asnumpy() for o in ex.run({model.X: X, model.y_: y})] for _ in range(3)]
    assert ex.swap_report()["offload_bytes"] > 0
    assert abs(ex.b1t[0] - 0.9 ** 4) < 1e-12
    for a_step, b_step in zip(want, got):
        for a, b in zip(a_step, b_step):
            assert a.tobytes() == b.tobytes()
    ex.close()


@pytest.mark.parametrize("budget", [False, True], ids=["pool", "arena"])
def test_copy_into_fresh_array_is_byte_exact_and_ordered_after_the_storage_s_previous_life(rt, budget):
    """DLArrayCopyIntoFresh: a block is filled by a kernel, read back, released and
    reallocated; the host -> device copy into the recycled storage must not overtake
    the kernel that was still queued when the block was released.  Run on the caching
    pool and, under a budget, on the arena (where the recycled range is found by address)."""
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(41)
    shape = (1 << 22,)
    side = gpu_op.create_cudaStream()
    host = ndarray.array(rng.normal(0, 1, shape).astype(np.float32), ndarray.cpu(0))
    if budget:
        gpu_op.set_device_memory_limit(gpu_op.device_memory_stats()[1] + (40 << 20))   # room for two of them
    try:
        _copy_into_fresh_trials(rt, gpu_op, ndarray, shape, host, side)
    finally:
        if budget:
            gpu_op.set_device_memory_limit(0)
    gpu_op.destroy_cudaStream(side)


def _copy_into_fresh_trials(rt, gpu_op, ndarray, shape, host, side):
    for trial in range(4):
        a = ndarray.empty(shape, rt.ctx)
        b = ndarray.empty(shape, rt.ctx)
        gpu_op.array_set(a, float(trial + 1), rt.stream)
        for _ in range(8):   # a queue of work that reads a
            gpu_op.matrix_elementwise_multiply_by_const(a, 1.0, b, rt.stream)
        a.free_gpu()         # stream-ordered release: the kernels above still read the block
        fresh = ndarray.empty(shape, rt.ctx)   # the same size: the pool hands the block back
        if trial % 2 == 0:
            fresh.prepare_fresh()   # with the fence: waits for the queue above only; without: for everything
        host.copy_into_fresh(fresh, side)
        np.testing.assert_array_equal(b.asnumpy(), np.full(shape, trial + 1, np.float32))
        assert fresh.asnumpy().tobytes() == host.asnumpy().tobytes()
        b.free_gpu()
        fresh.free_gpu()


def test_planned_budget_adapts_when_a_step_has_to_evict():
    """A plan made for more memory than the device limit grants runs into on-demand
    evictions; the executor then plans for 3 % less per offending step until the steps
    fit, and every step -- evicting or not -- gives the plain executor's bits."""
    from tinyflow_amd import gpu_op
    from tinyflow_amd.SwapExecute import SwapExecutor
    from tinyflow_amd.TrainExecute import TrainExecutor
    model, X, y = _shallow_resnet(batch=32, image=96, width=16)
    plain = TrainExecutor(model.loss, 0.01)
    plain.init_Variable(dict(model.variables))
    steps = 8
    want = [plain.run({model.X: X, model.y_: y})[0].asnumpy().tobytes() for _ in range(steps)]
    del plain
    # what the released-early executor needs at its peak, then a limit 25 % below it
    gpu_op.set_device_memory_limit(0)
    try:
        model, X, y = _shallow_resnet(batch=32, image=96, width=16)
        base = gpu_op.device_memory_stats(reset_peak=True)[1]
        probe = SwapExecutor(model.loss, 0.01, swap=False)
        probe.init_Variable(dict(model.variables))
        probe.run({model.X: X, model.y_: y})[0].asnumpy()
        need = gpu_op.device_memory_stats()[2] - base
        probe.close()
        del probe
        base = gpu_op.device_memory_stats()[1]
        limit = int(0.75 * need)
        gpu_op.set_device_memory_limit(base + limit)
        model, X, y = _shallow_resnet(batch=32, image=96, width=16)
        ex = SwapExecutor(model.loss, 0.01, swap=True, min_swap_bytes=1 << 16, prefetch_distance=4,
                          memory_budget=int(1.3 * limit))          # a plan that is too optimistic
        ex.init_Variable(dict(model.variables))
        got = [ex.run({model.X: X, model.y_: y})[0].asnumpy().tobytes() for _ in range(steps)]
        rep = ex.swap_report()
        assert got == want
        assert rep["passive_swap_out"] > 0 and rep["budget_reductions"] > 0
        assert rep["planned_budget_bytes"] < int(1.3 * limit)
        ex.close()
    finally:
        gpu_op.set_device_memory_limit(0)
