"""Training-step executor with activation swapping under a device-memory budget.

Counterpart of the swap protocol of the reference's ``Executor`` and its
``MemoryManager`` thread (pycode/tinyflow/autodiff.py:31-150, 2631-2836): node
values are allocated when they are computed and released after their last use,
forward activations that backward needs again are copied to pinned host memory on
a side stream and dropped from the device, and copied back shortly before their
first backward use.  The copies go through ``DLArrayCopyFromTo`` with a stream
cell, i.e. ``hipMemcpyAsync`` on a stream of their own, ordered after the compute
stream by events inside the library; they run on worker threads (ctypes releases
the GIL for the duration of the call), so they overlap with kernel launches.

Where the reference takes its swap / release lists from the TENSILE planner
process, this executor derives a static vDNN-style schedule from the graph
itself (``plan_schedule``); the lists have the reference's shape --
``(tensor, trigger node, to_gpu)`` and ``(trigger node, tensor)``
(pycode/tinyflow/Scheduler.py:304-331) -- so a planner could supply them instead.

The device budget is enforced by the allocator behind ``DLArrayAlloc``
(environment variable ``TINYFLOW_GPU_MEM_LIMIT_MB``, read when the library
first allocates), not by this module.
"""
import queue
import threading
import time

import numpy as np

from . import autodiff as ad
from . import gpu_op, ndarray
from .TrainExecute import getcomputelist, swapsgd

GPU, HOST, MOVING_OUT, MOVING_IN, FREED = "gpu", "host", "out", "in", "freed"


class _Tensor(object):
    """Where the value of one node currently lives."""
    __slots__ = ["node", "shape", "gpu", "host", "state", "ready", "nbytes"]

    def __init__(self, node, shape):
        self.node = node
        self.shape = shape
        self.gpu = None
        self.host = None
        self.state = FREED
        self.ready = threading.Event()
        self.nbytes = 4 * int(np.prod(shape))


class MemoryManager(threading.Thread):
    """Worker that moves tensors between device and pinned host memory on its own stream."""

    def __init__(self, name, ctx):
        threading.Thread.__init__(self, name=name, daemon=True)
        self.tasks = queue.Queue()
        self.ctx = ctx
        self.cpu_ctx = ndarray.cpu(0)
        self.stream = gpu_op.create_cudaStream()
        self.bytes_moved = 0
        self.busy_seconds = 0.0
        self.alloc_seconds = 0.0   # part of busy_seconds spent waiting for device memory
        self.deferred = 0
        self.error = None
        self.progress = threading.Condition()
        self.pending = 0

    def submit(self, tensor, to_gpu, destination=None):
        """Queue a transfer.  ``destination``: device array for a prefetch, allocated by
        the caller at the moment of the request -- its storage was then released before
        the request, so the copy has to wait for nothing younger than the request."""
        tensor.ready.clear()
        tensor.state = MOVING_IN if to_gpu else MOVING_OUT
        with self.progress:
            self.pending += 1
        self.tasks.put((tensor, to_gpu, destination))

    def wait_for_progress(self, timeout):
        """Block until one more queued transfer has finished (or nothing is queued)."""
        with self.progress:
            if self.pending:
                self.progress.wait(timeout)

    def stop(self):
        self.tasks.put(None)

    def run(self):
        while True:
            task = self.tasks.get()
            if task is None:
                return
            tensor, to_gpu, destination = task
            try:
                t0 = time.perf_counter()
                if to_gpu:
                    self._swap_in(tensor, destination)
                else:
                    self._swap_out(tensor)
                self.busy_seconds += time.perf_counter() - t0
            except BaseException as e:  # surfaced by the executor thread
                self.error = e
            finally:
                tensor.ready.set()
                with self.progress:
                    self.pending -= 1
                    self.progress.notify_all()

    def _swap_out(self, tensor):
        if tensor.host is None:
            host = ndarray.empty(tensor.shape, self.cpu_ctx)  # pinned, recycled by the library's pool
            if isinstance(host, int):
                raise MemoryError("pinned host memory exhausted (%d bytes wanted)" % host)
            tensor.host = host
        tensor.gpu.copyto(tensor.host, self.stream)  # returns once the copy has completed
        gpu_arr, tensor.gpu = tensor.gpu, None
        gpu_arr.free_gpu()
        tensor.state = HOST
        self.bytes_moved += tensor.nbytes

    def _swap_in(self, tensor, destination=None):
        arr = destination
        started = time.perf_counter()
        for _ in range(20 if arr is None else 0):  # the executor thread frees memory as it advances
            arr = ndarray.empty(tensor.shape, self.ctx)
            if not isinstance(arr, int):
                break
            time.sleep(0.002)
        self.alloc_seconds += time.perf_counter() - started
        if isinstance(arr, int):
            # no room yet: leave it on the host, the executor fetches it when it needs it
            self.deferred += 1
            tensor.state = HOST
            return
        # the array is fresh: only the previous life of its storage has to be waited for,
        # so the copy runs beside whatever the compute stream has queued
        tensor.host.copy_into_fresh(arr, self.stream)
        tensor.gpu = arr
        tensor.state = GPU
        self.bytes_moved += tensor.nbytes


def plan_schedule(topo_order, forward_nodes, keep, min_bytes_of, prefetch_distance, nbytes_of=None, budget=None,
                  recomputable=None, seconds_of=None, copy_seconds_of=None, copy_slack=1.25,
                  recompute_instead=None):
    """Static schedule in the manner of vDNN, optionally with recomputation.

    ``recompute_instead(node)`` (used with a budget): forward values that are far cheaper
    to evaluate again than to move over the host link (a convolution output whose
    multiply-adds take a fraction of a millisecond against several milliseconds per
    direction).  The schedule is first planned without them; those of the tensors it
    would move that qualify, and whose inputs are kept, moved or cheaply recomputable
    values, are then recomputed instead and the rest is planned again around them (the
    way Capuchin chooses between its two mechanisms by cost).  A chain of
    recomputations holds at most one such value and five evaluations.
    """
    plan = lambda heavy: _plan_schedule(topo_order, forward_nodes, keep, min_bytes_of, prefetch_distance, nbytes_of,
                                        budget, recomputable, seconds_of, copy_seconds_of, copy_slack, heavy)
    first = plan(frozenset())
    if budget is None or recompute_instead is None:
        return first[:4]
    moved, depth = first[4], first[5]
    heavy = frozenset(n for n in moved if recompute_instead(n) and n.inputs and
                      1 + max(depth.get(i, 0) for i in n.inputs) <= 3)
    return plan(heavy)[:4] if heavy else first[:4]


def _plan_schedule(topo_order, forward_nodes, keep, min_bytes_of, prefetch_distance, nbytes_of, budget,
                   recomputable, seconds_of, copy_seconds_of, copy_slack, heavy_nodes):
    """One planning pass (see plan_schedule); ``heavy_nodes``: values recomputed although
    they are not cheap.  Also returns the moved nodes and the chain depth of every
    recomputed node.

    Returns (swap_out, swap_in, release, recompute), each a dict ``trigger index ->
    [node]``: after the node at ``trigger`` has been issued, the listed tensors are
    swapped out / prefetched / released; the tensors of ``recompute`` are evaluated
    again *before* the trigger node.  ``keep`` (variables, feeds, the loss) is never
    moved or released.

    * Every value is released after its last use.
    * ``recomputable(node)`` marks forward values that are cheap to evaluate again
      (normalisation, activation).  Such a value is released after its last forward
      use and recomputed before its first backward use, provided that this does not
      chain more than two recomputations (its inputs are swapped or kept values, or
      values recomputed directly from those).  A recomputation is an additional,
      earlier use of its inputs, which the prefetch points below take into account.
    * A forward value that backward uses again and is not recomputed is swapped out
      after its last forward use and prefetched ``prefetch_distance`` nodes before
      its first backward use.  With ``budget`` (bytes) and ``nbytes_of`` only as
      many tensors move as it takes for the simulated footprint to fit: while the
      peak of the live-bytes timeline is above the budget, the candidate spanning
      the peak with the largest bytes x absence product goes (early, large
      activations first).  Without a budget every candidate moves.
    * With ``seconds_of`` (estimated device time of a node) and ``copy_seconds_of``
      (time to bring a tensor back over the host link) the prefetch points are placed
      by time instead of by node count: the copies are laid out back to back on the
      one host-to-device engine, last needed first, so that each finishes before the
      device reaches the tensor's first backward use (each copy is given
      ``copy_slack`` times its nominal duration); ``prefetch_distance`` then only acts
      as the minimum distance.
    """
    pos = {n: i for i, n in enumerate(topo_order)}
    uses = {n: [] for n in topo_order}
    for n in topo_order:
        for inp in n.inputs:
            uses[inp].append(pos[n])
    first_backward = min((pos[n] for n in topo_order if n not in forward_nodes and n.isw not in (1, 2)),
                         default=len(topo_order))
    movable = [n for n in topo_order if n not in keep and not n.issgd]

    # which forward values are recomputed (decided in forward order: depth of the chain)
    depth, heavy = {}, {}
    if recomputable is not None:
        for n in movable:
            is_heavy = n in heavy_nodes
            if n not in forward_nodes or not (is_heavy or recomputable(n)) or not n.inputs:
                continue
            if not any(u >= first_backward for u in uses[n]) or not any(u < first_backward for u in uses[n]):
                continue
            d = 1 + max((depth.get(i, 0) for i in n.inputs), default=0)
            h = int(is_heavy) + max((heavy.get(i, 0) for i in n.inputs), default=0)
            if (h == 0 and d <= 2) or (h == 1 and d <= 5):
                depth[n], heavy[n] = d, h
    # recompute triggers, consumers first, so that the extra use of an input is known
    # when the input's own trigger is chosen
    extra = {n: [] for n in topo_order}
    recompute, recompute_at = {}, {}
    for n in reversed(movable):
        if n not in depth:
            continue
        later = [u for u in uses[n] + extra[n] if u >= first_backward]
        trigger = min(later)
        recompute_at[n] = trigger
        recompute.setdefault(trigger, []).append(n)
        for inp in n.inputs:
            extra[inp].append(trigger)
    for trigger in recompute:   # producers before consumers
        recompute[trigger].sort(key=lambda n: pos[n])

    release, last_use, candidates, first_back_use = {}, {}, [], {}
    for n in movable:
        all_uses = sorted(uses[n] + extra[n])
        last = all_uses[-1] if all_uses else pos[n]
        last_use[n] = last
        release.setdefault(last, []).append(n)
        fwd_uses = [u for u in all_uses if u < first_backward]
        bwd_uses = [u for u in all_uses if u >= first_backward]
        if n in depth:
            release.setdefault(fwd_uses[-1], []).append(n)
            continue
        if n not in forward_nodes or not min_bytes_of(n) or not bwd_uses:
            continue
        out_at = fwd_uses[-1] if fwd_uses else pos[n]
        in_at = max(bwd_uses[0] - prefetch_distance, first_backward - 1, out_at + 1)
        if in_at >= bwd_uses[0] or bwd_uses[0] - out_at < 2 * prefetch_distance:
            continue  # needed again too soon for a round trip to pay
        candidates.append((n, out_at, in_at))
        first_back_use[n] = bwd_uses[0]
    timed = seconds_of is not None and copy_seconds_of is not None
    if timed:
        # device time at which each node starts, if nothing ever stalls
        clock = np.concatenate([[0.0], np.cumsum([seconds_of(n) for n in topo_order])])
        earliest = {n: max(first_backward - 1, out_at + 1) for n, out_at, _ in candidates}

        def by_time(cands, serial):
            """Prefetch points by time; ``serial``: the copies share one engine."""
            points, engine_free = {}, float("inf")
            for n, out_at, in_at in sorted(cands, key=lambda c: first_back_use[c[0]], reverse=True):
                finish = min(clock[first_back_use[n]], engine_free if serial else float("inf"))
                start = finish - copy_slack * copy_seconds_of(n)
                # a link that cannot keep up is not helped by asking ever earlier: the lead
                # over the tensor's use stays within eight of its own copy times
                start = max(start, clock[first_back_use[n]] - 8.0 * copy_slack * copy_seconds_of(n))
                if serial:
                    engine_free = start
                at = int(np.searchsorted(clock, start, side="right")) - 2   # last node that ends before `start`
                points[n] = max(min(at, in_at), earliest[n])
            return [(n, out_at, points[n]) for n, out_at, _ in cands]
        candidates = by_time(candidates, serial=False)
    if budget is not None:
        absent = {n: (max(u for u in uses[n] if u < first_backward), recompute_at[n]) for n in depth}
        fit = lambda cands, forced: _fit_budget(cands, pos, last_use, absent, nbytes_of,
                                                sum(nbytes_of(n) for n in keep), budget, len(topo_order),
                                                prefetch_distance, forced)
        chosen = fit(candidates, [])
        if timed:
            # the chosen copies queue behind each other, which moves some prefetch points
            # forward and keeps those tensors resident longer: fit again around them
            for _ in range(4):
                serial = by_time(chosen, serial=True)
                names = {c[0] for c in serial}
                again = fit([c for c in candidates if c[0] not in names], serial)
                chosen = again
                if {c[0] for c in again} == names:
                    break
            chosen = by_time(chosen, serial=True)
        candidates = chosen
    elif timed:
        candidates = by_time(candidates, serial=True)
    swap_out, swap_in = {}, {}
    for n, out_at, in_at in candidates:
        swap_out.setdefault(out_at, []).append(n)
        swap_in.setdefault(in_at, []).append(n)
    return swap_out, swap_in, release, recompute, [c[0] for c in candidates], depth


def _fit_budget(candidates, pos, last_use, absent, nbytes_of, persistent, budget, steps, lag, forced=()):
    """``forced`` plus the smallest greedy subset of ``candidates`` whose removal brings
    the simulated footprint under ``budget``.  A swapped-out block is counted as
    resident until ``lag`` nodes after its trigger (its copy has to finish first);
    ``absent`` maps a recomputed value to the (release, recompute) indices between
    which it is gone."""
    live = np.zeros(steps + 1, dtype=np.int64)
    for n, born in pos.items():
        if n in last_use:
            live[born] += nbytes_of(n)
            live[last_use[n] + 1] -= nbytes_of(n)
    live = np.cumsum(live)[:steps] + persistent
    for n, (gone, back) in absent.items():
        live[gone + 1:back] -= nbytes_of(n)
    chosen, remaining = list(forced), list(candidates)
    for c in forced:
        live[c[1] + lag + 1:c[2]] -= nbytes_of(c[0])
    while remaining:
        peak = int(np.argmax(live))
        if live[peak] <= budget:
            break
        spanning = [c for c in remaining if c[1] + lag < peak < c[2]]
        if not spanning:
            break
        best = max(spanning, key=lambda c: nbytes_of(c[0]) * (c[2] - c[1]))
        remaining.remove(best)
        chosen.append(best)
        live[best[1] + lag + 1:best[2]] -= nbytes_of(best[0])
    return sorted(chosen, key=lambda c: pos[c[0]])


def schedule_to_wire(swap_out, swap_in, release):
    """The three dicts of ``plan_schedule`` in the planner's wire format
    (pycode/tinyflow/Scheduler.py:304-331): a swap list of
    ``[tensor_id, wait_ms, trigger_node_id, to_gpu, 1]`` in issue order and a release
    list of ``(trigger_node_id, tensor_id)``; ids are positions in the topological order.
    Takes positions, i.e. dicts ``trigger index -> [tensor index]``."""
    swaps = []
    for trigger in sorted(set(swap_out) | set(swap_in)):
        swaps += [[t, 0, trigger, 0, 1] for t in swap_out.get(trigger, ())]
        swaps += [[t, 0, trigger, 1, 1] for t in swap_in.get(trigger, ())]
    releases = [(trigger, t) for trigger in sorted(release) for t in release[trigger]]
    return swaps, releases


def schedule_from_wire(swap_list, release_list, recompute_list=()):
    """Inverse of ``schedule_to_wire``, also accepting the recomputation list
    ``(trigger_node_id, tensor_id[, release_flag])``: returns
    (swap_out, swap_in, release, recompute) as dicts ``trigger index -> [tensor index]``,
    each list in the order the planner gave.  ``wait_ms`` (the pacing delay the
    reference's memory thread sleeps, pycode/tinyflow/autodiff.py:90-139) is not
    used: copies here are ordered by stream events, not by time."""
    swap_out, swap_in, release, recompute = {}, {}, {}, {}
    for msg in swap_list:
        tensor_id, trigger, to_gpu = int(msg[0]), int(msg[2]), int(msg[3])
        (swap_in if to_gpu else swap_out).setdefault(trigger, []).append(tensor_id)
    for msg in release_list:
        release.setdefault(int(msg[0]), []).append(int(msg[1]))
    for msg in recompute_list:
        recompute.setdefault(int(msg[0]), []).append(int(msg[1]))
    return swap_out, swap_in, release, recompute


def planner_message(topo_order, shapes, loss, runtimes=None):
    """What the executor reports to the planner before it asks for a schedule
    (pycode/tinyflow/autodiff.py:2473-2510): one entry per node, in topological order,
    ``[tensor_list, input_ids, op_name, op_id, is_input_or_output, [], runtime]`` with
    ``tensor_list = [(tensor_id, nbytes, shape)]``.  Ids are positions in the
    topological order.  An in-place update node owns no tensor of its own: it lists
    the tensors it rewrites (parameter; for Adam also the two moments) under
    ``id + len(topo_order)``, as the reference does for its Adam nodes.  The flag is 1
    for parameters and for the loss.  ``runtimes`` maps a node to seconds; nodes it
    does not cover get the reference's placeholder of 1e-8 s (1e-5 ms)."""
    pos = {n: i for i, n in enumerate(topo_order)}
    total = len(topo_order)
    runtimes = runtimes or {}
    message = []
    for node in topo_order:
        if node.issgd:
            rewritten = node.inputs[:3] if isinstance(node.op, ad.AdamOp) else node.inputs[:1]
            tensors = [(pos[i] + total, 4 * int(np.prod(shapes[i])), tuple(shapes[i])) for i in rewritten]
        else:
            tensors = [(pos[node], 4 * int(np.prod(shapes[node])), tuple(shapes[node]))]
        flag = 1 if (node.isw == 1 or node is loss) else 0
        message.append([tensors, [pos[i] for i in node.inputs], node.name, pos[node], flag, [],
                        float(runtimes.get(node, 1e-8))])
    return message


class SwapExecutor(object):
    """SGD step executor that keeps the device footprint small by releasing dead
    values and swapping forward activations to pinned host memory."""

    def __init__(self, targetloss, learning_rate, ctx=ndarray.gpu(0), swap=True, min_swap_bytes=1 << 20,
                 prefetch_distance=8, memory_budget=None, recompute=False, optimizer="sgd"):
        """``optimizer``: "sgd" (one ``sgd_op`` per variable, as ``TrainExecute``) or "adam"
        (one ``adam_op`` and two zero-initialised moment variables per variable with the
        bias-correction powers advanced after every step -- the optimizer of the
        reference's swap-capable executor, pycode/tinyflow/autodiff.py:2250-2272, 2843-2845)."""
        self.targetloss = targetloss
        self.ctx = ctx
        self.Variable_node_list = ad.get_Variable_node_list(targetloss)
        self.Variable_node_list.reverse()
        self.Variable_node_grad_list = ad.gradients(targetloss, self.Variable_node_list)
        assert optimizer in ("sgd", "adam"), optimizer
        self.optimizer = optimizer
        self.Variable_node_to_mv = {}
        if optimizer == "adam":
            from . import TrainExecuteAdam as _adam
            self.b1, self.b2, self.e = 0.9, 0.999, 0.00000001
            self.b1t, self.b2t = [0.9], [0.999]
            eval_nodes, self.mv, self.Variable_node_to_mv = _adam.getcomputelist(
                self.Variable_node_list, self.Variable_node_grad_list, self.b1, self.b2, self.b1t, self.b2t,
                self.e, learning_rate)
        else:
            eval_nodes = getcomputelist(self.Variable_node_list, self.Variable_node_grad_list, learning_rate)
        self.topo_order = swapsgd(ad.find_topo_sort(eval_nodes))
        self.forward_nodes = set(ad.find_topo_sort([targetloss]))
        self.swap = swap
        self.min_swap_bytes = min_swap_bytes
        self.prefetch_distance = prefetch_distance
        self.memory_budget = memory_budget   # bytes the schedule plans for; None: move every candidate
        self.recompute = recompute           # evaluate normalisation / activation outputs again instead of moving them
        # with ``recompute``: also evaluate again, rather than move, the convolution outputs that the budget
        # would send over the host link and that cost the device far less than the link (see plan_schedule)
        self.recompute_convolutions = True
        self.cudaStream = gpu_op.create_cudaStream()
        self.cudnnHandle = gpu_op.create_cudnnHandle(self.cudaStream)
        self.cublasHandle = gpu_op.create_cublasHandle(self.cudaStream)
        self.Variable_node_np_value = None
        self.tensors = None
        self.keep_values = set()   # extra nodes whose values must survive the step (for inspection)
        self.offloader = MemoryManager("tinyflow-offload", ctx)
        self.prefetcher = MemoryManager("tinyflow-prefetch", ctx)
        self.offloader.start()
        self.prefetcher.start()
        self.stats = {}
        self.wire_schedule = None
        # rate assumed for host <-> device copies when placing prefetches by time
        # (None / 0: by node count only); PCIe 5 x16 moves ~55 GB/s in practice
        self.host_link_bytes_per_second = 50e9
        self.prefetch_slack = 1.25   # each prefetch is planned with this multiple of its nominal copy time
        self.adapt_budget = True     # lower the planned budget when a step had to evict on demand
        self._evictions_seen = 0
        self.measure_runtimes = False   # time every node of the next steps (waits for the device around each)
        self.node_runtime = {}          # node -> seconds, filled while measure_runtimes is set
        self._sync_cell = None

    def _device_sync(self):
        """Wait until everything enqueued so far has run (a synchronous one-element read)."""
        if self._sync_cell is None:
            self._sync_cell = ndarray.array(np.zeros(1, np.float32), ctx=self.ctx)
        self._sync_cell.asnumpy()

    def _idle_sync_seconds(self):
        """Cost of ``_device_sync`` on an idle device, subtracted from measured runtimes."""
        self._device_sync()
        best = 1.0
        for _ in range(5):
            started = time.perf_counter()
            self._device_sync()
            best = min(best, time.perf_counter() - started)
        return best

    def planner_message(self, runtimes=None):
        """The per-node report a planner builds its schedule from (see the module-level
        ``planner_message``); call after the first step, when shapes are known.  Uses
        the runtimes measured under ``measure_runtimes`` unless others are given."""
        assert self.tensors is not None, "run one step first: shapes are inferred there"
        shapes = {n: t.shape for n, t in self.tensors.items()}
        return planner_message(self.topo_order, shapes, self.targetloss,
                               self.node_runtime if runtimes is None else runtimes)

    def set_schedule(self, swap_list, release_list, recompute_list=()):
        """Run the steps from a planner's lists (the wire format described at
        ``schedule_from_wire``) instead of the built-in static schedule.  Swaps and
        releases take effect after their trigger node has been issued, recomputations
        before it (pycode/tinyflow/autodiff.py:2675-2708, 2814-2835)."""
        n = len(self.topo_order)
        sched = schedule_from_wire(swap_list, release_list, recompute_list)
        for table in sched:
            for trigger, ids in table.items():
                assert 0 <= trigger < n and all(0 <= i < n for i in ids), "node id outside the graph"
        self.wire_schedule = sched
        self.tensors = None   # re-plan on the next run

    def init_Variable(self, feed_dict):
        values = dict(feed_dict)
        for node, (m, v) in self.Variable_node_to_mv.items():   # Adam moments start at zero
            values[m] = np.zeros(np.shape(feed_dict[node]), dtype=np.float32)
            values[v] = np.zeros(np.shape(feed_dict[node]), dtype=np.float32)
        self.Variable_node_np_value = values

    def close(self):
        """Stops the two copy workers and gives their streams, the compute stream and
        the handles back to the library.  Arrays already returned stay valid."""
        if self.cudaStream is None:
            return
        for worker in (self.offloader, self.prefetcher):
            worker.stop()
        for worker in (self.offloader, self.prefetcher):
            worker.join(30.0)
            if not worker.is_alive():
                gpu_op.destroy_cudaStream(worker.stream)
        stream, self.cudaStream = self.cudaStream, None
        gpu_op.destroy_cudnnHandle(self.cudnnHandle)
        gpu_op.destroy_cublasHandle(self.cublasHandle)
        gpu_op.destroy_cudaStream(stream)

    def __del__(self):
        try:
            self.close()
        except Exception:   # interpreter shutdown: the library may already be gone
            pass

    # ------------------------------------------------------------------ set-up

    def _prepare(self, feed_dict):
        shapes = {node: tuple(np.shape(v)) for node, v in feed_dict.items()}
        for node in self.topo_order:
            if node not in shapes:
                shapes[node] = tuple(node.op.infer_shape(node, [shapes[i] for i in node.inputs], self.cudnnHandle))
        self.tensors = {node: _Tensor(node, shapes[node]) for node in self.topo_order}
        self.keep = set(n for n in self.topo_order if n.isw in (1, 2)) | {self.targetloss} | self.keep_values
        self._plan()
        keep = self.keep
        pos = {n: i for i, n in enumerate(self.topo_order)}
        self.uses = {n: [] for n in self.topo_order}
        for n in self.topo_order:
            for inp in n.inputs:
                self.uses[inp].append(pos[n])
        self.evictable = [n for n in self.topo_order
                          if self.swap and n not in keep and not n.issgd and self.uses[n]]
        self.cursor = 0

    def replan(self):
        """Builds the schedule again, e.g. after a step run with ``measure_runtimes`` so
        that the prefetch points use measured node times instead of the estimate."""
        assert self.tensors is not None, "run one step first: shapes are inferred there"
        self._plan()

    def _plan(self):
        """(Re)builds the swap / release / recomputation tables for the current budget."""
        keep = self.keep
        big = lambda n: self.swap and self.tensors[n].nbytes >= self.min_swap_bytes
        self.recompute_at = {}
        if self.wire_schedule is not None:
            by_node = [{t: [self.topo_order[i] for i in ids if self.topo_order[i] not in keep]
                        for t, ids in table.items()} for table in self.wire_schedule]
            self.swap_out_at, self.swap_in_at, self.release_at, self.recompute_at = by_node
            return
        cheap = (ad.BNForwardOp, ad.ActivationForwardOp, ad.ReluOp)
        again = (lambda n: isinstance(n.op, cheap)) if (self.swap and self.recompute) else None
        timing = {}
        if self.host_link_bytes_per_second:
            # measured node times when a measured step has been run, else the estimate
            seconds_of = (lambda n: self.node_runtime.get(n, 0.0)) if self.node_runtime \
                else self._estimate_seconds
            timing = dict(seconds_of=seconds_of, copy_slack=self.prefetch_slack,
                          copy_seconds_of=lambda n: self.tensors[n].nbytes / self.host_link_bytes_per_second)
            if again is not None and self.recompute_convolutions:
                # a convolution output is recomputed rather than moved when that costs the
                # device less than an eighth of what the round trip costs the link
                timing["recompute_instead"] = lambda n: (
                    isinstance(n.op, ad.Convolution2DForwardOp) and
                    8.0 * self._estimate_seconds(n) < 2.0 * self.tensors[n].nbytes / self.host_link_bytes_per_second)
        self.swap_out_at, self.swap_in_at, self.release_at, self.recompute_at = plan_schedule(
            self.topo_order, self.forward_nodes, keep, big, self.prefetch_distance,
            nbytes_of=lambda n: self.tensors[n].nbytes, budget=self.memory_budget, recomputable=again,
            **timing)

    def _estimate_seconds(self, node):
        """Rough device time of a node for placing prefetches: a launch, the bytes the
        node touches at 6 TB/s, and for a convolution or matrix product its
        multiply-adds at 100 TFLOP/s (200 for the 3x3 / stride-1 layers, which run in a
        Winograd form).  These are the rates of the fast end of what the kernels reach:
        an estimate that is too short puts a prefetch early, which only holds its
        storage a little longer, while one that is too long lets the device wait for
        the copy."""
        if node.isw in (1, 2):
            return 0.0
        moved = self.tensors[node].nbytes + sum(self.tensors[i].nbytes for i in node.inputs)
        seconds = 5e-6 + moved / 6.0e12
        flops, rate = 0.0, 100e12
        if isinstance(node.op, (ad.Convolution2DForwardOp, ad.Convolution2DBackwardOp)):
            x, w = self.tensors[node.inputs[0]].shape, self.tensors[node.inputs[1]].shape
            y = self.tensors[node].shape if isinstance(node.op, ad.Convolution2DForwardOp) \
                else self.tensors[node.inputs[2]].shape
            flops = 2.0 * np.prod(y, dtype=np.float64) * w[1] * w[2] * w[3]
            if w[2] == 3 and w[3] == 3 and getattr(node, "u", 1) == 1 and getattr(node, "v", 1) == 1:
                rate = 200e12
        elif isinstance(node.op, ad.MatMulOp):
            a = self.tensors[node.inputs[0]].shape
            flops = 2.0 * np.prod(self.tensors[node].shape, dtype=np.float64) * (a[0] if node.matmul_attr_trans_A
                                                                                 else a[1])
        return seconds + flops / rate

    def _alloc(self, shape, what, protect=()):
        """Device array of ``shape``.  When the budget is exhausted: first wait for
        queued swap-outs (each frees its block when its copy completes), then evict
        the resident forward value whose next use is farthest away (a passive
        swap-out, pycode/tinyflow/autodiff.py:2741-2766 in the reference)."""
        deadline = time.perf_counter() + 120.0
        while True:
            arr = ndarray.empty(shape, self.ctx)
            if not isinstance(arr, int):
                return arr
            self._check_workers()
            if time.perf_counter() > deadline:
                break
            if self.offloader.pending or self.prefetcher.pending:
                waited = time.perf_counter()
                # wait on a worker that has something queued: the other one returns at once
                (self.offloader if self.offloader.pending else self.prefetcher).wait_for_progress(0.05)
                self.stats["alloc_wait_seconds"] = (self.stats.get("alloc_wait_seconds", 0.0)
                                                    + time.perf_counter() - waited)
                continue
            victim = self._pick_victim(protect)
            if victim is None:
                break
            self.stats["passive_swap_out"] = self.stats.get("passive_swap_out", 0) + 1
            self.offloader.submit(victim, False)
        raise MemoryError("device budget exhausted allocating %s for %s" % (shape, what))

    def _pick_victim(self, protect):
        best, best_next = None, -1
        for node in self.evictable:
            t = self.tensors[node]
            if t.state != GPU or node in protect:
                continue
            nxt = next((u for u in self.uses[node] if u >= self.cursor), None)
            if nxt is None or nxt == self.cursor:
                continue
            if nxt > best_next:
                best, best_next = t, nxt
        return best

    def _check_workers(self):
        for w in (self.offloader, self.prefetcher):
            if w.error is not None:
                raise w.error

    def _on_gpu(self, tensor, protect=()):
        """Device array of a tensor, fetching it back first if it was swapped out."""
        if tensor.state in (MOVING_OUT, MOVING_IN):
            waited = time.perf_counter()
            tensor.ready.wait()
            self.stats["transfer_wait_seconds"] = (self.stats.get("transfer_wait_seconds", 0.0)
                                                   + time.perf_counter() - waited)
            self._check_workers()
        if tensor.state == FREED and tensor.node.inputs and tensor.node.isw not in (1, 2):
            self._recompute(tensor.node, self._handles)   # released and not brought back: recompute
        if tensor.state == HOST:   # not prefetched in time: passive swap-in on the compute stream
            self.stats["passive_swap_in"] = self.stats.get("passive_swap_in", 0) + 1
            arr = self._alloc(tensor.shape, tensor.node.name, protect)
            tensor.host.copyto(arr, self.cudaStream)
            tensor.gpu, tensor.state = arr, GPU
            self.stats["passive_bytes"] = self.stats.get("passive_bytes", 0) + tensor.nbytes
        assert tensor.state == GPU, "%s is %s" % (tensor.node.name, tensor.state)
        return tensor.gpu

    # --------------------------------------------------------------------- step

    def run(self, feed_dict, convert_to_numpy_ret_vals=False):
        """One step; returns [loss, variables in network order]."""
        if self.tensors is None:
            first = dict(feed_dict)
            first.update(self.Variable_node_np_value or {})
            self._prepare(first)
            feed_dict = first
        for node, value in feed_dict.items():
            t = self.tensors[node]
            if node.isw == 1 and t.state == GPU:
                continue   # variables stay on the device between steps
            if t.gpu is None:
                t.gpu = ndarray.array(value, ctx=self.ctx)
                if isinstance(t.gpu, int):
                    raise MemoryError("device budget exhausted feeding %s" % node.name)
                t.state = GPU
            else:
                t.gpu._sync_copyfrom(value)
        handles = self._handles = (self.cudnnHandle, self.cublasHandle, self.cudaStream)
        sync_cost = self._idle_sync_seconds() if self.measure_runtimes else 0.0
        for t in self.tensors.values():
            if t.state == HOST and t.node not in self.keep:
                t.state = FREED   # last step's host copy is stale
        for idx, node in enumerate(self.topo_order):
            t = self.tensors[node]
            if node.isw in (1, 2):
                pass
            else:
                self.cursor = idx
                for again in self.recompute_at.get(idx, ()):
                    self._recompute(again, handles)
                input_vals = [self._on_gpu(self.tensors[i], node.inputs) for i in node.inputs]
                out = None
                if not node.issgd:
                    out = self._alloc(t.shape, node.name, node.inputs)
                if self.measure_runtimes:
                    self._device_sync()
                    started = time.perf_counter()
                wanted = node.op.compute(node, input_vals, out, *handles)
                if self.measure_runtimes:
                    self._device_sync()
                    self.node_runtime[node] = max(1e-8, time.perf_counter() - started - sync_cost)
                for _ in range(3):
                    if not wanted:
                        break
                    # the op found no room for its scratch: make room, hand the block
                    # back to the allocator's cache and run the op again
                    self._alloc(((int(wanted) + 3) // 4,), node.name + " scratch", node.inputs).free_gpu()
                    wanted = node.op.compute(node, input_vals, out, *handles)
                if wanted:
                    raise MemoryError("%s: %d bytes of device scratch could not be allocated" % (node.name, wanted))
                if out is not None:
                    t.gpu, t.state = out, GPU
            for n in self.swap_out_at.get(idx, ()):
                if self.tensors[n].state == GPU:
                    self.offloader.submit(self.tensors[n], False)
            for n in self.swap_in_at.get(idx, ()):
                tn = self.tensors[n]
                if tn.state == MOVING_OUT:
                    tn.ready.wait()
                if tn.state == HOST:
                    room = ndarray.empty(tn.shape, self.ctx)
                    if isinstance(room, int):
                        room = None   # no room now: the worker asks again later
                    else:
                        room.prepare_fresh()
                    self.prefetcher.submit(tn, True, room)
            for n in self.release_at.get(idx, ()):
                self._release(self.tensors[n])
        self._check_workers()
        self._adapt_budget()
        if self.optimizer == "adam":
            self.b1t[0] = self.b1t[0] * self.b1
            self.b2t[0] = self.b2t[0] * self.b2
        result = [self._on_gpu(self.tensors[self.targetloss])]
        result += [self.tensors[v].gpu for v in reversed(self.Variable_node_list)]
        if convert_to_numpy_ret_vals:
            return [r.asnumpy() for r in result]
        return result

    def _adapt_budget(self):
        """The schedule is planned for ``memory_budget``; what the plan does not model
        (scratch of the operators, fragmentation) can make a step that fits on paper
        evict on demand.  A step that had to do so lowers the planned budget by 3 % and
        plans again, at most ten times; steps that fit leave the plan alone."""
        evictions = self.stats.get("passive_swap_out", 0) + self.stats.get("passive_swap_in", 0)
        happened = evictions > self._evictions_seen
        self._evictions_seen = evictions
        if (happened and self.adapt_budget and self.memory_budget and self.wire_schedule is None
                and self.stats.get("budget_reductions", 0) < 10):
            self.memory_budget = int(self.memory_budget * 0.97)
            self.stats["budget_reductions"] = self.stats.get("budget_reductions", 0) + 1
            self._plan()

    def _recompute(self, node, handles):
        """Evaluate ``node`` again from its inputs (a planner released its value and
        asked for it back by recomputation rather than by a swap-in)."""
        t = self.tensors[node]
        if t.state == GPU:
            return
        input_vals = [self._on_gpu(self.tensors[i], node.inputs) for i in node.inputs]
        out = self._alloc(t.shape, node.name + " (recompute)", node.inputs)
        wanted = node.op.compute(node, input_vals, out, *handles)
        for _ in range(3):
            if not wanted:
                break
            # no room for the op's scratch (a convolution): make room and run it again
            self._alloc(((int(wanted) + 3) // 4,), node.name + " scratch", node.inputs).free_gpu()
            wanted = node.op.compute(node, input_vals, out, *handles)
        if wanted:
            raise MemoryError("%s: %d bytes of device scratch could not be allocated" % (node.name, wanted))
        t.gpu, t.state = out, GPU
        self.stats["recomputed"] = self.stats.get("recomputed", 0) + 1

    def _release(self, tensor):
        if tensor.state in (MOVING_OUT, MOVING_IN):
            tensor.ready.wait()
        if tensor.state == HOST:
            return   # the device copy is gone already; the host copy stays valid for this step
        if tensor.gpu is not None:
            # stream-ordered: kernels already enqueued keep reading the block safely,
            # and whoever receives it next is enqueued behind them
            gpu_arr, tensor.gpu = tensor.gpu, None
            gpu_arr.free_gpu()
        tensor.state = FREED

    def value_of(self, node):
        """Device array holding ``node`` after a step (list the node in ``keep_values`` first)."""
        return self._on_gpu(self.tensors[node])

    def swap_report(self):
        """Bytes moved and busy time of the two copy workers since construction."""
        return {"offload_bytes": self.offloader.bytes_moved, "offload_seconds": self.offloader.busy_seconds,
                "prefetch_bytes": self.prefetcher.bytes_moved, "prefetch_seconds": self.prefetcher.busy_seconds,
                "prefetch_alloc_seconds": self.prefetcher.alloc_seconds,
                "passive_swap_in": self.stats.get("passive_swap_in", 0),
                "passive_swap_out": self.stats.get("passive_swap_out", 0),
                "passive_bytes": self.stats.get("passive_bytes", 0),
                "prefetch_deferred": self.prefetcher.deferred, "recomputed": self.stats.get("recomputed", 0),
                # host time the step spent blocked: on memory (waiting for offloads to free
                # blocks) and on operands whose transfer had not finished
                "planned_budget_bytes": self.memory_budget, "budget_reductions": self.stats.get("budget_reductions", 0),
                "alloc_wait_seconds": self.stats.get("alloc_wait_seconds", 0.0),
                "transfer_wait_seconds": self.stats.get("transfer_wait_seconds", 0.0)}
