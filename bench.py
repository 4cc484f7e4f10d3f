"""Headline benchmark: train imgs/sec of one full training step (forward +
backward + SGD update) of ResNet-50, batch 64, fp32, on one MI355X, synthetic data.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  Next to the throughput it carries
  "roofline":     achieved vs fp32 MFMA peak for the BACKWARD contraction kernel symbol
                  (grad-data or grad-filter) that takes the most GPU time in the step,
                  measured with HIP events recorded on the compute stream around every
                  convolution launch of the timed steps;
  "roofline_fwd": the same for the dominant forward symbol;
  "roofline_bwd": all grad-data launches together and all grad-filter launches together
                  (executed flops / event time, fraction of peak, slowest symbol of each),
                  and the single op with the most time in the step;
  "hbm_kernels":  achieved GB/s against 8 TB/s for the bandwidth-bound gradient ops;
  "cpu_baseline": the CPU oracle (numpy restatement of the same step) timed on
                  this machine's host cores on a bounded sample (a smaller batch),
                  scaled linearly to images/sec; the HIP step on that same sample is
                  checked against it.
Everything here runs on one GPU; --gpus N with N > 1 is refused.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PASS_NAMES = {0: "forward", 1: "grad-data", 2: "grad-filter"}
MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0
HBM_PEAK_GBS = 8000.0


class Hip(object):
    """The few HIP runtime calls the benchmark needs for event timing."""

    def __init__(self):
        self.lib = ctypes.CDLL("libamdhip64.so")
        self.lib.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.lib.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.lib.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.lib.hipEventSynchronize.argtypes = [ctypes.c_void_p]

    def check(self, rc, what):
        if rc != 0:
            raise RuntimeError("%s failed with hipError %d" % (what, rc))

    def event(self):
        ev = ctypes.c_void_p()
        self.check(self.lib.hipEventCreate(ctypes.byref(ev)), "hipEventCreate")
        return ev

    def record(self, ev, stream):
        self.check(self.lib.hipEventRecord(ev, stream), "hipEventRecord")

    def elapsed_ms(self, e0, e1):
        ms = ctypes.c_float()
        self.check(self.lib.hipEventElapsedTime(ctypes.byref(ms), e0, e1), "hipEventElapsedTime")
        return ms.value

    def sync(self):
        self.check(self.lib.hipDeviceSynchronize(), "hipDeviceSynchronize")


def stream_handle(stream_cell):
    """hipStream_t stored in the cell that DLGpuCreatecudaStream filled."""
    return ctypes.cast(stream_cell, ctypes.POINTER(ctypes.c_void_p))[0]


def traffic_summary_path(config, batch):
    """The committed counter summary of one workload (written from two rocprofv3 --pmc runs of this script)."""
    return os.path.join(ROOT, "profiles", "%s_b%d_train_step_hbm_traffic.txt" % (config, batch))


def _normalise_symbol(name):
    """Kernel symbol with the spacing differences between profiler versions removed."""
    return name.replace(" >", ">").replace(", ", ",").strip()


def measured_traffic_bytes(config, batch):
    """{kernel symbol: HBM bytes per launch (reads + writes)} from the committed summary of
    the two rocprofv3 counter runs of this script (FETCH_SIZE, WRITE_SIZE, each scaled by
    what the same counter reads for a copy of known size; the summary states the commands
    and the factors).  One summary per workload (configuration at its own batch size, per-
    activation batch norm); a workload without one, or a symbol its summary does not list
    (a kernel changed since the counter run), reads null."""
    table = {}
    try:
        with open(traffic_summary_path(config, batch)) as fh:
            lines = fh.read().splitlines()
    except OSError:
        return table
    in_table = False
    for line in lines:
        if line.startswith("kernel") and "total MiB" in line:
            in_table = True
            continue
        if in_table:
            parts = line.rsplit(None, 4)
            if len(parts) != 5:
                if table:
                    break
                continue
            try:
                table[_normalise_symbol(parts[0])] = int(float(parts[4]) * (1 << 20))
            except ValueError:
                break
    return table


class ConvTimer(object):
    """Has the library record a HIP event pair on the compute stream around the
    contraction kernel of every convolution call (the kernel alone, without the
    layout / split-sum passes next to it) and attributes the time to the kernel
    symbol the library reports for that call."""

    def __init__(self, hip, gpu_op, lib):
        self.hip, self.gpu_op, self.lib = hip, gpu_op, lib
        self.pairs = []     # (which, kernel symbol, flops, e0, e1)
        self.pool = []
        self.enabled = False
        self._describe_cache = {}
        self._orig = {}
        for which, name in ((0, "convolution_2d_forward"), (1, "convolution_backward_data"),
                            (2, "convolution_backward_filter")):
            self._orig[name] = getattr(gpu_op, name)
            setattr(gpu_op, name, self._wrap(which, self._orig[name]))

    def _describe(self, cudnnlist, which):
        key = (ctypes.addressof(cudnnlist.contents), which)
        hit = self._describe_cache.get(key)
        if hit is None:
            buf = ctypes.create_string_buffer(256)
            flops = ctypes.c_double()
            rc = self.lib.DLGpuConvolutionDescribeKernel(cudnnlist, which, buf, 256, ctypes.byref(flops))
            if rc != 0:
                raise RuntimeError("DLGpuConvolutionDescribeKernel failed")
            variant, symbol = buf.value.decode().split(" | ")
            hit = (symbol, flops.value)
            self._describe_cache[key] = hit
        return hit

    def _event(self):
        return self.pool.pop() if self.pool else self.hip.event()

    def _wrap(self, which, fn):
        def timed(*args):
            if not self.enabled:
                return fn(*args)
            # (x, w|dy, y|w, out, cudnnlist, handle, stream) / forward: (x, w, y, cudnnlist, handle, stream)
            cudnnlist, stream = args[-3], args[-1]
            variant, flops = self._describe(cudnnlist, which)
            s = stream_handle(stream)
            e0, e1 = self._event(), self._event()
            self.lib.DLGpuConvolutionTimeNextKernel(e0, e1)
            ret = fn(*args)
            if ret:   # no room for scratch: nothing was launched, the caller makes room and calls again
                self.lib.DLGpuConvolutionTimeNextKernel(None, None)
                self.pool += [e0, e1]
            else:
                self.pairs.append((which, variant, flops, e0, e1))
            return ret
        return timed

    def pair_overhead_ms(self, stream, samples=24):
        """What an event pair adds to the kernel it brackets: a small copy kernel is
        launched `samples` times back to back inside one pair (per-launch time = the
        bulk time / samples) and then once per pair; the difference of the two
        per-launch times is subtracted from every kernel measurement."""
        from tinyflow_amd import ndarray
        src = ndarray.array(np.ones((4 << 20,), dtype=np.float32), ndarray.gpu(0))
        dst = ndarray.empty((4 << 20,), ndarray.gpu(0))
        cell = ctypes.cast(ctypes.pointer(ctypes.c_void_p(stream)), ctypes.POINTER(ctypes.c_void_p))
        launch = lambda: self.gpu_op.matrix_elementwise_multiply_by_const(src, 1.0, dst, cell)
        for _ in range(4):
            launch()
        e0, e1 = self._event(), self._event()
        self.hip.record(e0, stream)
        for _ in range(samples):
            launch()
        self.hip.record(e1, stream)
        pairs = [(self._event(), self._event()) for _ in range(samples)]
        for a, b in pairs:
            self.hip.record(a, stream)
            launch()
            self.hip.record(b, stream)
        self.hip.sync()
        bulk = self.hip.elapsed_ms(e0, e1) / samples
        single = sorted(self.hip.elapsed_ms(a, b) for a, b in pairs)[samples // 2]
        self.pool += [e0, e1] + [e for pair in pairs for e in pair]
        return max(single - bulk, 0.0)

    def collect(self, overhead_ms=0.0):
        """{(which, kernel symbol): [launches, total_ms, total_flops]} with which = 0 forward,
        1 grad-data, 2 grad-filter; call after a device sync."""
        stats = {}
        for which, variant, flops, e0, e1 in self.pairs:
            ms = max(self.hip.elapsed_ms(e0, e1) - overhead_ms, 1e-6)
            st = stats.setdefault((which, variant), [0, 0.0, 0.0])
            st[0] += 1
            st[1] += ms
            st[2] += flops
            self.pool += [e0, e1]
        self.pairs = []
        return stats


class HbmTimer(object):
    """HIP event pairs around the single-kernel, bandwidth-bound ops of a step
    (batch norm, ReLU, residual add, max-pool backward, SGD) with the algorithmic
    bytes each call moves, for the achieved-GB/s figures reported beside the
    roofline of the dominant contraction kernel."""

    def __init__(self, hip, gpu_op, pool, bn_mode):
        self.hip, self.pool = hip, pool
        self.enabled = False
        self.pairs = []
        self.streamless = None   # stream the library uses for entry points without a stream argument
        self.mask_counts = gpu_op.relu_mask_counts
        n = lambda a: int(np.prod(a.shape))
        bn_b = (8, 12) if bn_mode == "pre_activation" else (12, 20)
        table = {
            # op: bytes moved by one call, from its array arguments
            "bn_forward": lambda a: bn_b[0] * n(a[0]),
            "bn_backward": lambda a: bn_b[1] * n(a[0]),
            # a ReLU forward call that keeps its sign bits writes one more bit per element, and the
            # backward call that uses them reads dy and the bits instead of dy and x
            "activation_forward": lambda a, bits=False: (8.125 if bits else 8) * n(a[0]),
            "activation_backward": lambda a, bits=False: (8.125 if bits else 12) * n(a[0]),
            "matrix_elementwise_add": lambda a: 12 * n(a[2]),
            "pooling_2d_backward": lambda a: 4 * (n(a[0]) + n(a[1]) + n(a[2]) + n(a[3])),
            "sgd_update": lambda a: 12 * n(a[0]),
            # all updates of the step in one launch on the default stream: (tables, tables, count, lr)
            "sgd_compute_o": lambda a: 12 * int(a[2]),
        }
        for name, nbytes in table.items():
            setattr(gpu_op, name, self._wrap(name, getattr(gpu_op, name), nbytes))

    def _wrap(self, name, fn, nbytes):
        def timed(*args):
            if not self.enabled:
                return fn(*args)
            s = self.streamless if name == "sgd_compute_o" else stream_handle(args[-1])
            e0 = self.pool.pop() if self.pool else self.hip.event()
            e1 = self.pool.pop() if self.pool else self.hip.event()
            counts = self.mask_counts() if name.startswith("activation_") else None
            self.hip.record(e0, s)
            ret = fn(*args)
            self.hip.record(e1, s)
            moved = nbytes(args) if counts is None else nbytes(args, self.mask_counts() != counts)
            self.pairs.append((name, moved, e0, e1))
            return ret
        return timed

    def collect(self, overhead_ms):
        stats = {}
        for name, nbytes, e0, e1 in self.pairs:
            st = stats.setdefault(name, [0, 0.0, 0.0])
            st[0] += 1
            st[1] += max(self.hip.elapsed_ms(e0, e1) - overhead_ms, 1e-6)
            st[2] += nbytes
            self.pool += [e0, e1]
        self.pairs = []
        return [{"op": k, "launches": v[0], "avg_launch_us": v[1] / v[0] * 1e3, "bytes_per_launch": v[2] / v[0],
                 "achieved_GBps": v[2] / (v[1] * 1e-3) / 1e9, "frac_of_hbm_peak": v[2] / (v[1] * 1e-3) / 1e9 / HBM_PEAK_GBPS}
                for k, v in sorted(stats.items(), key=lambda kv: -kv[1][1])]


def cpu_baseline(bn_mode, sample_batch, image, repeats):
    """The oracle's ResNet-50 step on the host cores, on a reduced batch, timed; and the
    same reduced batch through the HIP step, whose loss and gradients are checked against
    the oracle's (the product is the thing measured, the oracle the checker)."""
    from oracle import models as OM
    from tinyflow_amd import models
    from tinyflow_amd.TrainExecute import TrainExecutor
    model, X, y = models.build("resnet50", batch=sample_batch, image=image, bn_mode=bn_mode)
    params = {v.name: val for v, val in model.variables.items()}
    net = OM.network("resnet50", bn_mode=bn_mode, image=image)
    times = []
    for _ in range(repeats + 1):
        t0 = time.perf_counter()
        loss_cpu, grads_cpu, _, _ = OM.train_step(net, params, X, y, 0.01)
        times.append(time.perf_counter() - t0)
    best = float(np.median(times[1:]))  # first call warms BLAS and the allocator
    ex = TrainExecutor(model.loss, 0.01)
    ex.init_Variable(dict(model.variables))
    loss_gpu = float(ex.run({model.X: X, model.y_: y})[0].asnumpy()[0])
    loss_cpu = float(np.asarray(loss_cpu).ravel()[0])
    if not abs(loss_gpu - loss_cpu) <= 1e-3 * abs(loss_cpu):
        raise RuntimeError("HIP step and CPU oracle disagree on the batch-%d loss: %r vs %r"
                           % (sample_batch, loss_gpu, loss_cpu))
    # the yardstick: the same step in float64.  Every gradient of the HIP step must be as close to it as the
    # fp32 CPU step is, up to a factor of three (relative L2 per tensor, + 1e-4)
    p64 = {k: v.astype(np.float64) for k, v in params.items()}
    _, grads_64, _, _ = OM.train_step(OM.network("resnet50", bn_mode=bn_mode, image=image), p64,
                                      X.astype(np.float64), y.astype(np.float64), 0.01)

    def rel(got, ref):
        ref = np.asarray(ref, dtype=np.float64).ravel()
        diff = np.asarray(got, dtype=np.float64).ravel() - ref
        return float(np.sqrt(np.dot(diff, diff)) / max(1e-30, np.sqrt(np.dot(ref, ref))))

    worst, worst_gap, worst_name, worst_ratio, failures = 0.0, 0.0, "", 0.0, []
    for var, g in zip(ex.Variable_node_list, ex.Variable_node_grad_list):
        err = rel(ex.value_of(g).asnumpy(), grads_64[var.name])
        gap = rel(grads_cpu[var.name], grads_64[var.name])
        worst_ratio = max(worst_ratio, err / max(gap, 1e-30))
        if err > worst:
            worst, worst_gap, worst_name = err, gap, var.name
        if not err <= 3 * gap + 1e-4:
            failures.append("%s: HIP %.3g, fp32 CPU %.3g" % (var.name, err, gap))
    ex.close()
    if failures:
        raise RuntimeError("HIP gradients of the batch-%d step are further from the float64 oracle than 3 x the "
                           "fp32 CPU oracle's own distance + 1e-4 (relative L2): %s" % (sample_batch, "; ".join(failures)))
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = len(os.sched_getaffinity(0))
    return {
        "value": sample_batch / best, "unit": "imgs/sec", "cores": threads, "kind": "port",
        "sample": "oracle numpy fp32 ResNet-50 step (fwd+bwd+SGD, bn_mode=%s) at batch %d, image %d; "
                  "median of %d steps after 1 warm-up, %.2f s per step; images/sec = batch / time "
                  "(os.cpu_count()=%d, affinity=%d).  Checked against the HIP step on the same batch: loss %.6f "
                  "(HIP) vs %.6f (oracle); every gradient within 3 x the fp32 oracle's own relative L2 distance from "
                  "a float64 oracle step + 1e-4 (worst: %s, HIP %.2e vs fp32 CPU %.2e from float64; largest "
                  "HIP / fp32-CPU distance ratio over the %d tensors %.2f)"
                  % (bn_mode, sample_batch, image, repeats, best, os.cpu_count(), len(os.sched_getaffinity(0)),
                     loss_gpu, loss_cpu, worst_name, worst, worst_gap, len(grads_64), worst_ratio),
        "hip_loss": loss_gpu, "oracle_loss": loss_cpu, "worst_gradient_rel_l2_from_f64": worst,
        "fp32_cpu_rel_l2_from_f64_same_tensor": worst_gap, "worst_hip_over_cpu32_distance_ratio": worst_ratio,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=None, help="default: the configuration's own batch size")
    ap.add_argument("--mem-limit-gb", type=float, default=0.0,
                    help="cap the device allocator and run the step with the swapping executor "
                         "(configuration 5: resnet152 at batch 128 under 16)")
    ap.add_argument("--bn-mode", default="pre_activation", choices=["pre_activation", "spatial"],
                    help="pre_activation is what every model graph of the reference passes")
    ap.add_argument("--config", default="resnet50", choices=["resnet50", "vgg16", "lenet5", "mlp", "resnet152"])
    ap.add_argument("--no-recompute", action="store_true",
                    help="with --mem-limit-gb: move every scheduled activation over PCIe instead of recomputing "
                         "batch-norm / ReLU outputs in the backward pass")
    ap.add_argument("--fuse-bn-relu", action="store_true",
                    help="run the timed steps with batch norm + ReLU evaluated as one kernel each way (an executor "
                         "option outside the reference's op-by-op protocol; bit-identical results).  Without the "
                         "flag the figure is still measured, on a second executor, and reported beside `value`")
    ap.add_argument("--no-fused-leg", action="store_true",
                    help="skip the extra measurement of the step with fused batch norm + ReLU (profiling runs)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-batch", type=int, default=8)
    ap.add_argument("--no-kernel-events", action="store_true",
                    help="do not record per-convolution HIP events in the timed region")
    ap.add_argument("--breakdown", action="store_true", help="print per-variant conv times to stderr")
    ap.add_argument("--event-every", type=int, default=10,
                    help="record the per-kernel HIP events in every n-th timed step only (each event pair "
                         "costs a few microseconds of queue time, which would otherwise weigh on `value`)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region launch a plain copy kernel (256 MiB read, 256 MiB written, "
                         "three times) so a counter run holds a dispatch of known traffic to scale by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)\n"
                         % args.gpus)
        sys.exit(2)

    from tinyflow_amd import gpu_op, models
    from tinyflow_amd._base import _LIB
    from tinyflow_amd.TrainExecute import TrainExecutor

    hip = Hip()
    timer = ConvTimer(hip, gpu_op, _LIB)
    hbm_timer = HbmTimer(hip, gpu_op, timer.pool, args.bn_mode)
    if args.batch is None:
        args.batch = {"mlp": 128, "lenet5": 64, "vgg16": 32, "resnet50": 64, "resnet152": 128}[args.config]
    kw = {"batch": args.batch}
    if args.config.startswith("resnet"):
        kw["bn_mode"] = args.bn_mode
    model, X, y = models.build(args.config, **kw)
    if args.mem_limit_gb > 0:
        from tinyflow_amd.SwapExecute import SwapExecutor
        limit = int(args.mem_limit_gb * (1 << 30))
        gpu_op.set_device_memory_limit(limit)
        # planned for the whole budget; a step that has to evict on demand makes the
        # executor plan for 3 % less (which the warm-up steps absorb)
        ex = SwapExecutor(model.loss, 0.01, swap=True, memory_budget=limit, prefetch_distance=12,
                          recompute=not args.no_recompute)
    else:
        ex = TrainExecutor(model.loss, 0.01, fuse_bn_relu=args.fuse_bn_relu)
    ex.init_Variable(dict(model.variables))
    feed = {model.X: X, model.y_: y}

    # The first run uploads the batch; later runs are given no feed, so the timed
    # region starts with images and labels resident in device memory.
    loss = ex.run(feed)[0]
    resident = {}
    for _ in range(max(args.warmup, 1) - 1):
        loss = ex.run(resident)[0]
    hip.sync()

    swap_before = ex.swap_report() if args.mem_limit_gb > 0 else None
    if swap_before:
        gpu_op.device_memory_stats(reset_peak=True)
    e_start, e_end = hip.event(), hip.event()
    s = stream_handle(ex.cudaStream)
    hip.sync()
    t0 = time.perf_counter()
    hip.record(e_start, s)
    event_steps = 0
    for step in range(args.steps):
        timer.enabled = (not args.no_kernel_events) and step % max(args.event_every, 1) == 0
        event_steps += timer.enabled
        loss = ex.run(resident)[0]
    hip.record(e_end, s)
    hip.sync()
    wall = time.perf_counter() - t0
    timer.enabled = False
    gpu_ms = hip.elapsed_ms(e_start, e_end)
    loss_val = float(loss.asnumpy()[0])
    swap_after = ex.swap_report() if swap_before else None
    swap_mem = gpu_op.device_memory_stats() if swap_before else None

    # Same step with the batch handed over as host (numpy) buffers every step, as a
    # data loader would: includes the PCIe upload.  Reported beside `value`, never as it.
    host_steps = max(2, min(args.steps, 5))
    hip.sync()
    t1 = time.perf_counter()
    for _ in range(host_steps):
        ex.run(feed)
    hip.sync()
    host_fed_ms = (time.perf_counter() - t1) * 1e3 / host_steps

    # Bandwidth-bound kernels: two more steps (outside the timed region, their event
    # pairs would weigh on `value`) with an event pair around each such call.
    hbm_kernels = None
    if not args.no_kernel_events:
        hbm_timer.streamless = s   # the executor's stream is the only one that runs kernels
        hbm_timer.enabled = True
        for _ in range(2):
            ex.run(resident)
        hbm_timer.enabled = False
        hip.sync()
        hbm_kernels = hbm_timer.collect(timer.pair_overhead_ms(s))

    if args.copy_calibration:
        from tinyflow_amd import ndarray
        src = ndarray.array(np.ones((64 << 20,), dtype=np.float32), ndarray.gpu(0))
        dst = ndarray.empty((64 << 20,), ndarray.gpu(0))
        for _ in range(3):
            gpu_op.matrix_elementwise_multiply_by_const(src, 1.0, dst, ex.cudaStream)
        hip.sync()

    pair_overhead = timer.pair_overhead_ms(s)
    # the executor is done: give its stream back, so that the executors created below are
    # again the only stream that runs kernels (entry points without a stream argument then
    # launch on it instead of on the default stream)
    ex.close()

    # The same step with every batch norm + ReLU pair fused, on an executor of its own.
    fused = None
    if (not args.fuse_bn_relu and not args.no_fused_leg and not args.mem_limit_gb
            and args.config.startswith("resnet") and args.bn_mode == "pre_activation"):
        model2, X2, y2 = models.build(args.config, **kw)
        ex2 = TrainExecutor(model2.loss, 0.01, fuse_bn_relu=True)
        ex2.init_Variable(dict(model2.variables))
        ex2.run({model2.X: X2, model2.y_: y2})
        for _ in range(2):
            ex2.run({})
        hip.sync()
        fused_steps = max(2, min(args.steps, 10))
        t2 = time.perf_counter()
        for _ in range(fused_steps):
            ex2.run({})
        hip.sync()
        fused_ms = (time.perf_counter() - t2) * 1e3 / fused_steps
        fused = {"ms_per_step": fused_ms, "imgs_per_sec": args.batch * 1e3 / fused_ms, "steps": fused_steps,
                 "fused_pairs": ex2.fused_pairs,
                 "note": "batch norm + ReLU pairs evaluated by the fused entry points (executor option, not the "
                         "reference's op-by-op protocol; results bit-identical)"}
        ex2.close()
        del ex2, model2

    ms_per_step = wall * 1e3 / args.steps
    imgs_per_sec = args.batch * args.steps / wall

    stats = timer.collect(pair_overhead)
    gpu_step_ms = gpu_ms / args.steps
    traffic = measured_traffic_bytes(args.config, args.batch) if args.bn_mode == "pre_activation" else {}
    RIDGE = MFMA_FP32_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBPS * 1e9)   # flop per HBM byte where the two roofs meet

    def bound_of(name, launches, total_ms, total_flops):
        """Which roof bounds a contraction symbol: with its counter traffic known, a launch that executes fewer
        flops per HBM byte than the ridge (19.7) is priced against HBM, not against the matrix pipes."""
        nbytes = traffic.get(_normalise_symbol(name))
        if not nbytes:
            return {"bound": "mfma", "traffic": None}
        intensity = total_flops / launches / nbytes
        gbps = nbytes * launches / (total_ms * 1e-3) / 1e9
        return {"bound": "hbm" if intensity < RIDGE else "mfma", "traffic": nbytes, "flop_per_hbm_byte": intensity,
                "hbm_GBps": gbps, "frac_of_hbm_peak": gbps / HBM_PEAK_GBPS}

    def symbol_roofline(which, name, launches, total_ms, total_flops):
        achieved = total_flops / (total_ms * 1e-3) / 1e12
        return {
            "bound": "mfma", "pass": PASS_NAMES[which], "kernel": name, "achieved": achieved,
            "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_FP32_PEAK_TFLOPS,
            "traffic": traffic.get(_normalise_symbol(name)),
            "against_hbm": bound_of(name, launches, total_ms, total_flops),
            "flops_per_launch": total_flops / launches,
            "launches": launches, "avg_launch_ms": total_ms / launches,
            "share_of_step": total_ms / event_steps / gpu_step_ms, "steps_with_events": event_steps,
            "event_pair_overhead_us": pair_overhead * 1e3,
        }

    def dominant(passes):
        """Contraction kernel symbol with the most event time among the given passes."""
        rows = [(k, v) for k, v in stats.items() if k[0] in passes]
        if not rows:
            return None
        (which, name), (launches, total_ms, total_flops) = max(rows, key=lambda kv: kv[1][1])
        return symbol_roofline(which, name, launches, total_ms, total_flops)

    def whole_pass(which):
        """All contraction launches of one pass together, and its slowest symbol."""
        rows = [(k[1], v) for k, v in stats.items() if k[0] == which]
        if not rows:
            return None
        ms = sum(v[1] for _, v in rows)
        flops = sum(v[2] for _, v in rows)
        slow_name, slow = min(rows, key=lambda kv: kv[1][2] / kv[1][1])
        return {
            "executed_tflops": flops / (ms * 1e-3) / 1e12, "frac": flops / (ms * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS,
            "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "ms_per_step": ms / event_steps,
            "launches_per_step": sum(v[0] for _, v in rows) / event_steps, "symbols": len(rows),
            "slowest_symbol": dict({"kernel": slow_name, "tflops": slow[2] / (slow[1] * 1e-3) / 1e12,
                                    "frac": slow[2] / (slow[1] * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS,
                                    "ms_per_step": slow[1] / event_steps, "launches_per_step": slow[0] / event_steps},
                                   **bound_of(slow_name, slow[0], slow[1], slow[2])),
        }

    # `roofline`: the backward contraction kernel (grad-data or grad-filter) with the most
    # time in the step -- the metric asks for the backward kernels; the dominant forward
    # symbol is reported beside it.
    roofline = dominant((1, 2)) if stats else None
    roofline_fwd = dominant((0,)) if stats else None
    roofline_bwd = None
    if stats:
        roofline_bwd = {"grad_data": whole_pass(1), "grad_filter": whole_pass(2), "forward": whole_pass(0),
                        "note": "flops are the ones the kernels execute (Winograd products count their own, "
                                "2.25x or 4x fewer than the direct form); time is the HIP-event time of the "
                                "contraction kernels alone, without transform and split-sum passes"}
        # the single op with the most time in the step, whatever bounds it
        conv_rows = [("%s %s" % (PASS_NAMES[k[0]], k[1]), v[1] / event_steps, "mfma",
                      v[2] / (v[1] * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS) for k, v in stats.items()]
        hbm_rows = [(h["op"], h["avg_launch_us"] * h["launches"] / 2 * 1e-3, "hbm", h["frac_of_hbm_peak"])
                    for h in (hbm_kernels or [])]   # the bandwidth-bound ops were timed over two steps
        if conv_rows or hbm_rows:
            name, ms, bound, frac = max(conv_rows + hbm_rows, key=lambda r: r[1])
            roofline_bwd["top_of_step"] = {"op": name, "ms_per_step": ms, "bound": bound, "frac_of_peak": frac,
                                           "share_of_step": ms / gpu_step_ms}
        if args.breakdown:
            conv_ms = sum(v[1] for v in stats.values()) / event_steps
            sys.stderr.write("GPU ms/step (events): %.3f, conv kernels: %.3f\n" % (gpu_step_ms, conv_ms))
            for (which, k), (n, ms, fl) in sorted(stats.items(), key=lambda kv: -kv[1][1]):
                sys.stderr.write("  %-11s %-90s launches/step %5.1f  ms/step %8.3f  TFLOP/s %7.2f\n"
                                 % (PASS_NAMES[which], k, n / event_steps, ms / event_steps, fl / (ms * 1e-3) / 1e12))

    result = {
        "metric": ("train imgs/sec ResNet-50 b64 fp32 fwd+bwd; bwd kernel % of HBM/MFMA peak"
                   if (args.config, args.batch) == ("resnet50", 64)
                   else "train imgs/sec %s b%d fp32 fwd+bwd; bwd kernel %% of HBM/MFMA peak" % (args.config, args.batch)),
        "value": imgs_per_sec, "unit": "imgs/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s batch %d fp32 3x224x224, fwd+bwd+SGD(lr 0.01), BN mode %s, "
                               "softmax-xent over %d random one-hot classes, He-normal weights"
                               % (args.config, args.batch, args.bn_mode, model.n_class)},
        "gpu_ms_per_step": gpu_ms / args.steps, "loss": loss_val,
        "host_fed": {"ms_per_step": host_fed_ms, "imgs_per_sec": args.batch * 1e3 / host_fed_ms, "steps": host_steps,
                     "note": "batch re-uploaded from pageable host memory every step (PCIe-inclusive)"},
        "roofline": roofline,
        "roofline_fwd": roofline_fwd,
        "roofline_bwd": roofline_bwd,
        "hbm_kernels": hbm_kernels,
        "fused_bn_relu": fused,
    }
    if swap_before:
        moved = {k: swap_after[k] - swap_before[k] for k in swap_after if k != "planned_budget_bytes"}
        reserved, _, peak = swap_mem
        result["swap"] = {
            "device_budget_bytes": int(args.mem_limit_gb * (1 << 30)), "peak_in_use_bytes": peak,
            "reserved_bytes": reserved,
            "offload_bytes_per_step": moved["offload_bytes"] / args.steps,
            "prefetch_bytes_per_step": (moved["prefetch_bytes"] + moved["passive_bytes"]) / args.steps,
            "offload_GBps_while_copying": moved["offload_bytes"] / max(moved["offload_seconds"], 1e-9) / 1e9,
            "prefetch_GBps_while_copying": moved["prefetch_bytes"] / max(moved["prefetch_seconds"], 1e-9) / 1e9,
            "pcie_GBps_over_step": (moved["offload_bytes"] + moved["prefetch_bytes"] + moved["passive_bytes"])
                                   / wall / 1e9,
            "passive_swap_in": moved["passive_swap_in"], "passive_swap_out": moved["passive_swap_out"],
            "recomputed_per_step": moved["recomputed"] / args.steps,
            "planned_budget_bytes": swap_after["planned_budget_bytes"],
            "budget_reductions_in_timed_steps": moved["budget_reductions"],
        }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.bn_mode, args.cpu_batch, 224, 3)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
