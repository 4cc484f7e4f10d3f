"""The column-sum entry point that allocates nothing.

DLGpuReduceSumAxisZeroNoAlloc keeps its partial sums in a device array built into
the library.  It must give the bits of DLGpuReduceSumAxisZero (same chunking, same
summation order) on consecutive calls that share that array -- the second call
here is smaller, so stale partials of the first would show -- must leave the
allocator's counters untouched, and must reject a shape whose partials do not fit.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _stats():
    import ctypes
    from tinyflow_amd._base import _LIB
    r, u, p = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    assert _LIB.DLGpuGetDeviceMemoryStats(ctypes.byref(r), ctypes.byref(u), ctypes.byref(p), 0) == 0
    return (r.value, u.value, p.value)


def test_no_alloc_column_sums_match_pool_version(rt):
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(20)
    # (rows, cols): chunked with large partials, then smaller, then a single chunk, then tiny
    shapes = [(4096, 3000), (500, 700), (64, 1000), (100000, 8), (7, 300000), (3, 5), (1, 1)]
    for shape in shapes:
        x = rng.normal(0, 1, shape).astype(np.float32)
        a = ndarray.array(x, rt.ctx)
        want = ndarray.empty((shape[1],), rt.ctx)
        got = ndarray.empty((shape[1],), rt.ctx)
        gpu_op.reduce_sum_axis_zero(a, want)
        gpu_op.array_set(got, -1.0, rt.stream)
        before = _stats()
        gpu_op.reduce_sum_axis_zero_no_alloc(a, got, rt.stream)
        after = _stats()
        assert before == after, "the entry point touched the allocator"
        w, g = want.asnumpy(), got.asnumpy()
        assert np.array_equal(w.view(np.uint32), g.view(np.uint32)), shape
        np.testing.assert_allclose(g, x.astype(np.float64).sum(axis=0), rtol=1e-4, atol=1e-3)


def test_no_alloc_1d_input(rt):
    from tinyflow_amd import gpu_op, ndarray
    x = np.random.RandomState(21).normal(0, 1, (100000,)).astype(np.float32)
    a = ndarray.array(x, rt.ctx)
    want, got = ndarray.empty((1,), rt.ctx), ndarray.empty((1,), rt.ctx)
    gpu_op.reduce_sum_axis_zero(a, want)
    gpu_op.reduce_sum_axis_zero_no_alloc(a, got, rt.stream)
    assert want.asnumpy().tobytes() == got.asnumpy().tobytes()
