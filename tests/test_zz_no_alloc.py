"""The column-sum entry point that allocates nothing.

DLGpuReduceSumAxisZeroNoAlloc keeps its partial sums in a device array built into
the library.  It must give the bits of DLGpuReduceSumAxisZero (same chunking, same
summation order) on consecutive calls that share that array -- the second call
here is smaller, so stale partials of the first would show -- must leave the
pool allocator's counters untouched (the test reads the pool's statistics; the
source has no other allocating call), and must refuse, launching nothing, a shape
whose partials do not fit the 1.5 MiB area.  The rule that decides this is host
arithmetic and is swept on the CPU in tests/test_host_logic.py.
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


def test_no_alloc_refuses_partials_beyond_the_builtin_area(rt):
    """Two chunks of 200 000 columns are 1.6 MB of partial sums: refused with -1, output
    untouched; the pool version of the same shape works, and so does the no-alloc one on
    a shape of the same width that runs as a single chunk (8 rows: nothing to split)."""
    import ctypes
    from tinyflow_amd import gpu_op, ndarray
    from tinyflow_amd._base import _LIB
    rows, cols = 64, 200000
    wanted, limit = ctypes.c_int64(), ctypes.c_int64()
    assert _LIB.DLGpuReduceSumAxisZeroNoAllocBytes(ctypes.c_int64(rows), ctypes.c_int64(cols), 0,
                                                   ctypes.byref(wanted), ctypes.byref(limit)) == 0
    assert wanted.value == 2 * cols * 4 > limit.value == 3 << 19
    x = np.random.RandomState(22).normal(0, 1, (rows, cols)).astype(np.float32)
    a = ndarray.array(x, rt.ctx)
    got = ndarray.empty((cols,), rt.ctx)
    gpu_op.array_set(got, -3.0, rt.stream)
    with pytest.raises(RuntimeError):
        gpu_op.reduce_sum_axis_zero_no_alloc(a, got, rt.stream)
    assert np.all(got.asnumpy() == -3.0)
    want = ndarray.empty((cols,), rt.ctx)
    gpu_op.reduce_sum_axis_zero(a, want)
    np.testing.assert_allclose(want.asnumpy(), x.astype(np.float64).sum(axis=0), rtol=1e-4, atol=1e-4)
    few = ndarray.array(x[:8], rt.ctx)
    gpu_op.reduce_sum_axis_zero(few, want)
    gpu_op.reduce_sum_axis_zero_no_alloc(few, got, rt.stream)
    assert want.asnumpy().tobytes() == got.asnumpy().tobytes()
