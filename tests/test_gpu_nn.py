"""GPU parity of pooling, activation and batch-norm entry points against the oracle.

Bit-exact: max-pool forward values, max-pool routing (which input receives each
dy, checked with distinct dy values and with tied inputs), ReLU masks.
fp32 within rtol 1e-3 / atol 1e-5: batch-norm reductions, softmax, mean pooling.
"""
import numpy as np
import pytest

from oracle import ops as O
import parity

pytestmark = pytest.mark.gpu


def _gpu(a, rt):
    from tinyflow_amd import ndarray
    return ndarray.array(np.asarray(a, dtype=np.float32), rt.ctx)


# (shape, mode, pad_h, pad_w, u, v, fh, fw)
POOL_CASES = [
    ((64, 6, 28, 28), "max", 0, 0, 2, 2, 2, 2),     # LeNet
    ((64, 16, 10, 10), "max", 0, 0, 2, 2, 2, 2),
    ((4, 64, 112, 112), "max", 1, 1, 2, 2, 3, 3),   # ResNet stem pool (pad 1)
    ((4, 64, 112, 112), "max", 0, 0, 2, 2, 3, 3),   # the reference graph's pad 0 variant
    ((8, 2048, 7, 7), "mean", 0, 0, 1, 1, 7, 7),    # global average pool
    ((3, 5, 4, 6), "mean", 0, 0, 1, 1, 4, 6),       # global, 15 planes of 24 values
    ((300, 3, 6, 6), "mean", 0, 0, 2, 2, 6, 6),     # global whatever the stride; several workgroups
    ((3, 5, 13, 9), "max", 1, 0, 2, 1, 3, 2),
    ((3, 5, 13, 9), "mean", 1, 1, 2, 2, 3, 3),
    ((2, 3, 8, 8), "max", 0, 0, 1, 1, 1, 1),
    ((2, 3, 11, 13), "max", 1, 1, 2, 2, 3, 3),      # odd extents: stride cells hang over the border
    ((2, 3, 11, 13), "max", 0, 0, 3, 3, 3, 3),      # stride 3: per-element backward path
    ((2, 3, 9, 10), "max", 1, 1, 1, 2, 3, 3),
    ((2, 3, 9, 10), "max", 2, 2, 2, 1, 5, 4),
    ((16, 64, 112, 112), "max", 1, 1, 2, 2, 3, 3),  # stem pool at full spatial size
    ((2, 3, 70, 130), "max", 0, 0, 2, 2, 2, 2),     # several tiles per plane, ragged last tile
    ((2, 3, 33, 67), "max", 1, 1, 2, 2, 3, 3),
    # planes too large to stage whole in LDS: the 16 x 64 tile kernel, ragged last tiles
    ((2, 2, 150, 130), "max", 0, 0, 2, 2, 2, 2),      # unpadded 2x2: bands of 50 rows go through the plane kernels
    ((2, 3, 224, 224), "max", 0, 0, 2, 2, 2, 2),      # VGG-16's first pool: bands of 56 rows
    ((1, 2, 146, 130), "max", 0, 0, 2, 2, 2, 2),      # 146 = 2 x 73: no even band divides it, the tile kernel
    ((1, 2, 140, 134), "max", 1, 1, 2, 2, 3, 3),
    # windows too large for the one-pass tile kernel: the two-pass kernels
    ((2, 3, 40, 80), "max", 4, 4, 1, 1, 9, 9),      # stride 1: cell kernel
    ((2, 3, 40, 90), "max", 0, 0, 3, 3, 15, 15),    # stride 3: per-element kernel
]


@pytest.mark.parametrize("case", POOL_CASES, ids=lambda c: "-".join(str(v) for v in c))
@pytest.mark.parametrize("ties", [False, True])
def test_pooling(rt, case, ties):
    from tinyflow_amd import gpu_op, ndarray
    shape, mode, ph, pw, u, v, fh, fw = case
    rng = np.random.RandomState(21)
    x = rng.normal(0, 1, shape).astype(np.float32)
    if ties:  # post-ReLU style input: many exact zeros and repeated values
        x = np.maximum(np.round(x * 2) / 2, 0).astype(np.float32)
    out_shape, lst = gpu_op.pooling_2d_forward_get_out_shape(shape, "NCHW", mode, ph, pw, u, v, fh, fw)
    assert out_shape[2] == O.pool_out_extent(shape[2], fh, ph, u)
    assert out_shape[3] == O.pool_out_extent(shape[3], fw, pw, v)
    # distinct upstream values identify where each one is routed
    dy = (rng.permutation(int(np.prod(out_shape))).reshape(out_shape) + 1).astype(np.float32)
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx = ndarray.empty(out_shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    gpu_op.pooling_2d_forward(gx, gy, lst, rt.cudnn, rt.stream)
    gpu_op.pooling_2d_backward(gx, gy, gdy, gdx, lst, rt.cudnn, rt.stream)
    if mode == "max":
        np.testing.assert_array_equal(gy.asnumpy(), O.max_pool_forward(x, fh, fw, ph, pw, u, v))
        dx_ref = O.max_pool_backward(x.astype(np.float64), dy.astype(np.float64), fh, fw, ph, pw, u, v)
        if u >= fh and v >= fw:   # disjoint windows: every dx is a single dy -> exact
            np.testing.assert_array_equal(gdx.asnumpy(), dx_ref.astype(np.float32))
        else:                     # overlapping windows: sums of a few dy
            np.testing.assert_allclose(gdx.asnumpy(), dx_ref, rtol=1e-6)
        np.testing.assert_allclose(gdx.asnumpy().astype(np.float64).sum(), dy.astype(np.float64).sum(), rtol=1e-6)
    else:
        np.testing.assert_allclose(gy.asnumpy(), O.avg_pool_forward(x.astype(np.float64), fh, fw, ph, pw, u, v),
                                   rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(gdx.asnumpy(),
                                   O.avg_pool_backward(shape, dy.astype(np.float64), fh, fw, ph, pw, u, v),
                                   rtol=1e-5)


def test_max_pool_routing_is_first_maximum(rt):
    """All-equal window: the gradient goes to the first position in row-major order."""
    from tinyflow_amd import gpu_op, ndarray
    x = np.zeros((1, 1, 4, 4), np.float32)
    out_shape, lst = gpu_op.pooling_2d_forward_get_out_shape(x.shape, "NCHW", "max", 0, 0, 2, 2, 2, 2)
    dy = np.arange(1, 5, dtype=np.float32).reshape(out_shape)
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx = ndarray.empty(out_shape, rt.ctx), ndarray.empty(x.shape, rt.ctx)
    gpu_op.pooling_2d_forward(gx, gy, lst, rt.cudnn, rt.stream)
    gpu_op.pooling_2d_backward(gx, gy, gdy, gdx, lst, rt.cudnn, rt.stream)
    expect = np.zeros((4, 4), np.float32)
    expect[0, 0], expect[0, 2], expect[2, 0], expect[2, 2] = 1, 2, 3, 4
    np.testing.assert_array_equal(gdx.asnumpy()[0, 0], expect)


@pytest.mark.parametrize("case", [((4, 8, 28, 28), 1, 1, 2, 2, 3, 3), ((2, 3, 40, 80), 4, 4, 1, 1, 9, 9),
                                  ((2, 3, 40, 90), 0, 0, 3, 3, 15, 15)],
                         ids=["one-pass", "large-window-stride1", "large-window-stride3"])
def test_max_pool_backward_without_scratch_memory(rt, case):
    """With no device memory left for the arg-max scratch the backward pass still
    runs (the entry point cannot report out-of-memory) and gives the same bits."""
    from tinyflow_amd import gpu_op, ndarray
    shape, ph, pw, u, v, fh, fw = case
    rng = np.random.RandomState(23)
    x = np.maximum(np.round(rng.normal(0, 1, shape) * 2) / 2, 0).astype(np.float32)
    out_shape, lst = gpu_op.pooling_2d_forward_get_out_shape(shape, "NCHW", "max", ph, pw, u, v, fh, fw)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx, gdx2 = ndarray.empty(out_shape, rt.ctx), ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    gpu_op.pooling_2d_forward(gx, gy, lst, rt.cudnn, rt.stream)
    gpu_op.pooling_2d_backward(gx, gy, gdy, gdx, lst, rt.cudnn, rt.stream)
    _, in_use, _ = gpu_op.device_memory_stats()
    gpu_op.set_device_memory_limit(max(in_use, 1))   # nothing more can be allocated
    try:
        assert isinstance(ndarray.empty((1 << 20,), rt.ctx), int)   # the budget really is exhausted
        gpu_op.pooling_2d_backward(gx, gy, gdy, gdx2, lst, rt.cudnn, rt.stream)
        got = gdx2.asnumpy()
    finally:
        gpu_op.set_device_memory_limit(0)
    np.testing.assert_array_equal(got, gdx.asnumpy())


@pytest.mark.parametrize("mode", ["pre_activation", "spatial"])
def test_batch_norm_reports_all_the_scratch_it_needs(rt, mode):
    """The out-of-memory convention: a call that finds no room writes the bytes it wants
    and returns 0; a caller that then makes exactly that much room must be able to repeat
    the call.  Forward needs two statistics blocks (and spatial mode a partial-sum block
    on top): with room for one and a half of them the report has to cover all of them."""
    from tinyflow_amd import gpu_op, ndarray
    shape = (4, 64, 32, 32) if mode == "pre_activation" else (4, 131072, 2, 2)
    stats = int(np.prod(shape[1:])) if mode == "pre_activation" else shape[1]
    block = 4 * stats                                   # 256 KiB / 512 KiB: a multiple of the allocator's rounding
    x = np.random.RandomState(5).normal(0, 1, shape).astype(np.float32)
    gx, gy = _gpu(x, rt), ndarray.empty(shape, rt.ctx)
    mean_p, var_p, lst = gpu_op.bn_get_cudnnlist(shape, "NCHW", mode)
    in_use = gpu_op.device_memory_stats()[1]
    gpu_op.set_device_memory_limit(in_use + block + block // 2)
    try:
        wanted = gpu_op.bn_forward(gx, gy, mode, 0, mean_p, var_p, lst, rt.cudnn, rt.stream)
        assert wanted >= 2 * block, "only %d bytes reported for two blocks of %d" % (wanted, block)
        gpu_op.set_device_memory_limit(0)
        gpu_op.set_device_memory_limit(in_use + wanted)
        assert gpu_op.bn_forward(gx, gy, mode, 0, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
        y_ref = O.batch_norm_forward(x.astype(np.float64), mode)[0]
        np.testing.assert_allclose(gy.asnumpy(), y_ref, rtol=1e-3, atol=2e-5)
    finally:
        gpu_op.set_device_memory_limit(0)
    # backward consumes (and releases) the statistics of the repeated call
    dy = np.random.RandomState(6).normal(0, 1, shape).astype(np.float32)
    gdx = ndarray.empty(shape, rt.ctx)
    assert gpu_op.bn_backward(gx, _gpu(dy, rt), gdx, mode, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    _, mean, istd = O.batch_norm_forward(x.astype(np.float64), mode)
    dx_ref = O.batch_norm_backward(x.astype(np.float64), dy.astype(np.float64), mode, mean, istd)
    np.testing.assert_allclose(gdx.asnumpy(), dx_ref, rtol=1e-3, atol=2e-5 * max(1.0, float(np.abs(dx_ref).max())))


@pytest.mark.parametrize("shape", [(64, 256, 14, 14), (3, 5, 7, 9), (128, 100), (7, 1, 33)])
@pytest.mark.parametrize("mode", ["relu", "sigmoid", "tanh", "softmax"])
def test_activation(rt, shape, mode):
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(22)
    x = rng.normal(0, 2, shape).astype(np.float32)
    x.flat[::5] = 0.0
    dy = rng.normal(0, 1, shape).astype(np.float32)
    lst = gpu_op.activation_get_cudnnlist(shape, "NCHW", mode)
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    gpu_op.activation_forward(gx, gy, mode, lst, rt.cudnn, rt.stream)
    gpu_op.activation_backward(gx, gdx, gy, gdy, mode, lst, rt.cudnn, rt.stream)
    y_ref = O.activation_forward(x.astype(np.float64), mode)
    dx_ref = O.activation_backward(x.astype(np.float64), y_ref, dy.astype(np.float64), mode)
    if mode == "relu":
        np.testing.assert_array_equal(gy.asnumpy(), y_ref.astype(np.float32))
        np.testing.assert_array_equal(gdx.asnumpy(), dx_ref.astype(np.float32))
        assert np.all(gdx.asnumpy().flat[::5] == 0)   # mask is x > 0
    elif mode == "softmax" and int(np.prod(shape[1:])) > 4096:
        # an instance of 50 176 elements (no model has one, the library takes it): probabilities of 1e-6 ... 1e-3,
        # so the absolute terms are scaled to the largest value; sums of 50 176 fp32 terms: rtol 1e-4 / 1e-3
        np.testing.assert_allclose(gy.asnumpy(), y_ref, rtol=1e-4, atol=1e-6 * float(y_ref.max()))
        np.testing.assert_allclose(gdx.asnumpy(), dx_ref, rtol=1e-3, atol=1e-5 * float(np.abs(dx_ref).max()))
        np.testing.assert_allclose(gy.asnumpy().astype(np.float64).reshape(shape[0], -1).sum(axis=1), 1.0, rtol=1e-5)
    else:
        np.testing.assert_allclose(gy.asnumpy(), y_ref, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(gdx.asnumpy(), dx_ref, rtol=1e-4, atol=1e-6)


BN_SHAPES = [(64, 64, 28, 28), (32, 16, 7, 9), (5, 3, 4, 4), (128, 8, 6, 6), (200, 4, 3, 3), (2, 2048, 7, 7),
             (65, 5, 9, 7), (100, 64, 14, 14), (128, 256, 14, 14),   # 64 < N <= 128: the 128-row form, ragged and full
             (64, 1, 100), (3, 5, 1, 1), (1, 1300, 2, 2), (7, 300, 5, 5),
             (64, 256, 56, 56)]   # the last one: the largest ResNet-50 b64 activation


K_BN = 3.0


@pytest.mark.parametrize("shape", BN_SHAPES, ids=str)
@pytest.mark.parametrize("mode", ["pre_activation", "spatial"])
def test_batch_norm(rt, shape, mode):
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(23)
    x = (rng.normal(0, 1, shape) * rng.uniform(0.5, 3, (1,) + shape[1:]) + rng.normal(0, 2, (1,) + shape[1:]))
    x = x.astype(np.float32)
    dy = rng.normal(0, 1, shape).astype(np.float32)
    mean_p, var_p, lst = gpu_op.bn_get_cudnnlist(shape, "NCHW", mode)
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    assert gpu_op.bn_forward(gx, gy, mode, 0, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.bn_backward(gx, gdy, gdx, mode, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    y_ref, mean, istd = O.batch_norm_forward(x64, mode)
    dx_ref = O.batch_norm_backward(x64, dy64, mode, mean, istd)
    np.testing.assert_allclose(gy.asnumpy(), y_ref, rtol=1e-3, atol=2e-5)
    scale = max(1.0, float(np.abs(dx_ref).max()))
    np.testing.assert_allclose(gdx.asnumpy(), dx_ref, rtol=1e-3, atol=2e-5 * scale)
    # against what a numpy fp32 executor gives on the same inputs: the HIP error may be
    # at most K_BN times the float32 oracle's own distance from the float64 one
    y32, mean32, istd32 = O.batch_norm_forward(x, mode)
    dx32 = O.batch_norm_backward(x, dy, mode, mean32, istd32)
    assert y32.dtype == dx32.dtype == np.float32
    parity.compare(gy.asnumpy(), y_ref, y32, "batch norm forward, %s" % mode, "bn fwd %s %s" % (shape, mode), K_BN)
    parity.compare(gdx.asnumpy(), dx_ref, dx32, "batch norm backward, %s" % mode, "bn bwd %s %s" % (shape, mode), K_BN)
    # invariants of the batch-norm gradient per statistic group:
    #   sum(dx) = 0 and sum(dx * xhat) = istd/m * sum(dy*xhat) * (m - sum(xhat^2))
    # (the second is 0 only in the limit eps -> 0, because sum(xhat^2) = m*var/(var+eps))
    axes = (0,) if mode == "pre_activation" else (0,) + tuple(range(2, len(shape)))
    dx = gdx.asnumpy().astype(np.float64)
    xhat = (x64 - mean) * istd
    m = np.prod([shape[a] for a in axes])
    bound = 1e-4 * m * np.abs(dx).max() + 1e-6
    assert np.abs(dx.sum(axis=axes)).max() <= bound
    expect = (istd / m * (dy64 * xhat).sum(axis=axes, keepdims=True)
              * (m - (xhat * xhat).sum(axis=axes, keepdims=True)))
    assert np.abs((dx * xhat).sum(axis=axes, keepdims=True) - expect).max() <= 10 * bound
    # a second backward without a forward is refused (statistics were consumed)
    with pytest.raises(RuntimeError):
        gpu_op.bn_backward(gx, gdy, gdx, mode, mean_p, var_p, lst, rt.cudnn, rt.stream)


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["pre_activation", "spatial"])
def test_batch_norm_with_mean_far_from_zero(rt, mode):
    """Statistics whose mean is a thousand standard deviations from zero (mean about
    100, std about 0.1): a variance computed as E[x^2] - mean^2 in fp32 would be lost to
    cancellation.  Forward and backward against the float64 oracle; the fp32 CPU oracle
    (two-pass variance) is the yardstick for the error."""
    from tinyflow_amd import gpu_op, ndarray
    shape = (32, 24, 14, 14)
    rng = np.random.RandomState(29)
    offset = rng.choice([-1.0, 1.0], (1,) + shape[1:]) * rng.uniform(80, 120, (1,) + shape[1:])
    x = (offset + rng.normal(0, 1, shape) * rng.uniform(0.05, 0.2, (1,) + shape[1:])).astype(np.float32)
    dy = rng.normal(0, 1, shape).astype(np.float32)
    mean_p, var_p, lst = gpu_op.bn_get_cudnnlist(shape, "NCHW", mode)
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    assert gpu_op.bn_forward(gx, gy, mode, 0, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.bn_backward(gx, gdy, gdx, mode, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    x64, dy64 = x.astype(np.float64), dy.astype(np.float64)
    y_ref, mean, istd = O.batch_norm_forward(x64, mode)
    dx_ref = O.batch_norm_backward(x64, dy64, mode, mean, istd)
    y32, mean32, istd32 = O.batch_norm_forward(x, mode)
    dx32 = O.batch_norm_backward(x, dy, mode, mean32, istd32)
    # x itself carries 100 * 2^-24 = 6e-6 of rounding against a spread of 0.1: the
    # normalised values are only defined to about 1e-4, whoever computes them
    np.testing.assert_allclose(gy.asnumpy(), y_ref, rtol=1e-3, atol=2e-3)
    np.testing.assert_allclose(gdx.asnumpy(), dx_ref, rtol=1e-3, atol=2e-3 * float(np.abs(dx_ref).max()))
    parity.compare(gy.asnumpy(), y_ref, y32, "batch norm forward, %s, |mean| >> std" % mode, "bn fwd offset", K_BN)
    parity.compare(gdx.asnumpy(), dx_ref, dx32, "batch norm backward, %s, |mean| >> std" % mode, "bn bwd offset", K_BN)


@pytest.mark.gpu
@pytest.mark.parametrize("rows", [5, 33, 65, 100])
def test_batch_norm_with_fewer_rows_than_its_registers_writes_only_its_rows(rt, rows):
    """The per-activation kernels hold 32, 64 or 128 rows and leave the rows a batch does not
    have to the bounds check of their buffer descriptors.  The arrays handed over here are the
    first `rows` rows of larger allocations filled with a sentinel: after forward and backward
    the rows behind the batch must still hold it (a store that escaped the check would land
    exactly there), and the batch's own rows must equal a run on arrays of their own."""
    import ctypes
    from tinyflow_amd import gpu_op, ndarray
    L, slack, sentinel = 3 * 5 * 7, 128, -7.5
    rng = np.random.RandomState(24)
    x = rng.normal(0, 1, (rows, 3, 5, 7)).astype(np.float32)
    dy = rng.normal(0, 1, (rows, 3, 5, 7)).astype(np.float32)

    def view(big, values=None):
        """NDArray over the first `rows` rows of `big` (not an owner: never freed through the library)."""
        if values is not None:
            host = np.full((rows + slack, L), sentinel, np.float32)
            host[:rows] = values.reshape(rows, L)
            big._sync_copyfrom(host)
        shape = (ctypes.c_int64 * 4)(rows, 3, 5, 7)
        arr = ndarray.DLArray(big.handle.contents.data, rt.ctx, 4, shape)
        v = ndarray.NDArray(ctypes.pointer(arr))
        v.is_freed = True            # the storage belongs to `big`
        return v, (arr, shape)

    bigs = [ndarray.empty((rows + slack, L), rt.ctx) for _ in range(4)]
    (vx, k0), (vdy, k1) = view(bigs[0], x), view(bigs[1], dy)
    (vy, k2), (vdx, k3) = view(bigs[2], np.zeros_like(x)), view(bigs[3], np.zeros_like(x))
    mp, vp, lst = gpu_op.bn_get_cudnnlist(x.shape, "NCHW", "pre_activation")
    assert gpu_op.bn_forward(vx, vy, "pre_activation", 0, mp, vp, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.bn_backward(vx, vdy, vdx, "pre_activation", mp, vp, lst, rt.cudnn, rt.stream) == 0
    got_y, got_dx = bigs[2].asnumpy(), bigs[3].asnumpy()
    assert np.all(got_y[rows:] == sentinel) and np.all(got_dx[rows:] == sentinel)
    assert np.all(bigs[0].asnumpy()[rows:] == sentinel) and np.all(bigs[1].asnumpy()[rows:] == sentinel)
    # the same call on arrays of their own
    gx, gdy = _gpu(x, rt), _gpu(dy, rt)
    gy, gdx = ndarray.empty(x.shape, rt.ctx), ndarray.empty(x.shape, rt.ctx)
    mp2, vp2, lst2 = gpu_op.bn_get_cudnnlist(x.shape, "NCHW", "pre_activation")
    gpu_op.bn_forward(gx, gy, "pre_activation", 0, mp2, vp2, lst2, rt.cudnn, rt.stream)
    gpu_op.bn_backward(gx, gdy, gdx, "pre_activation", mp2, vp2, lst2, rt.cudnn, rt.stream)
    assert got_y[:rows].tobytes() == gy.asnumpy().tobytes()
    assert got_dx[:rows].tobytes() == gdx.asnumpy().tobytes()
    y_ref = O.batch_norm_forward(x.astype(np.float64), "pre_activation")[0]
    np.testing.assert_allclose(got_y[:rows].reshape(x.shape), y_ref, rtol=1e-3, atol=2e-5)
    del k0, k1, k2, k3


# ------------------------------------------------------- dropout, concatenation

@pytest.mark.gpu
@pytest.mark.parametrize("shape,p,seed", [((64, 1000), 0.5, 3), ((8, 3, 17, 19), 0.25, 0), ((5,), 0.9, 100),
                                          ((32, 64, 28, 28), 0.1, 42), ((7, 1, 13), 0.0, 9)])
def test_dropout_matches_oracle_bit_for_bit(rt, shape, p, seed):
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(1)
    x = rng.normal(0, 1, shape).astype(np.float32)
    dy = rng.normal(0, 1, shape).astype(np.float32)
    want, keep = O.dropout_forward(x, p, seed)
    inputd = gpu_op.get_input_descriptor(shape, "NCHW")
    dev_x, dev_dy = ndarray.array(x, rt.ctx), ndarray.array(dy, rt.ctx)
    out, dx = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    reserve, cudnnlist, wanted = gpu_op.dropout_forward(dev_x, out, "NCHW", p, seed, inputd, rt.cudnn, rt.stream)
    assert wanted == 0
    assert out.asnumpy().tobytes() == want.tobytes()
    gpu_op.dropout_backward(dev_dy, dx, reserve, cudnnlist, rt.cudnn, rt.stream)
    assert dx.asnumpy().tobytes() == O.dropout_backward(dy, keep, p).tobytes()


@pytest.mark.gpu
def test_dropout_backward_needs_its_forward(rt):
    from tinyflow_amd import gpu_op, ndarray
    x = ndarray.array(np.ones((4, 8), np.float32), rt.ctx)
    out = ndarray.empty((4, 8), rt.ctx)
    inputd = gpu_op.get_input_descriptor((4, 8), "NCHW")
    reserve, cudnnlist, _ = gpu_op.dropout_forward(x, out, "NCHW", 0.5, 1, inputd, rt.cudnn, rt.stream)
    gpu_op.dropout_backward(x, out, reserve, cudnnlist, rt.cudnn, rt.stream)
    with pytest.raises(RuntimeError):   # the list was consumed
        gpu_op.dropout_backward(x, out, reserve, cudnnlist, rt.cudnn, rt.stream)


@pytest.mark.gpu
def test_dropout_forward_twice_releases_the_first_mask(rt):
    """A forward whose backward never runs (an evaluation pass) must not leak its mask:
    the next forward through the same input descriptor releases it, and a backward on
    the discarded cells is refused."""
    from tinyflow_amd import gpu_op, ndarray
    shape = (64, 4096)
    x = ndarray.array(np.ones(shape, np.float32), rt.ctx)
    out = ndarray.empty(shape, rt.ctx)
    inputd = gpu_op.get_input_descriptor(shape, "NCHW")
    first = gpu_op.dropout_forward(x, out, "NCHW", 0.5, 1, inputd, rt.cudnn, rt.stream)
    in_use = gpu_op.device_memory_stats()[1]
    for seed in range(2, 12):
        last = gpu_op.dropout_forward(x, out, "NCHW", 0.5, seed, inputd, rt.cudnn, rt.stream)
    assert gpu_op.device_memory_stats()[1] == in_use    # ten more forwards hold one mask, not eleven
    with pytest.raises(RuntimeError):
        gpu_op.dropout_backward(x, out, first[0], first[1], rt.cudnn, rt.stream)
    gpu_op.dropout_backward(x, out, last[0], last[1], rt.cudnn, rt.stream)
    assert gpu_op.device_memory_stats()[1] < in_use


@pytest.mark.gpu
@pytest.mark.parametrize("sa,sb", [((3, 2, 4, 5), (3, 7, 4, 5)), ((64, 256, 28, 28), (64, 64, 28, 28)),
                                   ((4, 10), (4, 1)), ((1, 1, 1), (1, 3, 1))])
def test_concat_forward_and_backward(rt, sa, sb):
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(2)
    a, b = rng.normal(0, 1, sa).astype(np.float32), rng.normal(0, 1, sb).astype(np.float32)
    want = O.concat_forward(a, b)
    da_, db_ = ndarray.array(a, rt.ctx), ndarray.array(b, rt.ctx)
    out = ndarray.empty(want.shape, rt.ctx)
    gpu_op.concat_forward(da_, db_, out, rt.stream)
    assert out.asnumpy().tobytes() == want.tobytes()
    dout = rng.normal(0, 1, want.shape).astype(np.float32)
    wa, wb = O.concat_backward(a, b, dout)
    dev_dout = ndarray.array(dout, rt.ctx)
    ga, gb = ndarray.empty(sa, rt.ctx), ndarray.empty(sb, rt.ctx)
    gpu_op.concat_a_backward(da_, db_, dev_dout, ga, rt.stream)
    gpu_op.concat_b_backward(da_, db_, dev_dout, gb, rt.stream)
    assert ga.asnumpy().tobytes() == wa.tobytes() and gb.asnumpy().tobytes() == wb.tobytes()


@pytest.mark.gpu
def test_dropout_and_concat_in_a_graph(rt):
    """y = concat(dropout(x W1), x W2); loss = sum(y * t): gradients through the
    graph equal the oracle's, with the seed the op drew."""
    import random
    from tinyflow_amd import autodiff as ad
    from tinyflow_amd.TrainExecute import TrainExecutor
    rng = np.random.RandomState(6)
    X = rng.normal(0, 1, (16, 12)).astype(np.float32)
    T = rng.normal(0, 1, (16, 9)).astype(np.float32)
    W1v, W2v = rng.normal(0, 1, (12, 5)).astype(np.float32), rng.normal(0, 1, (12, 4)).astype(np.float32)
    x, t = ad.Placeholder("x"), ad.Placeholder("t")
    W1, W2 = ad.Variable("W1"), ad.Variable("W2")
    h1 = ad.fullydropout_forward_op(ad.matmul_op(x, W1), "NCHW", 0.4)
    y = ad.concat_forward_op(h1, ad.matmul_op(x, W2))
    # scalar loss through the ops that exist on the path: sum over rows then columns
    loss = ad.reducesumaxiszero_op(ad.reducesumaxiszero_op(ad.mul_op(y, t)))
    ex = TrainExecutor(loss, 0.0)
    ex.init_Variable({W1: W1v, W2: W2v})
    random.seed(123)
    ex.run({x: X, t: T})
    seed = h1.seed[0]
    grads = {v: ex.value_of(g).asnumpy() for v, g in zip(ex.Variable_node_list, ex.Variable_node_grad_list)}
    a1 = X @ W1v
    _, keep = O.dropout_forward(a1, 0.4, seed)
    dy1, dy2 = O.concat_backward(a1, X @ W2v, T)
    da1 = O.dropout_backward(dy1, keep, 0.4)
    np.testing.assert_allclose(grads[W1], X.T @ da1, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(grads[W2], X.T @ dy2, rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
def test_relu_masks_at_full_activation_size(rt):
    """ReLU forward / backward on the largest ResNet-50 batch-64 activation
    (64 x 256 x 56 x 56, 205 MB), through both entry-point families: bit-exact."""
    from tinyflow_amd import gpu_op, ndarray
    gen = np.random.default_rng(5)
    shape = (64, 256, 56, 56)
    x = gen.standard_normal(shape, dtype=np.float32)
    x.reshape(-1)[::7] = 0.0          # exact zeros: the mask is x > 0
    dy = gen.standard_normal(shape, dtype=np.float32)
    want_y, want_dx = O.relu(x), O.relu_gradient(x, dy)
    gx, gdy = ndarray.array(x, rt.ctx), ndarray.array(dy, rt.ctx)
    gy, gdx = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    gpu_op.relu(gx, gy)
    gpu_op.relu_gradient(gx, gdy, gdx)
    assert gy.asnumpy().tobytes() == want_y.tobytes() and gdx.asnumpy().tobytes() == want_dx.tobytes()
    lst = gpu_op.activation_get_cudnnlist(shape, "NCHW", "relu")
    gpu_op.array_set(gy, np.nan, rt.stream)
    gpu_op.array_set(gdx, np.nan, rt.stream)
    gpu_op.activation_forward(gx, gy, "relu", lst, rt.cudnn, rt.stream)
    gpu_op.activation_backward(gx, gdx, gy, gdy, "relu", lst, rt.cudnn, rt.stream)
    assert gy.asnumpy().tobytes() == want_y.tobytes() and gdx.asnumpy().tobytes() == want_dx.tobytes()


def _relu_mask_counts():
    from tinyflow_amd import gpu_op
    return gpu_op.relu_mask_counts()


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(8, 64, 56, 56), (3, 7, 60, 56), (1, 1, 256, 257), (64, 256, 56, 56)], ids=str)
def test_relu_backward_from_kept_sign_bits_is_bit_identical(rt, shape):
    """From a descriptor's second step on, the ReLU forward call keeps one bit per element
    and the backward call reads dy and the bits instead of dy and x.  Same bytes as the
    oracle and as the first step (which read x), also with exact zeros, negative zeros,
    a ragged last workgroup, and different data in each step."""
    from tinyflow_amd import gpu_op, ndarray
    gen = np.random.default_rng(17)
    lst = gpu_op.activation_get_cudnnlist(shape, "NCHW", "relu")
    gy, gdx = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    for step in range(3):
        x = gen.standard_normal(shape, dtype=np.float32)
        x.reshape(-1)[::7] = 0.0
        x.reshape(-1)[3::11] = -0.0
        dy = gen.standard_normal(shape, dtype=np.float32)
        gx, gdy = ndarray.array(x, rt.ctx), ndarray.array(dy, rt.ctx)
        gpu_op.array_set(gy, np.nan, rt.stream)
        gpu_op.array_set(gdx, np.nan, rt.stream)
        kept0, used0 = _relu_mask_counts()
        gpu_op.activation_forward(gx, gy, "relu", lst, rt.cudnn, rt.stream)
        gpu_op.activation_backward(gx, gdx, gy, gdy, "relu", lst, rt.cudnn, rt.stream)
        kept1, used1 = _relu_mask_counts()
        assert (kept1 - kept0, used1 - used0) == ((0, 0) if step == 0 else (1, 1)), step
        assert gy.asnumpy().tobytes() == O.relu(x).tobytes(), step
        assert gdx.asnumpy().tobytes() == O.relu_gradient(x, dy).tobytes(), step


@pytest.mark.gpu
def test_kept_relu_sign_bits_follow_the_input_array(rt):
    """The kept bits describe x as the forward call read it.  A backward call must not use
    them once x was overwritten, when it is given another array, under a device-memory
    budget, for an array too small or of a length that is no multiple of four, or when
    the forward call ran in place; each time it reads x and gives the oracle's bytes."""
    from tinyflow_amd import gpu_op, ndarray
    gen = np.random.default_rng(19)
    shape = (4, 32, 28, 28)

    def fresh(shape):
        x = gen.standard_normal(shape, dtype=np.float32)
        dy = gen.standard_normal(shape, dtype=np.float32)
        return x, dy, ndarray.array(x, rt.ctx), ndarray.array(dy, rt.ctx)

    def backward(lst, gx, gy, gdy, shape):
        gdx = ndarray.empty(shape, rt.ctx)
        gpu_op.array_set(gdx, np.nan, rt.stream)
        gpu_op.activation_backward(gx, gdx, gy, gdy, "relu", lst, rt.cudnn, rt.stream)
        return gdx.asnumpy()

    lst = gpu_op.activation_get_cudnnlist(shape, "NCHW", "relu")
    gy = ndarray.empty(shape, rt.ctx)
    x, dy, gx, gdy = fresh(shape)
    gpu_op.activation_forward(gx, gy, "relu", lst, rt.cudnn, rt.stream)
    assert backward(lst, gx, gy, gdy, shape).tobytes() == O.relu_gradient(x, dy).tobytes()   # the descriptor has now seen a backward call

    # x overwritten between the two calls
    kept0, used0 = _relu_mask_counts()
    gpu_op.activation_forward(gx, gy, "relu", lst, rt.cudnn, rt.stream)
    x2 = -x
    gx[:] = x2
    assert backward(lst, gx, gy, gdy, shape).tobytes() == O.relu_gradient(x2, dy).tobytes()
    assert _relu_mask_counts() == (kept0 + 1, used0)

    # another array of the same shape given to the backward call
    gpu_op.activation_forward(gx, gy, "relu", lst, rt.cudnn, rt.stream)
    x3, _, gx3, _ = fresh(shape)
    assert backward(lst, gx3, gy, gdy, shape).tobytes() == O.relu_gradient(x3, dy).tobytes()
    assert _relu_mask_counts() == (kept0 + 2, used0)
    # the bits stay with the array they describe, untouched since: its own backward call uses them
    assert backward(lst, gx, gy, gdy, shape).tobytes() == O.relu_gradient(x2, dy).tobytes()
    assert _relu_mask_counts() == (kept0 + 2, used0 + 1)

    # the bits of an array whose storage was released and handed out again are gone
    gpu_op.activation_forward(gx, gy, "relu", lst, rt.cudnn, rt.stream)
    del gx
    x4, _, gx4, _ = fresh(shape)
    assert backward(lst, gx4, gy, gdy, shape).tobytes() == O.relu_gradient(x4, dy).tobytes()
    assert _relu_mask_counts() == (kept0 + 3, used0 + 1)

    # under a device-memory budget nothing is kept
    kept0, used0 = _relu_mask_counts()
    in_use = gpu_op.device_memory_stats()[1]
    gpu_op.set_device_memory_limit(in_use + (1 << 30))
    try:
        gpu_op.activation_forward(gx4, gy, "relu", lst, rt.cudnn, rt.stream)
        assert backward(lst, gx4, gy, gdy, shape).tobytes() == O.relu_gradient(x4, dy).tobytes()
    finally:
        gpu_op.set_device_memory_limit(0)
    assert _relu_mask_counts() == (kept0, used0)

    # small arrays and lengths that are no multiple of four take the plain kernels
    for small in [(2, 3, 5, 5), (1, 1, 257, 257)]:
        slst = gpu_op.activation_get_cudnnlist(small, "NCHW", "relu")
        sy = ndarray.empty(small, rt.ctx)
        for _ in range(2):
            xs, dys, gxs, gdys = fresh(small)
            gpu_op.activation_forward(gxs, sy, "relu", slst, rt.cudnn, rt.stream)
            assert sy.asnumpy().tobytes() == O.relu(xs).tobytes()
            assert backward(slst, gxs, sy, gdys, small).tobytes() == O.relu_gradient(xs, dys).tobytes()
    assert _relu_mask_counts() == (kept0, used0)

    # in place: y overwrites x, and the backward call is then given y, whose sign is x's
    x5, dy5, gx5, gdy5 = fresh(shape)
    gpu_op.activation_forward(gx5, gx5, "relu", lst, rt.cudnn, rt.stream)
    assert gx5.asnumpy().tobytes() == O.relu(x5).tobytes()
    assert backward(lst, gx5, gx5, gdy5, shape).tobytes() == O.relu_gradient(x5, dy5).tobytes()
    assert _relu_mask_counts() == (kept0, used0)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(64, 64, 28, 28), (5, 3, 4, 4), (128, 8, 6, 6), (200, 4, 3, 3), (64, 256, 56, 56)],
                         ids=str)
def test_fused_batch_norm_relu_equals_the_two_ops(rt, shape):
    """DLGpuBatchNormalizationRelu{Forward,Backward} against the separate batch-norm
    and ReLU entry points: bit for bit, forward and backward."""
    from tinyflow_amd import gpu_op, ndarray
    gen = np.random.default_rng(8)
    x = gen.standard_normal(shape, dtype=np.float32) * np.float32(1.7) + np.float32(0.3)
    dy = gen.standard_normal(shape, dtype=np.float32)
    gx, gdy = ndarray.array(x, rt.ctx), ndarray.array(dy, rt.ctx)
    e = lambda: ndarray.empty(shape, rt.ctx)
    # the two separate ops
    mean_p, var_p, lst = gpu_op.bn_get_cudnnlist(shape, "NCHW", "pre_activation")
    alst = gpu_op.activation_get_cudnnlist(shape, "NCHW", "relu")
    bn_out, relu_out, relu_dx, dx = e(), e(), e(), e()
    assert gpu_op.bn_forward(gx, bn_out, "pre_activation", 0, mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    gpu_op.activation_forward(bn_out, relu_out, "relu", alst, rt.cudnn, rt.stream)
    gpu_op.activation_backward(bn_out, relu_dx, relu_out, gdy, "relu", alst, rt.cudnn, rt.stream)
    assert gpu_op.bn_backward(gx, relu_dx, dx, "pre_activation", mean_p, var_p, lst, rt.cudnn, rt.stream) == 0
    # the fused pair
    mean_p2, var_p2, lst2 = gpu_op.bn_get_cudnnlist(shape, "NCHW", "pre_activation")
    fused_out, fused_dx = e(), e()
    assert gpu_op.bn_relu_forward(gx, fused_out, "pre_activation", 0, mean_p2, var_p2, lst2, rt.cudnn, rt.stream) == 0
    assert gpu_op.bn_relu_backward(gx, gdy, fused_dx, "pre_activation", mean_p2, var_p2, lst2, rt.cudnn,
                                   rt.stream) == 0
    assert fused_out.asnumpy().tobytes() == relu_out.asnumpy().tobytes()
    assert fused_dx.asnumpy().tobytes() == dx.asnumpy().tobytes()
    # and against the oracle's composition, within the batch-norm tolerance
    if np.prod(shape) < 5_000_000:
        x64 = x.astype(np.float64)
        y_ref, mean, istd = O.batch_norm_forward(x64, "pre_activation")
        np.testing.assert_allclose(fused_out.asnumpy(), np.maximum(y_ref, 0), rtol=1e-4, atol=1e-5)
        dx_ref = O.batch_norm_backward(x64, np.where(y_ref > 0, dy.astype(np.float64), 0.0), "pre_activation", mean, istd)
        got = fused_dx.asnumpy()
        # elements whose normalised value is within rounding of 0 may fall on the other side of the mask
        near = np.abs(y_ref) < 1e-5
        if not near.any():
            np.testing.assert_allclose(got, dx_ref, rtol=1e-3, atol=1e-5 * max(1.0, float(np.abs(dx_ref).max())))


@pytest.mark.gpu
def test_fused_batch_norm_relu_refuses_spatial_mode(rt):
    from tinyflow_amd import gpu_op, ndarray
    shape = (4, 3, 5, 5)
    mean_p, var_p, lst = gpu_op.bn_get_cudnnlist(shape, "NCHW", "spatial")
    x, y = ndarray.array(np.ones(shape, np.float32), rt.ctx), ndarray.empty(shape, rt.ctx)
    with pytest.raises(RuntimeError):
        gpu_op.bn_relu_forward(x, y, "spatial", 0, mean_p, var_p, lst, rt.cudnn, rt.stream)
