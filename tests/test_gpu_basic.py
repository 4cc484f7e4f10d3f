"""GPU parity of the elementwise, reduction, softmax and matmul entry points.

Cases and tolerances follow the reference's own unit tests
(tests/test_gpu_op.py:5-182): exact for set/broadcast/relu masks, rtol 1e-5 for
sums, softmax and matmul at the reference's shapes.
"""
import numpy as np
import pytest

from oracle import ops as O

pytestmark = pytest.mark.gpu


def _gpu(a, rt):
    from tinyflow_amd import ndarray
    return ndarray.array(np.asarray(a, dtype=np.float32), rt.ctx)


def _empty(shape, rt):
    from tinyflow_amd import ndarray
    return ndarray.empty(shape, rt.ctx)


def test_array_roundtrip_and_set(rt):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(0)
    for shape in [(1,), (3,), (5, 7), (2000, 2500), (2, 3, 5, 7), (1025,)]:
        x = rng.uniform(-1, 1, shape).astype(np.float32)
        a = _gpu(x, rt)
        assert a.shape == shape
        np.testing.assert_array_equal(a.asnumpy(), x)
        gpu_op.array_set(a, 3.25, rt.stream)
        np.testing.assert_array_equal(a.asnumpy(), np.full(shape, 3.25, np.float32))


@pytest.mark.parametrize("shape", [(1,), (7,), (500, 200), (2000, 2500), (3, 5, 7, 11), (64, 256, 56, 56)])
def test_elementwise(rt, shape):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(1)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    y = rng.uniform(-1, 1, shape).astype(np.float32)
    x.flat[::7] = 0.0  # exact zeros for the relu mask
    a, b, c = _gpu(x, rt), _gpu(y, rt), _empty(shape, rt)
    gpu_op.matrix_elementwise_add(a, b, c, rt.stream)
    np.testing.assert_array_equal(c.asnumpy(), O.add(x, y))
    gpu_op.matrix_elementwise_multiply(a, b, c, rt.stream)
    np.testing.assert_array_equal(c.asnumpy(), O.multiply(x, y))
    gpu_op.matrix_elementwise_add_by_const(a, 0.37, c, rt.stream)
    np.testing.assert_array_equal(c.asnumpy(), O.add_by_const(x, 0.37))
    gpu_op.matrix_elementwise_multiply_by_const(a, -1.5, c, rt.stream)
    np.testing.assert_array_equal(c.asnumpy(), O.multiply_by_const(x, -1.5))
    gpu_op.relu(a, c)
    np.testing.assert_array_equal(c.asnumpy(), O.relu(x))
    gpu_op.relu_gradient(a, b, c)
    np.testing.assert_array_equal(c.asnumpy(), O.relu_gradient(x, y))
    # mask is x > 0: nothing passes at exact zeros
    assert np.all(c.asnumpy().flat[::7] == 0)
    # SGD in place; a*b+c may or may not be fused, so allow one rounding
    w = _gpu(x, rt)
    gpu_op.sgd_update(w, b, 0.01, rt.stream)
    np.testing.assert_allclose(w.asnumpy(), O.sgd_update(x, y, 0.01), rtol=1e-6, atol=1e-7)


def test_broadcast(rt):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(2)
    b = rng.uniform(-1, 1, (100,)).astype(np.float32)
    out = _empty((128, 100), rt)
    gpu_op.broadcast_to(_gpu(b, rt), out, "NHWC", rt.stream)
    np.testing.assert_array_equal(out.asnumpy(), O.broadcast_to_trailing(b, (128, 100)))
    for shape in [(4, 6, 28, 28), (3, 5, 7, 9), (2, 16, 10, 10)]:
        b = rng.uniform(-1, 1, (shape[1],)).astype(np.float32)
        out = _empty(shape, rt)
        gpu_op.broadcast_to(_gpu(b, rt), out, "NCHW", rt.stream)
        np.testing.assert_array_equal(out.asnumpy(), O.broadcast_to_channel(b, shape))


@pytest.mark.parametrize("shape", [(500, 200, 100), (128, 256), (1000, 10), (7,), (64, 1000), (100000, 3)])
def test_reduce_sum_axis_zero(rt, shape):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(3)
    x = rng.uniform(0, 20, shape).astype(np.float32)
    out_shape = shape[1:] if len(shape) > 1 else (1,)
    out = _empty(out_shape, rt)
    gpu_op.reduce_sum_axis_zero(_gpu(x, rt), out)
    ref = np.sum(x.astype(np.float64), axis=0).reshape(out_shape)
    np.testing.assert_allclose(out.asnumpy(), ref, rtol=1e-5)


@pytest.mark.parametrize("shape,fmt", [((128, 256), "NHWC"), ((128, 10), "NHWC"), ((64, 6, 28, 28), "NCHW"),
                                      ((32, 64, 56, 56), "NCHW"), ((5, 3, 7, 9), "NCHW"), ((2, 16, 10, 10), "NCHW")])
def test_bias_gradient_reduce_sum(rt, shape, fmt):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(4)
    dy = rng.normal(0, 1, shape).astype(np.float32)
    C = shape[1]
    in_s, out_s = gpu_op.reduce_sum_get_real_shape(shape, (C,), fmt)
    lst = gpu_op.reduce_sum_get_cudnnlist(in_s, out_s, fmt, rt.cudnn)
    out = _empty((C,), rt)
    assert gpu_op.reduce_sum_new(_gpu(dy, rt), out, lst, rt.cudnn, rt.stream) == 0
    ref = O.bias_gradient(dy.astype(np.float64), fmt)
    np.testing.assert_allclose(out.asnumpy(), ref, rtol=1e-4, atol=1e-4)
    # legacy entry points compute the same sums
    out2 = _empty((C,), rt)
    gpu_op.broadcast_to_backward(_gpu(dy, rt), out2, fmt)
    np.testing.assert_allclose(out2.asnumpy(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("shape", [(400, 1000), (128, 10), (64, 1000), (1, 3), (5000, 17)])
def test_softmax_and_cross_entropy(rt, shape):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(5)
    y = rng.uniform(-5, 5, shape).astype(np.float32)
    labels = np.zeros(shape, np.float32)
    labels[np.arange(shape[0]), rng.randint(0, shape[1], shape[0])] = 1
    out = _empty(shape, rt)
    gpu_op.softmax(_gpu(y, rt), out, rt.stream)
    np.testing.assert_allclose(out.asnumpy(), O.softmax(y), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(out.asnumpy().sum(axis=1), 1.0, rtol=1e-5)
    loss = _empty((1,), rt)
    gpu_op.softmax_cross_entropy(_gpu(y, rt), _gpu(labels, rt), loss, rt.stream)
    np.testing.assert_allclose(loss.asnumpy(), O.softmax_cross_entropy(y.astype(np.float64), labels), rtol=1e-5)


def test_cross_entropy_without_scratch_memory(rt):
    """More than 16 rows take a two-launch form that needs a small scratch array; with
    no device memory left the one-launch form runs and gives the same bits."""
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(6)
    shape = (70, 1000)
    y = rng.uniform(-5, 5, shape).astype(np.float32)
    labels = np.zeros(shape, np.float32)
    labels[np.arange(shape[0]), rng.randint(0, shape[1], shape[0])] = 1
    gy, gl = _gpu(y, rt), _gpu(labels, rt)
    loss, loss2 = _empty((1,), rt), _empty((1,), rt)
    gpu_op.softmax_cross_entropy(gy, gl, loss, rt.stream)
    _, in_use, _ = gpu_op.device_memory_stats()
    gpu_op.set_device_memory_limit(max(in_use, 1))
    try:
        assert isinstance(ndarray.empty((1 << 20,), rt.ctx), int)
        gpu_op.softmax_cross_entropy(gy, gl, loss2, rt.stream)
        got = loss2.asnumpy()
    finally:
        gpu_op.set_device_memory_limit(0)
    np.testing.assert_array_equal(got, loss.asnumpy())


MM_CASES = [
    # the reference's own cases (tests/test_gpu_op.py:103-131)
    ((500, 700), False, (700, 1000), False),
    ((1000, 700), False, (500, 700), True),   # NT
    ((700, 500), True, (1000, 700), True),    # TT
    # MLP config shapes: forward, dA = dZ W^T, dW = A^T dZ
    ((128, 784), False, (784, 256), False),
    ((128, 256), False, (784, 256), True),
    ((128, 784), True, (128, 256), False),
    ((128, 100), False, (100, 10), False),
    # ragged edges and tiny sizes
    ((3, 2), False, (2, 3), False),
    ((1, 1), False, (1, 1), False),
    ((65, 17), False, (17, 129), False),
    ((33, 130), True, (33, 70), False),
    # extents that are multiples of 4 but not of a tile (16-byte loaders, all four
    # transpose cases), and a reduction that is not (one-element loaders)
    ((132, 36), False, (36, 68), False),
    ((36, 132), True, (36, 68), False),
    ((132, 36), False, (68, 36), True),
    ((36, 132), True, (68, 36), True),
    ((132, 34), False, (34, 68), False),
    ((260, 520), False, (520, 388), False),
    # skinny with a long reduction (split-k path)
    ((32, 4096), False, (4096, 1000), False),
    ((64, 2048), False, (2048, 1000), False),
    ((64, 2048), True, (64, 1000), False),
]


@pytest.mark.parametrize("sa,ta,sb,tb", MM_CASES)
def test_matmul(rt, sa, ta, sb, tb):
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(6)
    a = rng.uniform(-1, 1, sa).astype(np.float32)
    b = rng.uniform(-1, 1, sb).astype(np.float32)
    ref = O.matmul(a.astype(np.float64), ta, b.astype(np.float64), tb)
    c = _empty(ref.shape, rt)
    gpu_op.matrix_multiply(_gpu(a, rt), ta, _gpu(b, rt), tb, c, rt.cublas, rt.stream)
    np.testing.assert_allclose(c.asnumpy(), ref, rtol=1e-5, atol=1e-4)


def test_matmul_reference_integer_case(rt):
    """3x2 . 2x3 integer matrices and their gradients with a ones upstream
    (reference tests/autodiff_test.py:188-208)."""
    from tinyflow_amd import gpu_op
    x2 = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    x3 = np.array([[7, 8, 9], [10, 11, 12]], np.float32)
    y = _empty((3, 3), rt)
    gpu_op.matrix_multiply(_gpu(x2, rt), False, _gpu(x3, rt), False, y, rt.cublas, rt.stream)
    np.testing.assert_array_equal(y.asnumpy(), np.matmul(x2, x3))
    ones = np.ones((3, 3), np.float32)
    d2, d3 = _empty((3, 2), rt), _empty((2, 3), rt)
    gpu_op.matrix_multiply(_gpu(ones, rt), False, _gpu(x3, rt), True, d2, rt.cublas, rt.stream)
    gpu_op.matrix_multiply(_gpu(x2, rt), True, _gpu(ones, rt), False, d3, rt.cublas, rt.stream)
    np.testing.assert_array_equal(d2.asnumpy(), np.matmul(ones, x3.T))
    np.testing.assert_array_equal(d3.asnumpy(), np.matmul(x2.T, ones))


def test_alloc_oom_convention(rt):
    """An allocation the device cannot serve reports the byte count (as a
    32-bit int) and returns no array (reference ndarray.py:251-259)."""
    from tinyflow_amd import ndarray
    ret = ndarray.empty((1 << 20, 1 << 20), rt.ctx)  # 4 TiB
    assert isinstance(ret, int)
    # the reference casts the size to int, which wraps for 2 GiB and more (a request of
    # exactly 4 GiB would read as "no error"); here the report saturates
    assert ret == 2 ** 31 - 1


def test_copy_with_stream_and_d2d(rt):
    from tinyflow_amd import ndarray
    rng = np.random.RandomState(7)
    x = rng.normal(0, 1, (257, 129)).astype(np.float32)
    a = _gpu(x, rt)
    b = _empty(x.shape, rt)
    a.copyto(b, rt.stream)  # device to device on the compute stream
    np.testing.assert_array_equal(b.asnumpy(), x)
    host = ndarray.empty(x.shape, ndarray.cpu(0))  # pinned
    b.copyto(host, rt.stream)
    np.testing.assert_array_equal(host.asnumpy(), x)
    c = host.copyto(rt.ctx, rt.stream)
    np.testing.assert_array_equal(c.asnumpy(), x)


def test_d2d_copy_on_a_side_stream_is_complete_on_return(rt):
    """A device-to-device copy on a stream no op launches on, followed at once by a
    kernel on the compute stream that reads the destination and by a release and
    reuse of the source: the call has to have waited for the copy."""
    from tinyflow_amd import gpu_op, ndarray
    side = gpu_op.create_cudaStream()
    rng = np.random.RandomState(8)
    n = 64 << 20   # 256 MiB: long enough that an unfinished copy would be caught
    x = rng.normal(0, 1, (n,)).astype(np.float32)
    for _ in range(3):
        src = _gpu(x, rt)
        dst = _empty((n,), rt)
        out = _empty((n,), rt)
        gpu_op.array_set(dst, 0.0, rt.stream)
        src.copyto(dst, side)
        gpu_op.matrix_elementwise_multiply_by_const(dst, 2.0, out, rt.stream)   # reads dst on the compute stream
        src.free_gpu()
        clobber = _empty((n,), rt)                                               # may take src's storage
        gpu_op.array_set(clobber, -7.0, rt.stream)
        np.testing.assert_array_equal(out.asnumpy(), x * np.float32(2.0))
        np.testing.assert_array_equal(dst.asnumpy(), x)
    gpu_op.destroy_cudaStream(side)


def test_empty_tensors_are_accepted_everywhere(rt):
    """Zero-element operands: every entry point returns success and launches nothing
    (an empty batch, a layer with no outputs)."""
    from tinyflow_amd import gpu_op, ndarray
    e = lambda *shape: ndarray.empty(shape, rt.ctx)
    a, b, c = e(0, 7), e(0, 7), e(0, 7)
    gpu_op.array_set(a, 1.0, rt.stream)
    gpu_op.matrix_elementwise_add(a, b, c, rt.stream)
    gpu_op.matrix_elementwise_multiply(a, b, c, rt.stream)
    gpu_op.matrix_elementwise_add_by_const(a, 2.0, c, rt.stream)
    gpu_op.matrix_elementwise_multiply_by_const(a, 2.0, c, rt.stream)
    gpu_op.relu(a, c)
    gpu_op.relu_gradient(a, b, c)
    gpu_op.softmax(a, c, rt.stream)
    gpu_op.sgd_update(a, b, 0.1, rt.stream)
    assert c.asnumpy().shape == (0, 7)
    # matmul with an empty row set, and with an empty reduction (result is all zeros)
    out = e(0, 5)
    gpu_op.matrix_multiply(e(0, 7), False, e(7, 5), False, out, rt.cublas, rt.stream)
    out = ndarray.array(np.full((3, 5), np.nan, np.float32), rt.ctx)
    gpu_op.matrix_multiply(e(3, 0), False, e(0, 5), False, out, rt.cublas, rt.stream)
    assert np.array_equal(out.asnumpy(), np.zeros((3, 5), np.float32))
    # convolution, pooling, batch norm, activation on an empty batch
    shape, wshape = (0, 3, 8, 8), (4, 3, 3, 3)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(shape, wshape, "NCHW", "SAME", 1, 1)
    assert out_shape == (0, 4, 8, 8)
    x, w, y = e(*shape), ndarray.array(np.ones(wshape, np.float32), rt.ctx), e(*out_shape)
    dw = ndarray.array(np.full(wshape, np.nan, np.float32), rt.ctx)
    assert gpu_op.convolution_2d_forward(x, w, y, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.convolution_backward_data(x, y, w, e(*shape), lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.convolution_backward_filter(x, y, w, dw, lst, rt.cudnn, rt.stream) == 0
    assert np.array_equal(dw.asnumpy(), np.zeros(wshape, np.float32))   # empty reduction: zeros, not stale data
    pshape, plst = gpu_op.pooling_2d_forward_get_out_shape(shape, "NCHW", "max", 0, 0, 2, 2, 2, 2)
    py = e(*pshape)
    gpu_op.pooling_2d_forward(x, py, plst, rt.cudnn, rt.stream)
    gpu_op.pooling_2d_backward(x, py, py, e(*shape), plst, rt.cudnn, rt.stream)
    alst = gpu_op.activation_get_cudnnlist(shape, "NCHW", "relu")
    gpu_op.activation_forward(x, e(*shape), "relu", alst, rt.cudnn, rt.stream)
    gpu_op.activation_backward(x, e(*shape), x, x, "relu", alst, rt.cudnn, rt.stream)


@pytest.mark.parametrize("shape", [(64, 256, 28, 28), (5, 3), (1,), (1025,)])
def test_add_relu_equals_add_then_relu(rt, shape):
    from tinyflow_amd import gpu_op, ndarray
    gen = np.random.default_rng(3)
    a = gen.standard_normal(shape, dtype=np.float32)
    b = gen.standard_normal(shape, dtype=np.float32)
    b.reshape(-1)[::5] = -a.reshape(-1)[::5]      # exact zeros in the sum
    ga, gb = ndarray.array(a, rt.ctx), ndarray.array(b, rt.ctx)
    s, want, got = ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx), ndarray.empty(shape, rt.ctx)
    gpu_op.matrix_elementwise_add(ga, gb, s, rt.stream)
    gpu_op.relu(s, want)
    gpu_op.matrix_elementwise_add_relu(ga, gb, got, rt.stream)
    assert got.asnumpy().tobytes() == want.asnumpy().tobytes()
    assert got.asnumpy().tobytes() == O.relu(O.add(a, b)).tobytes()


def test_adam_two_kernel_form(rt):
    """DLGpuAdam_mv then DLGpuAdam against the written-out formulas (gpu_op.cu:4461-4506)."""
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(31)
    shape = (257, 33)
    w, g = rng.normal(0, 1, shape).astype(np.float32), rng.normal(0, 0.1, shape).astype(np.float32)
    m, v = rng.normal(0, 0.1, shape).astype(np.float32), rng.uniform(0, 0.01, shape).astype(np.float32)
    gw, gg, gm, gv = (_gpu(a, rt) for a in (w, g, m, v))
    # the coefficients reach the kernels as C floats: the oracle gets the same rounded values
    b1, b2, b1t, b2t = (float(np.float32(c)) for c in (0.9, 0.999, 0.9 ** 3, 0.999 ** 3))
    gpu_op.adam_mv(gm, gv, gg, b1, b2, rt.stream)
    m_ref, v_ref = O.adam_mv(m.astype(np.float64), v.astype(np.float64), g.astype(np.float64), b1, b2)
    np.testing.assert_allclose(gm.asnumpy(), m_ref, rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(gv.asnumpy(), v_ref, rtol=1e-6, atol=1e-10)
    gpu_op.adam_compute(gw, gm, gv, b1t, b2t, 1e-8, 0.001, rt.stream)
    w_ref = O.adam_update(w.astype(np.float64), m_ref, v_ref, b1t, b2t, 1e-8, 0.001)
    np.testing.assert_allclose(gw.asnumpy(), w_ref, rtol=1e-5, atol=1e-7)


def _flat_index_tables(sizes):
    """index -> (tensor number, offset inside it) for tensors laid end to end, the
    tables DLGpuSgd_o / DLGpuAdam_o walk (gpu_op.cu:4824-4836)."""
    number = np.concatenate([np.full(n, t, dtype=np.int32) for t, n in enumerate(sizes)])
    offset = np.concatenate([np.arange(n, dtype=np.int32) for n in sizes])
    return [int(i) for i in number], [int(i) for i in offset]


def test_fused_multi_tensor_sgd_and_adam(rt):
    """One launch over all parameter tensors equals the per-tensor entry points bit for
    bit (same arithmetic per element; Adam: same expressions as the two-kernel form)."""
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(32)
    _fused_case(rt, scattered=False)


def test_fused_multi_tensor_updates_with_scattered_indices(rt):
    """The same with the index tables in a shuffled order: no runs of consecutive offsets,
    so the launch walks the per-parameter tables instead of whole pieces of tensors."""
    _fused_case(rt, scattered=True)


def test_fused_multi_tensor_updates_from_tensor_sizes(rt):
    """The same with the tables built from the tensors' element counts."""
    _fused_case(rt, scattered=False, from_sizes=True)


def test_fused_update_tables_are_counted_and_released(rt):
    """The index and pointer tables come from the device pool and go back to it: the
    allocator's in-use figure returns to where it started (the reference never frees
    them, gpu_op.cu:4628-4700).  Tables that describe whole tensors cost a few hundred
    bytes, not 8 bytes per parameter; a launch with another count than the tables were
    built for is refused."""
    from tinyflow_amd import gpu_op
    sizes = [1 << 20, 3, 1 << 18]
    w = [_gpu(np.zeros(n, np.float32), rt) for n in sizes]
    g = [_gpu(np.ones(n, np.float32), rt) for n in sizes]
    before = gpu_op.device_memory_stats()[1]
    number, offset = _flat_index_tables(sizes)
    t1 = gpu_op.get_index_to_VaribaleNumber_cuda_pointer(np.array(number, np.int32), np.array(offset, np.int32),
                                                         len(number))
    t2, count = gpu_op.get_tensor_runs_cuda_pointer(sizes)
    assert count == sum(sizes)
    n2 = gpu_op.get_n2_cuda_pointer([a.handle.contents.data for a in w], [a.handle.contents.data for a in g], 3)
    held = gpu_op.device_memory_stats()[1] - before
    assert 0 < held < 64 * 1024, held
    gpu_op.sgd_compute_o(n2, t1, count, 0.5)
    gpu_op.sgd_compute_o(n2, t2, count, 0.25)
    with pytest.raises(Exception):
        gpu_op.sgd_compute_o(n2, t2, count - 1, 0.25)
    for a in w:
        np.testing.assert_array_equal(a.asnumpy(), np.full(a.shape, -0.75, np.float32))
    gpu_op.free_index_cuda_pointer(t1)
    gpu_op.free_index_cuda_pointer(t2)
    gpu_op.free_n_cuda_pointer(n2, 2)
    assert gpu_op.device_memory_stats()[1] == before
    gpu_op.free_index_cuda_pointer(t1)   # a released cell is null: nothing happens


def _fused_case(rt, scattered, from_sizes=False):
    from tinyflow_amd import gpu_op
    # several pieces per tensor (a piece is 4096 elements), odd sizes, one-element tensors
    shapes = [(64, 3, 3, 3), (10,), (1,), (129, 7), (2, 2), (5000, 3), (4096,), (3, 4099)]
    sizes = [int(np.prod(s)) for s in shapes]
    number, offset = _flat_index_tables(sizes)
    count = len(number)
    if scattered:
        order = np.random.RandomState(31).permutation(count)
        number, offset = [number[i] for i in order], [offset[i] for i in order]
        tables = gpu_op.get_index_to_VaribaleNumber_cuda_pointer(number, offset, count)
    elif from_sizes:   # as the step executor builds them
        tables, total = gpu_op.get_tensor_runs_cuda_pointer(sizes)
        assert total == count
    else:   # numpy tables
        tables = gpu_op.get_index_to_VaribaleNumber_cuda_pointer(np.array(number, np.int32), np.array(offset, np.int64),
                                                                 count)

    def fresh():
        r = np.random.RandomState(33)
        return [[_gpu(r.normal(0, 1, s) if k != 2 else r.uniform(0, 0.01, s), rt) for s in shapes]
                for k in range(4)]   # w, m, v, g

    def pointers(arrays):
        return [a.handle.contents.data for a in arrays]

    # SGD
    w1, _, _, g1 = fresh()
    w2, _, _, g2 = fresh()
    for w, g in zip(w1, g1):
        gpu_op.sgd_update(w, g, 0.05, rt.stream)
    n2 = gpu_op.get_n2_cuda_pointer(pointers(w2), pointers(g2), len(shapes))
    gpu_op.sgd_compute_o(n2, tables, count, 0.05)
    for a, b in zip(w1, w2):
        np.testing.assert_array_equal(a.asnumpy(), b.asnumpy())
    # Adam
    w1, m1, v1, g1 = fresh()
    w2, m2, v2, g2 = fresh()
    b1t, b2t = 0.9 ** 2, 0.999 ** 2
    for w, m, v, g in zip(w1, m1, v1, g1):
        gpu_op.adam_mv(m, v, g, 0.9, 0.999, rt.stream)
        gpu_op.adam_compute(w, m, v, b1t, b2t, 1e-8, 0.001, rt.stream)
    n4 = gpu_op.get_n4_cuda_pointer(pointers(w2), pointers(m2), pointers(v2), pointers(g2), len(shapes))
    gpu_op.adam_compute_o(n4, tables, count, 0.9, 0.999, b1t, b2t, 1e-8, 0.001)
    for name, one, two in (("m", m1, m2), ("v", v1, v2), ("w", w1, w2)):
        for a, b in zip(one, two):
            np.testing.assert_allclose(a.asnumpy(), b.asnumpy(), rtol=2e-7, atol=1e-7, err_msg=name)
    gpu_op.free_index_cuda_pointer(tables)
    gpu_op.free_n_cuda_pointer(n2, 2)
    gpu_op.free_n_cuda_pointer(n4, 4)


@pytest.mark.parametrize("shape", [(128, 10), (32, 1000), (7, 3)])
def test_cross_and_its_gradient(rt, shape):
    """DLGpuCross / DLGpuCrossBackward: -b * y * log(x) and -b * y / x * dout
    (gpu_op.cu:4538-4597)."""
    from tinyflow_amd import gpu_op
    rng = np.random.RandomState(34)
    x = rng.uniform(0.01, 1.0, shape).astype(np.float32)
    y = np.zeros(shape, np.float32)
    y[np.arange(shape[0]), rng.randint(0, shape[1], shape[0])] = 1.0
    dout = rng.normal(0, 1, shape).astype(np.float32)
    b = 1.0 / x.size
    out, dx = _empty(shape, rt), _empty(shape, rt)
    gpu_op.cross(_gpu(x, rt), _gpu(y, rt), out, b, rt.stream)
    np.testing.assert_allclose(out.asnumpy(), O.cross(x.astype(np.float64), y, b), rtol=1e-5, atol=1e-12)
    gpu_op.cross_backward(_gpu(x, rt), _gpu(y, rt), _gpu(dout, rt), dx, b, rt.stream)
    np.testing.assert_allclose(dx.asnumpy(), O.cross_backward(x.astype(np.float64), y, dout.astype(np.float64), b),
                               rtol=1e-5, atol=1e-12)


def test_stream_and_handle_life_cycle(rt):
    """Create / use / destroy a stream with its two handles; a second destroy of the
    same cell is reported as an error instead of touching freed memory."""
    from tinyflow_amd import gpu_op
    stream = gpu_op.create_cudaStream()
    cudnn, cublas = gpu_op.create_cudnnHandle(stream), gpu_op.create_cublasHandle(stream)
    a = _gpu(np.arange(6, dtype=np.float32).reshape(2, 3), rt)
    b = _gpu(np.ones((3, 2), np.float32), rt)
    c = _empty((2, 2), rt)
    gpu_op.matrix_multiply(a, False, b, False, c, cublas, stream)
    np.testing.assert_array_equal(c.asnumpy(), [[3, 3], [12, 12]])
    gpu_op.destroy_cudnnHandle(cudnn)
    gpu_op.destroy_cublasHandle(cublas)
    gpu_op.destroy_cudaStream(stream)
    with pytest.raises(RuntimeError):
        gpu_op.destroy_cudnnHandle(cudnn)
    with pytest.raises(RuntimeError):
        gpu_op.destroy_cudaStream(stream)
