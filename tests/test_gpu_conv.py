"""GPU parity of conv2d forward / grad-data / grad-filter against the oracle.

Two bars per tensor.  (i) rtol 1e-3 / atol 1e-5 x the tensor's largest magnitude
against a float64 evaluation of the oracle.  (ii) The HIP result's distance from
that float64 evaluation is at most K_DIRECT (direct form) or K_WINOGRAD (forced
Winograd forms) times the distance of the oracle's own float32 evaluation on the
same inputs -- the figure a numpy fp32 executor would show.  The fraction of
elements inside the unscaled rtol 1e-3 / atol 1e-5 band is recorded per tensor
(tests/parity.py).  The cases cover every filter/stride/padding family of the
LeNet, VGG-16 and ResNet-50 configs at reduced batch or spatial size, plus ragged
sizes that exercise every tile tail.  Inputs are seeded from the case's text, so a
failure replays.
"""
import numpy as np
import pytest

from oracle import ops as O
import parity

pytestmark = pytest.mark.gpu

# largest allowed ratio of the HIP error to the fp32 CPU oracle's error (both against float64)
# (numpy's fp32 matmul is BLAS, which spreads a reduction over 16-32 SIMD partial sums; a
# contraction that keeps one fp32 accumulator per output element, as the matrix cores do,
# rounds along a 16-32 times longer chain -- tests/test_gpu_conv_fullsize.py also holds
# the kernels to 3x a one-accumulator fp32 loop)
K_DIRECT = 16.0
K_WINOGRAD = 24.0

# (N, C, H, W, K, R, S, padding, u, v)
CONV_CASES = [
    # reference tests/autodiff_test.py:335-343: x (5,1,4,4), w (1,1,3,3)
    (5, 1, 4, 4, 1, 3, 3, "VALID", 1, 1),
    (5, 1, 4, 4, 1, 3, 3, "SAME", 1, 1),
    # LeNet-5
    (64, 1, 28, 28, 6, 5, 5, "SAME", 1, 1),
    (64, 6, 14, 14, 16, 5, 5, "VALID", 1, 1),
    # VGG-style 3x3 pad 1
    (2, 3, 32, 32, 64, 3, 3, "SAME", 1, 1),
    (2, 64, 28, 28, 128, 3, 3, "SAME", 1, 1),
    # ResNet-50 families (batch 4)
    (4, 3, 64, 64, 64, 7, 7, "SAME", 2, 2),      # stem 7x7 s2 p3
    (4, 64, 56, 56, 64, 1, 1, "VALID", 1, 1),    # 1x1 s1
    (4, 64, 56, 56, 256, 1, 1, "VALID", 1, 1),
    (4, 256, 56, 56, 128, 1, 1, "VALID", 2, 2),  # 1x1 s2 (first conv of a stage)
    (4, 256, 56, 56, 512, 1, 1, "VALID", 2, 2),  # 1x1 s2 shortcut
    (4, 128, 28, 28, 128, 3, 3, "SAME", 1, 1),
    (4, 512, 7, 7, 512, 3, 3, "SAME", 1, 1),
    (4, 2048, 7, 7, 512, 1, 1, "VALID", 1, 1),
    (4, 1024, 14, 14, 2048, 1, 1, "VALID", 2, 2),
    # ragged everything: odd sizes, non-square filter, different strides
    (3, 5, 13, 11, 7, 3, 2, "SAME", 1, 1),
    (2, 9, 17, 19, 70, 3, 3, "VALID", 2, 2),     # strided 3x3 (generic grad-data path)
    (2, 4, 15, 15, 5, 5, 5, "SAME", 3, 2),
    (1, 1, 1, 1, 1, 1, 1, "VALID", 1, 1),
    (2, 3, 9, 9, 4, 1, 1, "VALID", 2, 2),        # 1x1 s2 on an odd extent
    (2, 130, 6, 6, 67, 1, 1, "VALID", 3, 3),
    # around the conditions of the 16-byte loaders (channels, pixels per image multiples of 4 or not)
    (3, 8, 6, 6, 10, 1, 1, "VALID", 1, 1),       # 1x1, 36 pixels, 8 channels: both operands vectorised
    (2, 12, 10, 10, 7, 1, 1, "VALID", 1, 1),
    (2, 6, 8, 8, 10, 1, 1, "VALID", 1, 1),       # 6 channels: one-element loaders
    (2, 8, 5, 5, 12, 1, 1, "VALID", 1, 1),       # 25 pixels per image: one-element loaders
    (2, 8, 9, 9, 12, 3, 3, "SAME", 1, 1),        # 3x3: vectorised filter, gathered input, 81 pixels
    (2, 8, 10, 10, 12, 3, 3, "SAME", 1, 1),      # 100 pixels: vectorised dy in grad-filter
    (2, 8, 12, 12, 16, 1, 1, "VALID", 2, 2),     # 1x1 s2, even extents: paired scatter stores
    (130, 4, 2, 2, 4, 1, 1, "VALID", 1, 1),      # many tiny images: a 4-vector per image
]


def _gpu(a, rt):
    from tinyflow_amd import ndarray
    return ndarray.array(np.asarray(a, dtype=np.float32), rt.ctx)


def _describe(lst, which):
    """Plan of the launch for `which` (0 forward, 1 grad-data, 2 grad-filter)."""
    import ctypes
    from tinyflow_amd import _base
    buf = ctypes.create_string_buffer(256)
    assert _base._LIB.DLGpuConvolutionDescribeKernel(lst, which, buf, 256, None) == 0
    return buf.value.decode()


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_conv_forward_and_gradients(rt, case):
    _check_conv_case(rt, case)


# 3x3 / stride-1 shapes for the Winograd form (forced on: the planner would pick the
# direct form for most of these small sizes).  (.., expect forward, expect grad-data)
WINOGRAD_CASES = [
    ((4, 128, 28, 28, 128, 3, 3, "SAME", 1, 1), True, True),
    ((4, 64, 56, 56, 64, 3, 3, "SAME", 1, 1), True, True),
    ((2, 64, 30, 26, 128, 3, 3, "SAME", 1, 1), True, True),     # extents that are not multiples of 4
    ((4, 512, 7, 7, 512, 3, 3, "SAME", 1, 1), True, True),      # odd extent: half-empty edge tiles
    ((2, 516, 6, 6, 520, 3, 3, "SAME", 1, 1), True, True),      # more than 512 channels: 2x2 tiles only
    ((2, 64, 14, 14, 256, 3, 3, "SAME", 1, 1), True, True),
    ((3, 8, 5, 5, 12, 3, 3, "SAME", 1, 1), True, True),         # 27 tiles: padded to 28 columns
    ((1, 4, 7, 9, 4, 3, 3, "SAME", 1, 1), True, True),
    ((2, 8, 9, 9, 12, 3, 3, "VALID", 1, 1), True, True),        # no padding: grad-data pads by 2
    ((5, 1, 4, 4, 1, 3, 3, "SAME", 1, 1), False, False),        # one channel: not a multiple of 4
    ((2, 3, 32, 32, 64, 3, 3, "SAME", 1, 1), False, False),     # 3 input channels
    ((2, 132, 6, 6, 68, 3, 3, "SAME", 1, 1), True, True),
    ((2, 8, 8, 8, 6, 3, 3, "SAME", 1, 1), True, False),         # 6 output channels: grad-data reduces over 6
    ((2, 6, 8, 8, 8, 3, 3, "SAME", 1, 1), False, False),
    ((130, 4, 2, 2, 4, 3, 3, "SAME", 1, 1), True, True),        # one tile per image
    ((2, 8, 9, 9, 12, 3, 3, "SAME", 2, 2), False, False),       # strided: never
]


@pytest.mark.parametrize("force", ["2", "4"])
@pytest.mark.parametrize("case,fwd,dgrad", WINOGRAD_CASES, ids=lambda c: "x".join(str(v) for v in c) if isinstance(c, tuple) else str(c))
def test_conv_winograd_form(rt, monkeypatch, case, fwd, dgrad, force):
    """F(2x2, 3x3) and F(4x4, 3x3), forced; the latter is limited to 512 reduction channels."""
    from tinyflow_amd import gpu_op
    monkeypatch.setenv("TINYFLOW_WINOGRAD", force)
    N, C, H, W, K, R, S, padding, u, v = case
    _, lst = gpu_op.convolution_2d_forward_get_out_shape((N, C, H, W), (K, C, R, S), "NCHW", padding, u, v)
    tag = "winograd4x4" if force == "4" else "winograd "
    assert (tag in _describe(lst, 0)) == (fwd and (force == "2" or C <= 512))
    assert (tag in _describe(lst, 1)) == (dgrad and (force == "2" or K <= 512))
    # grad-filter reduces over the tiles: no condition on the channel counts for 2x2 tiles,
    # which also stand in where 4x4 tiles are not allowed (more than 512 channels)
    wtag = "wgrad_winograd4x4" if force == "4" and C <= 512 and K <= 512 else "wgrad_winograd "
    assert (wtag in _describe(lst, 2)) == (u == 1 and v == 1)
    _check_conv_case(rt, case)
    monkeypatch.setenv("TINYFLOW_WINOGRAD", "0")
    assert not any("winograd" in _describe(lst, which) for which in range(3))


def _check_conv_case(rt, case):
    from tinyflow_amd import gpu_op, ndarray
    N, C, H, W, K, R, S, padding, u, v = case
    rng = np.random.RandomState(parity.stable_seed(case))
    x = rng.normal(0, 1, (N, C, H, W)).astype(np.float32)
    w = rng.normal(0, np.sqrt(2.0 / (C * R * S)), (K, C, R, S)).astype(np.float32)
    pad_h, pad_w = O.conv_pad(R, padding), O.conv_pad(S, padding)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", padding, u, v)
    P, Q = O.conv_out_extent(H, R, pad_h, u), O.conv_out_extent(W, S, pad_w, v)
    assert out_shape == (N, K, P, Q)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)

    x64, w64, dy64 = x.astype(np.float64), w.astype(np.float64), dy.astype(np.float64)
    y_ref = O.conv2d_forward(x64, w64, pad_h, pad_w, u, v)
    dx_ref = O.conv2d_backward_data(dy64, w64, x.shape, pad_h, pad_w, u, v)
    dw_ref = O.conv2d_backward_filter(x64, dy64, w.shape, pad_h, pad_w, u, v)
    # the same three in float32: what a numpy fp32 executor produces
    y_cpu32 = O.conv2d_forward(x, w, pad_h, pad_w, u, v)
    dx_cpu32 = O.conv2d_backward_data(dy, w, x.shape, pad_h, pad_w, u, v)
    dw_cpu32 = O.conv2d_backward_filter(x, dy, w.shape, pad_h, pad_w, u, v)
    assert y_cpu32.dtype == dx_cpu32.dtype == dw_cpu32.dtype == np.float32

    gx, gw, gdy = _gpu(x, rt), _gpu(w, rt), _gpu(dy, rt)
    gy = ndarray.empty(out_shape, rt.ctx)
    gdx = ndarray.empty(x.shape, rt.ctx)
    gdw = ndarray.empty(w.shape, rt.ctx)
    # poison the outputs: every element must be written (beta = 0 semantics)
    gpu_op.array_set(gy, np.nan, rt.stream)
    gpu_op.array_set(gdx, np.nan, rt.stream)
    gpu_op.array_set(gdw, np.nan, rt.stream)
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream) == 0

    def check(got, ref, cpu32, which, what):
        scale = max(1.0, float(np.abs(ref).max()))
        np.testing.assert_allclose(got, ref, rtol=1e-3, atol=1e-5 * scale, err_msg=what)
        plan = _describe(lst, which)
        form = "winograd F(4x4)" if "winograd4x4" in plan else "winograd F(2x2)" if "winograd" in plan else "direct"
        parity.compare(got, ref, cpu32, "conv %s, %s" % (what, form), "%s %s" % (what, (case,)),
                       K_DIRECT if form == "direct" else K_WINOGRAD)

    check(gy.asnumpy(), y_ref, y_cpu32, 0, "forward")
    check(gdx.asnumpy(), dx_ref, dx_cpu32, 1, "grad-data")
    check(gdw.asnumpy(), dw_ref, dw_cpu32, 2, "grad-filter")


def test_conv_gradients_are_deterministic(rt):
    """Split reductions are added in a fixed order: two runs agree bit for bit."""
    from tinyflow_amd import gpu_op, ndarray
    rng = np.random.RandomState(11)
    x = rng.normal(0, 1, (8, 64, 28, 28)).astype(np.float32)
    w = rng.normal(0, 0.05, (64, 64, 3, 3)).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", "SAME", 1, 1)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gw, gdy = _gpu(x, rt), _gpu(w, rt), _gpu(dy, rt)
    outs = []
    for _ in range(2):
        gdw = ndarray.empty(w.shape, rt.ctx)
        gdx = ndarray.empty(x.shape, rt.ctx)
        gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream)
        gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream)
        outs.append((gdw.asnumpy(), gdx.asnumpy()))
    np.testing.assert_array_equal(outs[0][0], outs[1][0])
    np.testing.assert_array_equal(outs[0][1], outs[1][1])


SCRATCH_CASES = [
    ((2, 64, 16, 16, 64, 3, 3, "SAME", 1, 1), "0"),     # direct forms: re-laid filter, k-split partials or fold pieces
    ((1, 64, 8, 8, 1024, 3, 3, "SAME", 1, 1), "0"),     # one tile, long reduction: grad-data splits
    ((8, 128, 7, 7, 256, 1, 1, "VALID", 1, 1), "0"),    # 1x1
    ((4, 64, 28, 28, 64, 3, 3, "SAME", 1, 1), "4"),     # Winograd scratch
]


@pytest.mark.parametrize("case,wino", SCRATCH_CASES, ids=lambda c: "x".join(str(v) for v in c) if isinstance(c, tuple) else "w" + str(c))
def test_conv_reports_all_the_scratch_it_needs(rt, monkeypatch, case, wino):
    """With no room for scratch an entry point writes the bytes it wants and returns 0
    (the reference's workspace convention); a caller that then makes exactly that much
    room must be able to repeat the call, however many blocks the entry point takes,
    and gets the bits of a call without a limit."""
    from tinyflow_amd import gpu_op, ndarray
    monkeypatch.setenv("TINYFLOW_WINOGRAD", wino)
    N, C, H, W, K, R, S, padding, u, v = case
    rng = np.random.RandomState(parity.stable_seed(case))
    x = rng.normal(0, 1, (N, C, H, W)).astype(np.float32)
    w = rng.normal(0, 0.05, (K, C, R, S)).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", padding, u, v)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gw, gdy = _gpu(x, rt), _gpu(w, rt), _gpu(dy, rt)
    outs = [ndarray.empty(sh, rt.ctx) for sh in (out_shape, x.shape, w.shape)]
    calls = [lambda o: gpu_op.convolution_2d_forward(gx, gw, o, lst, rt.cudnn, rt.stream),
             lambda o: gpu_op.convolution_backward_data(gx, gdy, gw, o, lst, rt.cudnn, rt.stream),
             lambda o: gpu_op.convolution_backward_filter(gx, gdy, gw, o, lst, rt.cudnn, rt.stream)]
    free = []
    for call, o in zip(calls, outs):
        assert call(o) == 0
        free.append(o.asnumpy())
    in_use = gpu_op.device_memory_stats()[1]
    needed_scratch = 0
    try:
        for call, o, want in zip(calls, outs, free):
            gpu_op.set_device_memory_limit(0)
            gpu_op.set_device_memory_limit(max(in_use, 1))     # nothing more can be allocated
            gpu_op.array_set(o, np.nan, rt.stream)
            wanted = call(o)
            if wanted == 0:                                     # this form takes no scratch
                assert o.asnumpy().tobytes() == want.tobytes()
                continue
            needed_scratch += 1
            gpu_op.set_device_memory_limit(0)
            gpu_op.set_device_memory_limit(in_use + -(-wanted // 65536) * 65536)   # budgets count in 64 KiB units
            assert call(o) == 0, "%d bytes were reported, and with that much room the call still finds none" % wanted
            assert o.asnumpy().tobytes() == want.tobytes()
    finally:
        gpu_op.set_device_memory_limit(0)
    assert needed_scratch > 0 or wino == "0"


def _kept_counts():
    import ctypes
    from tinyflow_amd import _base
    kept, taken, held = ctypes.c_longlong(), ctypes.c_longlong(), ctypes.c_int()
    assert _base._LIB.DLGpuKeptByproductCounts(ctypes.byref(kept), ctypes.byref(taken), ctypes.byref(held)) == 0
    return kept.value, taken.value, held.value


def test_kept_transformed_input_follows_the_input_array(rt, monkeypatch):
    """A Winograd forward call keeps its transformed input for the grad-filter call on the
    same array.  Grad-filter must give the bits it gives without the kept block, and must
    not use a block whose source array was overwritten, freed or replaced in between."""
    from tinyflow_amd import gpu_op, ndarray
    monkeypatch.setenv("TINYFLOW_WINOGRAD", "4")
    rng = np.random.RandomState(23)
    xs, ws = (4, 64, 28, 28), (64, 64, 3, 3)
    x1 = rng.normal(0, 1, xs).astype(np.float32)
    x2 = rng.normal(0, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.05, ws).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(xs, ws, "NCHW", "SAME", 1, 1)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gw, gdy = _gpu(w, rt), _gpu(dy, rt)
    gy = ndarray.empty(out_shape, rt.ctx)

    def grad_filter(gx):
        gdw = ndarray.empty(ws, rt.ctx)
        assert gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream) == 0
        return gdw.asnumpy()

    gx = _gpu(x1, rt)
    want1 = grad_filter(gx)                    # nothing kept yet: transforms x itself
    gx2 = _gpu(x2, rt)
    want2 = grad_filter(gx2)
    assert not np.array_equal(want1, want2)

    # forward then grad-filter on the untouched array: the kept block is taken over
    kept0, taken0, _ = _kept_counts()
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    kept1, taken1, held1 = _kept_counts()
    assert kept1 == kept0 + 1 and held1 >= 1
    np.testing.assert_array_equal(grad_filter(gx), want1)
    assert _kept_counts()[1] == taken1 + 1

    # the array is overwritten between the two calls: the block is dropped, x2 is transformed
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    gx[:] = x2
    taken = _kept_counts()[1]
    np.testing.assert_array_equal(grad_filter(gx), want2)
    assert _kept_counts()[1] == taken

    # an in-place kernel writes the array
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    gpu_op.matrix_elementwise_multiply_by_const(gx, 2.0, gx, rt.stream)
    np.testing.assert_array_equal(grad_filter(gx), grad_filter(_gpu(2.0 * x2, rt)))

    # the array is freed and another one (most likely at the same address) takes its place
    gx = _gpu(x1, rt)
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    del gx
    gx = _gpu(x2, rt)
    taken = _kept_counts()[1]
    np.testing.assert_array_equal(grad_filter(gx), want2)
    assert _kept_counts()[1] == taken

    # grad-filter on another array than the one forward saw
    gx = _gpu(x1, rt)
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    np.testing.assert_array_equal(grad_filter(gx2), want2)


def test_kept_transformed_filter_follows_the_filter_array(rt, monkeypatch):
    """A Winograd forward call also writes the transformed filter that grad-data needs and
    keeps it.  Grad-data must give the bits it gives without the kept block, and must not
    use a block whose filter was updated in between."""
    from tinyflow_amd import gpu_op, ndarray
    monkeypatch.setenv("TINYFLOW_WINOGRAD", "4")
    rng = np.random.RandomState(29)
    xs, ws = (4, 64, 28, 28), (128, 64, 3, 3)
    x = rng.normal(0, 1, xs).astype(np.float32)
    w1 = rng.normal(0, 0.05, ws).astype(np.float32)
    g = rng.normal(0, 0.05, ws).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(xs, ws, "NCHW", "SAME", 1, 1)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gdy, gg = _gpu(x, rt), _gpu(dy, rt), _gpu(g, rt)
    gy = ndarray.empty(out_shape, rt.ctx)

    def grad_data(gw):
        gdx = ndarray.empty(xs, rt.ctx)
        assert gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream) == 0
        return gdx.asnumpy()

    gw = _gpu(w1, rt)
    want1 = grad_data(gw)                      # nothing kept yet
    gw2 = _gpu(w1 - 0.5 * g, rt)
    want2 = grad_data(gw2)
    assert not np.array_equal(want1, want2)

    kept0, taken0, _ = _kept_counts()
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    assert _kept_counts()[0] >= kept0 + 1
    taken = _kept_counts()[1]
    np.testing.assert_array_equal(grad_data(gw), want1)
    assert _kept_counts()[1] == taken + 1

    # the update of the filter comes between forward and grad-data: the block is dropped
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    gpu_op.sgd_update(gw, gg, 0.5, rt.stream)
    taken = _kept_counts()[1]
    np.testing.assert_array_equal(grad_data(gw), want2)
    assert _kept_counts()[1] == taken

    # forward itself gives the same bits with and without the second output
    y_with = gy.asnumpy()
    gw3 = _gpu(w1, rt)
    assert gpu_op.convolution_2d_forward(gx, gw3, gy, lst, rt.cudnn, rt.stream) == 0
    y1 = gy.asnumpy()
    _, lst_fresh = gpu_op.convolution_2d_forward_get_out_shape(xs, ws, "NCHW", "SAME", 1, 1)
    assert gpu_op.convolution_2d_forward(gx, gw3, gy, lst_fresh, rt.cudnn, rt.stream) == 0
    np.testing.assert_array_equal(gy.asnumpy(), y1)
    assert y_with.shape == y1.shape


@pytest.mark.parametrize("shape", [(4, 64, 28, 28, 64), (3, 32, 14, 14, 48), (2, 16, 7, 9, 24)],
                         ids=lambda s: "x".join(str(v) for v in s))
def test_shared_dy_transform_of_the_two_gradients(rt, monkeypatch, shape):
    """Grad-data and grad-filter of a padded 3x3 layer both transform dy; whichever runs
    first writes the other's form too.  Either order gives the bits of the separate
    passes, and a dy overwritten between the two calls is transformed again."""
    from tinyflow_amd import gpu_op, ndarray
    monkeypatch.setenv("TINYFLOW_WINOGRAD", "4")
    N, C, H, W, K = shape
    rng = np.random.RandomState(31)
    xs, ws = (N, C, H, W), (K, C, 3, 3)
    x = rng.normal(0, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.05, ws).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(xs, ws, "NCHW", "SAME", 1, 1)
    dy1 = rng.normal(0, 1, out_shape).astype(np.float32)
    dy2 = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gw = _gpu(x, rt), _gpu(w, rt)

    def grad_data(gdy):
        gdx = ndarray.empty(xs, rt.ctx)
        assert gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream) == 0
        return gdx.asnumpy()

    def grad_filter(gdy):
        gdw = ndarray.empty(ws, rt.ctx)
        assert gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream) == 0
        return gdw.asnumpy()

    def fresh(fn, dy):
        """The call on a descriptor that has seen nothing yet: no sharing."""
        nonlocal lst
        keep = lst
        _, lst = gpu_op.convolution_2d_forward_get_out_shape(xs, ws, "NCHW", "SAME", 1, 1)
        out = fn(_gpu(dy, rt))
        lst = keep
        return out

    want_dx1, want_dw1 = fresh(grad_data, dy1), fresh(grad_filter, dy1)
    want_dx2, want_dw2 = fresh(grad_data, dy2), fresh(grad_filter, dy2)
    gdy = _gpu(dy1, rt)
    grad_filter(gdy), grad_data(gdy)        # the descriptor now knows both forms

    # grad-filter first: it leaves grad-data's transform
    taken = _kept_counts()[1]
    np.testing.assert_array_equal(grad_filter(gdy), want_dw1)
    np.testing.assert_array_equal(grad_data(gdy), want_dx1)
    assert _kept_counts()[1] == taken + 1
    # grad-data first
    np.testing.assert_array_equal(grad_data(gdy), want_dx1)
    np.testing.assert_array_equal(grad_filter(gdy), want_dw1)
    assert _kept_counts()[1] == taken + 2
    # dy changes between the two calls
    np.testing.assert_array_equal(grad_filter(gdy), want_dw1)
    gdy[:] = dy2
    np.testing.assert_array_equal(grad_data(gdy), want_dx2)
    gdy[:] = dy1
    np.testing.assert_array_equal(grad_filter(gdy), want_dw1)
    assert _kept_counts()[1] == taken + 2
    # the other call comes with another dy (grad-data first takes what the last grad-filter left for dy1)
    gdy2 = _gpu(dy2, rt)
    np.testing.assert_array_equal(grad_data(gdy), want_dx1)
    assert _kept_counts()[1] == taken + 3
    np.testing.assert_array_equal(grad_data(gdy), want_dx1)      # leaves grad-filter's form of dy1
    np.testing.assert_array_equal(grad_filter(gdy2), want_dw2)
    assert _kept_counts()[1] == taken + 3


# ResNet-50 batch-64 layer shapes, one per kernel family: (C, H, K, R, padding, stride)
FULL_SIZE_LAYERS = [
    (128, 28, 128, 3, "SAME", 1),    # 3x3, Winograd 4x4 tiles
    (64, 56, 64, 3, "SAME", 1),
    (256, 14, 256, 3, "SAME", 1),    # 3x3, Winograd 2x2 tiles
    (512, 7, 512, 3, "SAME", 1),
    (64, 56, 256, 1, "VALID", 1),    # 1x1, 16-byte loaders
    (2048, 7, 512, 1, "VALID", 1),   # 1x1, 49 pixels per image
    (1024, 14, 2048, 1, "VALID", 2), # 1x1 stride 2: gathered forward, scatter grad-data
    (3, 224, 64, 7, "SAME", 2),      # stem
]


@pytest.mark.parametrize("layer", FULL_SIZE_LAYERS, ids=lambda l: "x".join(str(v) for v in l))
def test_conv_adjoint_identities_full_size(rt, layer):
    """<conv(x,w), dy> = <x, dgrad(dy,w)> = <w, wgrad(x,dy)> at full ResNet-50 batch-64
    layer shapes (too large for the CPU oracle in a unit test).  The three kernels
    share no code path beyond the tile engine, so a wrong index in one breaks an
    identity; each convolution is also checked against the float64 oracle on the
    first image and a few output channels."""
    from tinyflow_amd import gpu_op, ndarray
    C, H, K, R, padding, stride = layer
    rng = np.random.RandomState(12)
    x = rng.normal(0, 1, (64, C, H, H)).astype(np.float32)
    w = rng.normal(0, np.sqrt(2.0 / (C * R * R)), (K, C, R, R)).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", padding, stride, stride)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gw, gdy = _gpu(x, rt), _gpu(w, rt), _gpu(dy, rt)
    gy, gdx, gdw = ndarray.empty(out_shape, rt.ctx), ndarray.empty(x.shape, rt.ctx), ndarray.empty(w.shape, rt.ctx)
    gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream)
    gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream)
    gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream)
    y = gy.asnumpy()
    a = np.vdot(y.astype(np.float64), dy.astype(np.float64))
    b = np.vdot(x.astype(np.float64), gdx.asnumpy().astype(np.float64))
    c = np.vdot(w.astype(np.float64), gdw.asnumpy().astype(np.float64))
    assert abs(a - b) <= 1e-4 * abs(a) and abs(a - c) <= 1e-4 * abs(a)
    pad = O.conv_pad(R, padding)
    k_some = slice(0, min(K, 8))
    y_ref = O.conv2d_forward(x[:1].astype(np.float64), w[k_some].astype(np.float64), pad, pad, stride, stride)
    scale = max(1.0, float(np.abs(y_ref).max()))
    np.testing.assert_allclose(y[:1, k_some], y_ref, rtol=1e-3, atol=1e-5 * scale)


# Layers whose launches fold tiles in the kernel: a short k-split whose pieces are added by
# the last workgroup of each tile (forward of 1024 -> 256 at 14x14), and a remainder
# round cut into pieces (forward and grad-data of 512 -> 1024 stride 2, 784 tiles on 256 CUs).
FOLDED_LAYERS = [(64, 1024, 14, 256, 1, 1), (64, 512, 28, 1024, 1, 2), (64, 256, 14, 1024, 1, 1),
                 (64, 512, 7, 2048, 1, 1)]


@pytest.mark.parametrize("layer", FOLDED_LAYERS, ids=lambda l: "x".join(str(v) for v in l))
def test_in_kernel_fold_matches_the_unfolded_launch(rt, monkeypatch, layer):
    """Tiles computed in pieces and added by the last workgroup to arrive must equal the
    same launch without pieces (up to the rounding of a different summation order), on
    every element and on every one of many repetitions: a piece read before it was
    complete, or from a stale cache line, would show as a wrong 64x64 or 128x128 block.
    Repetitions of the folded launch must also agree with each other bit for bit."""
    from tinyflow_amd import gpu_op, ndarray
    N, C, HW, K, R, stride = layer
    rng = np.random.RandomState(parity.stable_seed(layer))
    x = rng.normal(0, 1, (N, C, HW, HW)).astype(np.float32)
    w = rng.normal(0, np.sqrt(2.0 / (C * R * R)), (K, C, R, R)).astype(np.float32)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", "VALID", stride, stride)
    dy = rng.normal(0, 1, out_shape).astype(np.float32)
    gx, gw, gdy = _gpu(x, rt), _gpu(w, rt), _gpu(dy, rt)

    def run():
        gy, gdx, gdw = ndarray.empty(out_shape, rt.ctx), ndarray.empty(x.shape, rt.ctx), ndarray.empty(w.shape, rt.ctx)
        for arr in (gy, gdx, gdw):
            gpu_op.array_set(arr, np.nan, rt.stream)
        assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
        assert gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream) == 0
        assert gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream) == 0
        return gy.asnumpy(), gdx.asnumpy(), gdw.asnumpy()

    monkeypatch.setenv("TINYFLOW_FOLD", "0")
    plain = run()
    monkeypatch.setenv("TINYFLOW_FOLD", "3")
    first = run()
    assert any(not np.array_equal(a, b) for a, b in zip(plain, first)), "no launch of this layer folds anything"
    for a, b, what in zip(plain, first, ("forward", "grad-data", "grad-filter")):
        scale = max(1.0, float(np.abs(a).max()))
        np.testing.assert_allclose(b, a, rtol=1e-4, atol=1e-5 * scale, err_msg=what)
    for _ in range(15):
        again = run()
        for a, b in zip(first, again):
            assert a.tobytes() == b.tobytes()


def test_conv_rejects_mismatched_arrays(rt, capfd):
    from tinyflow_amd import gpu_op, ndarray
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape((2, 3, 8, 8), (4, 3, 3, 3), "NCHW", "SAME", 1, 1)
    x = ndarray.empty((2, 3, 8, 8), rt.ctx)
    w = ndarray.empty((4, 3, 3, 3), rt.ctx)
    bad = ndarray.empty((2, 4, 7, 8), rt.ctx)
    with pytest.raises(RuntimeError):
        gpu_op.convolution_2d_forward(x, w, bad, lst, rt.cudnn, rt.stream)
