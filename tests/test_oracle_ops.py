"""Pins the CPU oracle (oracle/ops.py) -- runs without a GPU.

Every oracle function is checked against something it does not share code with:
the reference's own known-answer cases, closed forms, a brute-force C
implementation (oracle/conv_direct.c), finite differences, mathematical
invariants, and torch's CPU kernels as a library cross-check.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import direct as D
from oracle import ops as O


# ---------------------------------------------------------------- reference-held cases

def test_matmul_reference_shapes_and_transposes():
    """tests/test_gpu_op.py:103-131: C = A B, A B^T, A^T B^T against np.dot."""
    rng = np.random.RandomState(0)
    x = rng.uniform(0, 10, (500, 700)).astype(np.float32)
    y = rng.uniform(0, 10, (700, 1000)).astype(np.float32)
    np.testing.assert_allclose(O.matmul(x, False, y, False), np.dot(x, y), rtol=1e-5)
    x = rng.uniform(0, 10, (1000, 700)).astype(np.float32)
    y = rng.uniform(0, 10, (500, 700)).astype(np.float32)
    np.testing.assert_allclose(O.matmul(x, False, y, True), np.dot(x, np.transpose(y)), rtol=1e-5)
    x = rng.uniform(0, 10, (700, 500)).astype(np.float32)
    y = rng.uniform(0, 10, (1000, 700)).astype(np.float32)
    np.testing.assert_allclose(O.matmul(x, True, y, True), np.dot(np.transpose(x), np.transpose(y)), rtol=1e-5)


def test_matmul_gradients_reference_integer_case():
    """tests/autodiff_test.py:188-208: y = x2 x3 with a ones upstream gives
    dx2 = 1 x3^T and dx3 = x2^T 1."""
    x2 = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    x3 = np.array([[7, 8, 9], [10, 11, 12]], np.float32)
    ones = np.ones((3, 3), np.float32)
    d2, d3 = O.matmul_gradients(x2, False, x3, False, ones)
    assert np.array_equal(d2, np.matmul(ones, x3.T)) and np.array_equal(d3, np.matmul(x2.T, ones))


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_matmul_gradients_by_finite_differences(ta, tb):
    rng = np.random.RandomState(1)
    a = rng.normal(0, 1, (4, 3) if ta else (3, 4))
    b = rng.normal(0, 1, (5, 4) if tb else (4, 5))
    dy = rng.normal(0, 1, (3, 5))
    da, db = O.matmul_gradients(a, ta, b, tb, dy)
    f = lambda a_, b_: np.sum(O.matmul(a_, ta, b_, tb) * dy)
    for arr, grad, which in ((a, da, 0), (b, db, 1)):
        num = np.zeros_like(arr)
        for idx in np.ndindex(arr.shape):
            e = np.zeros_like(arr)
            e[idx] = 1e-6
            num[idx] = ((f(a + e, b) - f(a - e, b)) if which == 0 else (f(a, b + e) - f(a, b - e))) / 2e-6
        np.testing.assert_allclose(grad, num, rtol=1e-6, atol=1e-8)


def test_relu_and_gradient_mask_rule():
    """tests/test_gpu_op.py:134-155: relu = max(x,0); gradient = (x > 0) * g -- zero at x == 0."""
    x = np.array([-2.0, -0.0, 0.0, 1e-30, 3.0], np.float32)
    g = np.array([1.0, 2.0, 3.0, 4.0, 5.0], np.float32)
    assert np.array_equal(O.relu(x), np.maximum(x, 0))
    assert np.array_equal(O.relu_gradient(x, g), np.array([0, 0, 0, 4, 5], np.float32))
    # the reference's numpy branch would give 0.5 * g at zero; the CUDA kernel and its test give 0
    assert O.relu_gradient(np.zeros(1, np.float32), np.ones(1, np.float32))[0] == 0


def test_softmax_and_cross_entropy_reference_formulas():
    """tests/test_gpu_op.py:158-182."""
    rng = np.random.RandomState(2)
    y = rng.uniform(-5, 5, (400, 1000)).astype(np.float64)
    sm = O.softmax(y)
    np.testing.assert_allclose(sm.sum(axis=1), 1.0, rtol=1e-12)
    np.testing.assert_allclose(sm, torch.softmax(torch.from_numpy(y), 1).numpy(), rtol=1e-10)
    y_ = rng.uniform(-5, 5, (400, 1000))
    expect = np.mean(-np.sum(y_ * np.log(sm), axis=1), keepdims=True)
    np.testing.assert_allclose(O.softmax_cross_entropy(y, y_), expect, rtol=1e-12)
    assert O.softmax_cross_entropy(y, y_).shape == (1,)


def test_softmax_cross_entropy_gradient_has_no_batch_division():
    """autodiff.py:701-713: the loss is a batch MEAN but the gradient is softmax - y_,
    i.e. N times the true derivative of the loss."""
    rng = np.random.RandomState(3)
    N, C = 6, 5
    y = rng.normal(0, 1, (N, C))
    y_ = np.eye(C)[rng.randint(0, C, N)]
    g = O.softmax_cross_entropy_gradient(y, y_, 1.0)
    np.testing.assert_allclose(g.sum(axis=1), 0, atol=1e-12)   # one-hot labels: rows sum to zero
    num = np.zeros_like(y)
    for idx in np.ndindex(y.shape):
        e = np.zeros_like(y)
        e[idx] = 1e-6
        num[idx] = (O.softmax_cross_entropy(y + e, y_)[0] - O.softmax_cross_entropy(y - e, y_)[0]) / 2e-6
    np.testing.assert_allclose(g, N * num, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(O.softmax_cross_entropy_gradient(y, y_, 0.25), 0.25 * g)


def test_elementwise_and_reductions_reference_cases():
    """tests/test_gpu_op.py:5-100."""
    rng = np.random.RandomState(4)
    x = rng.uniform(0, 10, (500, 200)).astype(np.float32)
    y = rng.uniform(0, 10, (500, 200)).astype(np.float32)
    assert np.array_equal(O.add(x, y), x + y) and np.array_equal(O.multiply(x, y), x * y)
    assert np.array_equal(O.add_by_const(x, 0.25), x + np.float32(0.25))
    assert np.array_equal(O.multiply_by_const(x, 3.5), x * np.float32(3.5))
    assert np.array_equal(O.array_set((10, 3), 1.0), np.ones((10, 3), np.float32))
    z = rng.uniform(0, 20, (500, 200, 100)).astype(np.float32)
    np.testing.assert_allclose(O.reduce_sum_axis_zero(z), np.sum(z, axis=0), rtol=1e-6)
    b = rng.uniform(0, 1, (200, 300)).astype(np.float32)
    assert np.array_equal(O.broadcast_to_trailing(b, (130, 200, 300)), np.broadcast_to(b, (130, 200, 300)))
    c = np.arange(3, dtype=np.float32)
    out = O.broadcast_to_channel(c, (2, 3, 4, 5))
    assert all(np.all(out[:, i] == i) for i in range(3))
    dy = rng.normal(0, 1, (4, 3, 5, 6))
    np.testing.assert_allclose(O.bias_gradient(dy, "NCHW"), [dy[:, i].sum() for i in range(3)], rtol=1e-12)
    np.testing.assert_allclose(O.bias_gradient(dy[:, :, 0, 0], "NHWC"), dy[:, :, 0, 0].sum(axis=0), rtol=1e-12)
    w = rng.normal(0, 1, (7, 7)).astype(np.float32)
    assert np.array_equal(O.sgd_update(w, w * 2, 0.5), w - np.float32(0.5) * (w * 2))


def test_conv1d_upstream_vector_held_by_the_reference():
    """tests/test_gpu_op.py:219-229 holds [0.07676768, 0.23838384, 0.40000007,
    0.5616162, 0.7232323]: the upstream gradient 2y/5 of loss = y^T y / 5 for the VALID
    conv of x = linspace(0,100,100).reshape(5,1,20) with w = 0.001*ones(1,1,20)
    (tests/autodiff_test.py:299-311).  As a 2-D conv with H = 1."""
    x = np.linspace(0, 100, 100).reshape(5, 1, 1, 20).astype(np.float32)
    w = (np.ones((1, 1, 1, 20)) * 0.001).astype(np.float32)
    y = O.conv2d_forward(x, w, 0, 0, 1, 1)
    assert y.shape == (5, 1, 1, 1)
    held = np.array([0.07676768, 0.23838384, 0.40000007, 0.5616162, 0.7232323], np.float32)
    np.testing.assert_allclose(2.0 / 5.0 * y.reshape(5), held, rtol=2e-6)


def test_tiny_conv2d_case_of_the_reference():
    """tests/autodiff_test.py:335-343: x = linspace(0,100,80) -> (5,1,4,4), w = 0.001*ones(1,1,3,3):
    every output is 0.001 * (sum of its 3x3 window)."""
    x = np.linspace(0, 100, 80).reshape(5, 1, 4, 4)
    w = np.ones((1, 1, 3, 3)) * 0.001
    y = O.conv2d_forward(x, w, 0, 0, 1, 1)
    assert y.shape == (5, 1, 2, 2)
    for n in range(5):
        for p in range(2):
            for q in range(2):
                assert abs(y[n, 0, p, q] - 0.001 * x[n, 0, p:p + 3, q:q + 3].sum()) < 1e-12


# ---------------------------------------------------------------------------- convolution

CONV_CASES = [
    # N, C, H, W, K, R, S, padding, u, v
    (2, 3, 7, 6, 4, 3, 3, "SAME", 1, 1),
    (2, 3, 7, 6, 4, 3, 3, "VALID", 1, 1),
    (1, 2, 9, 9, 3, 5, 5, "SAME", 1, 1),
    (2, 2, 8, 8, 3, 1, 1, "VALID", 2, 2),
    (2, 4, 9, 7, 2, 1, 1, "VALID", 2, 3),
    (1, 3, 12, 12, 5, 7, 7, "SAME", 2, 2),
    (2, 3, 10, 11, 4, 3, 2, "SAME", 2, 1),
    (3, 1, 5, 5, 1, 3, 3, "VALID", 2, 2),
    (1, 1, 1, 1, 1, 1, 1, "VALID", 1, 1),
]


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c)))
def test_conv_against_brute_force_c(case):
    N, C, H, W, K, R, S, padding, u, v = case
    rng = np.random.RandomState(5)
    x = rng.normal(0, 1, (N, C, H, W))
    w = rng.normal(0, 1, (K, C, R, S))
    ph, pw = O.conv_pad(R, padding), O.conv_pad(S, padding)
    y = O.conv2d_forward(x, w, ph, pw, u, v)
    np.testing.assert_allclose(y, D.forward(x, w, padding, u, v), rtol=1e-12, atol=1e-12)
    dy = rng.normal(0, 1, y.shape)
    np.testing.assert_allclose(O.conv2d_backward_data(dy, w, x.shape, ph, pw, u, v),
                               D.backward_data(dy, w, x.shape, padding, u, v), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(O.conv2d_backward_filter(x, dy, w.shape, ph, pw, u, v),
                               D.backward_filter(x, dy, w.shape, padding, u, v), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: "x".join(map(str, c)))
def test_conv_adjoint_identities_and_torch(case):
    N, C, H, W, K, R, S, padding, u, v = case
    rng = np.random.RandomState(6)
    x = rng.normal(0, 1, (N, C, H, W))
    w = rng.normal(0, 1, (K, C, R, S))
    ph, pw = O.conv_pad(R, padding), O.conv_pad(S, padding)
    y = O.conv2d_forward(x, w, ph, pw, u, v)
    dy = rng.normal(0, 1, y.shape)
    dx = O.conv2d_backward_data(dy, w, x.shape, ph, pw, u, v)
    dw = O.conv2d_backward_filter(x, dy, w.shape, ph, pw, u, v)
    # <conv(x,w), dy> = <x, dgrad(dy,w)> = <w, wgrad(x,dy)>
    a, b, c = np.vdot(y, dy), np.vdot(x, dx), np.vdot(w, dw)
    assert abs(a - b) < 1e-9 * max(1, abs(a)) and abs(a - c) < 1e-9 * max(1, abs(a))
    # library cross-check
    tx = torch.from_numpy(x).requires_grad_(True)
    tw = torch.from_numpy(w).requires_grad_(True)
    ty = F.conv2d(tx, tw, stride=(u, v), padding=(ph, pw))
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-10, atol=1e-10)
    ty.backward(torch.from_numpy(dy))
    np.testing.assert_allclose(dx, tx.grad.numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(dw, tw.grad.numpy(), rtol=1e-10, atol=1e-10)


def test_conv_1x1_is_a_matmul():
    rng = np.random.RandomState(7)
    x = rng.normal(0, 1, (3, 5, 4, 6))
    w = rng.normal(0, 1, (7, 5, 1, 1))
    y = O.conv2d_forward(x, w, 0, 0, 1, 1)
    ref = np.einsum("kc,nchw->nkhw", w[:, :, 0, 0], x)
    np.testing.assert_allclose(y, ref, rtol=1e-12)


def test_conv_output_extent_matches_cudnn_formula():
    """out = 1 + (in + 2*pad - k) / stride; "SAME" = symmetric k//2 (gpu_op.cu:2081-2087)."""
    assert O.conv_pad(7, "SAME") == 3 and O.conv_pad(5, "SAME") == 2 and O.conv_pad(1, "SAME") == 0
    assert O.conv_pad(3, "VALID") == 0
    assert O.conv_out_extent(224, 7, 3, 2) == 112
    assert O.conv_out_extent(56, 1, 0, 2) == 28
    assert O.conv_out_extent(28, 5, 2, 1) == 28 and O.conv_out_extent(14, 5, 0, 1) == 10
    assert O.conv_out_extent(4, 2, 1, 1) == 5  # even filter with "SAME" grows the map, as in the reference


# ------------------------------------------------------------------------------- pooling

def _max_pool_loops(x, dy, fh, fw, ph, pw, u, v):
    N, C, H, W = x.shape
    P, Q = O.pool_out_extent(H, fh, ph, u), O.pool_out_extent(W, fw, pw, v)
    y = np.zeros((N, C, P, Q))
    dx = np.zeros_like(x)
    for n in range(N):
        for c in range(C):
            for p in range(P):
                for q in range(Q):
                    best, arg = -np.inf, None
                    for r in range(fh):
                        for s in range(fw):
                            h, w = p * u + r - ph, q * v + s - pw
                            if 0 <= h < H and 0 <= w < W and x[n, c, h, w] > best:  # strict: first max wins
                                best, arg = x[n, c, h, w], (h, w)
                    y[n, c, p, q] = best
                    dx[n, c, arg[0], arg[1]] += dy[n, c, p, q]
    return y, dx


POOL_CASES = [(2, 2, 0, 0, 2, 2), (3, 3, 1, 1, 2, 2), (3, 3, 0, 0, 2, 2), (3, 2, 1, 0, 2, 1), (1, 1, 0, 0, 1, 1)]


@pytest.mark.parametrize("geo", POOL_CASES, ids=str)
@pytest.mark.parametrize("ties", [False, True])
def test_max_pool_against_loops(geo, ties):
    fh, fw, ph, pw, u, v = geo
    rng = np.random.RandomState(8)
    x = rng.normal(0, 1, (2, 3, 9, 8))
    if ties:
        x = np.maximum(np.round(x), 0)
    y = O.max_pool_forward(x, fh, fw, ph, pw, u, v)
    dy = rng.normal(0, 1, y.shape)
    y_ref, dx_ref = _max_pool_loops(x, dy, fh, fw, ph, pw, u, v)
    assert np.array_equal(y, y_ref)
    dx = O.max_pool_backward(x, dy, fh, fw, ph, pw, u, v)
    np.testing.assert_allclose(dx, dx_ref, rtol=1e-12, atol=1e-12)
    assert abs(dx.sum() - dy.sum()) < 1e-9
    if not ties:
        ty = F.max_pool2d(torch.from_numpy(x), (fh, fw), (u, v), (ph, pw))
        assert np.array_equal(y, ty.numpy())


@pytest.mark.parametrize("geo", POOL_CASES + [(7, 7, 0, 0, 1, 1)], ids=str)
def test_avg_pool_counts_padding(geo):
    fh, fw, ph, pw, u, v = geo
    rng = np.random.RandomState(9)
    x = rng.normal(0, 1, (2, 3, 9, 8))
    tx = torch.from_numpy(x).requires_grad_(True)
    ty = F.avg_pool2d(tx, (fh, fw), (u, v), (ph, pw), count_include_pad=True)
    y = O.avg_pool_forward(x, fh, fw, ph, pw, u, v)
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-12, atol=1e-12)
    dy = rng.normal(0, 1, y.shape)
    ty.backward(torch.from_numpy(dy))
    np.testing.assert_allclose(O.avg_pool_backward(x.shape, dy, fh, fw, ph, pw, u, v), tx.grad.numpy(),
                               rtol=1e-12, atol=1e-12)


def test_pool_output_extent():
    assert O.pool_out_extent(112, 3, 1, 2) == 56 and O.pool_out_extent(112, 3, 0, 2) == 55
    assert O.pool_out_extent(28, 2, 0, 2) == 14 and O.pool_out_extent(7, 7, 0, 1) == 1


# ---------------------------------------------------------------------------- activation

@pytest.mark.parametrize("mode", ["relu", "sigmoid", "tanh", "softmax"])
def test_activation_backward_by_finite_differences(mode):
    rng = np.random.RandomState(10)
    x = rng.normal(0, 1, (3, 2, 2, 2))
    x[np.abs(x) < 0.05] += 0.2   # keep clear of the relu kink
    dy = rng.normal(0, 1, x.shape)
    y = O.activation_forward(x, mode)
    dx = O.activation_backward(x, y, dy, mode)
    num = np.zeros_like(x)
    for idx in np.ndindex(x.shape):
        e = np.zeros_like(x)
        e[idx] = 1e-6
        num[idx] = np.sum((O.activation_forward(x + e, mode) - O.activation_forward(x - e, mode)) * dy) / 2e-6
    np.testing.assert_allclose(dx, num, rtol=1e-6, atol=1e-8)
    if mode == "softmax":
        np.testing.assert_allclose(y.reshape(3, -1).sum(axis=1), 1.0, rtol=1e-12)


# ---------------------------------------------------------------------------- batch norm

@pytest.mark.parametrize("shape", [(8, 3, 5, 4), (16, 2, 1, 1), (4, 6, 3, 3)], ids=str)
def test_batch_norm_spatial_against_torch(shape):
    rng = np.random.RandomState(11)
    x = rng.normal(1, 2, shape)
    dy = rng.normal(0, 1, shape)
    tx = torch.from_numpy(x).requires_grad_(True)
    ty = F.batch_norm(tx, None, None, None, None, True, 0.0, O.BN_EPS)
    y, mean, istd = O.batch_norm_forward(x, "spatial")
    np.testing.assert_allclose(y, ty.detach().numpy(), rtol=1e-10, atol=1e-10)
    ty.backward(torch.from_numpy(dy))
    np.testing.assert_allclose(O.batch_norm_backward(x, dy, "spatial", mean, istd), tx.grad.numpy(),
                               rtol=1e-9, atol=1e-10)


@pytest.mark.parametrize("shape", [(8, 3, 5, 4), (16, 2, 1, 1)], ids=str)
def test_batch_norm_per_activation_against_torch(shape):
    """Per-activation statistics = spatial statistics of the array viewed as (N, C*H*W, 1, 1)."""
    rng = np.random.RandomState(12)
    x = rng.normal(1, 2, shape)
    dy = rng.normal(0, 1, shape)
    flat = (shape[0], int(np.prod(shape[1:])), 1, 1)
    tx = torch.from_numpy(x.reshape(flat)).requires_grad_(True)
    ty = F.batch_norm(tx, None, None, None, None, True, 0.0, O.BN_EPS)
    y, mean, istd = O.batch_norm_forward(x, "pre_activation")
    assert mean.shape == (1,) + shape[1:]
    np.testing.assert_allclose(y.reshape(flat), ty.detach().numpy(), rtol=1e-10, atol=1e-10)
    ty.backward(torch.from_numpy(dy.reshape(flat)))
    np.testing.assert_allclose(O.batch_norm_backward(x, dy, "pre_activation").reshape(flat), tx.grad.numpy(),
                               rtol=1e-9, atol=1e-10)


@pytest.mark.parametrize("mode", ["pre_activation", "spatial"])
def test_batch_norm_closed_form_and_invariants(mode):
    rng = np.random.RandomState(13)
    x = rng.normal(0, 3, (32, 4, 3, 3))
    dy = rng.normal(0, 1, x.shape)
    axes = (0,) if mode == "pre_activation" else (0, 2, 3)
    y, mean, istd = O.batch_norm_forward(x, mode)
    np.testing.assert_allclose(mean, x.mean(axis=axes, keepdims=True))
    np.testing.assert_allclose(istd, 1 / np.sqrt(x.var(axis=axes, keepdims=True) + 1e-5))   # biased variance
    np.testing.assert_allclose(y.mean(axis=axes), 0, atol=1e-12)
    dx = O.batch_norm_backward(x, dy, mode)
    np.testing.assert_allclose(dx.sum(axis=axes), 0, atol=1e-10)
    m = np.prod([x.shape[a] for a in axes])
    expect = istd / m * (dy * y).sum(axis=axes, keepdims=True) * (m - (y * y).sum(axis=axes, keepdims=True))
    np.testing.assert_allclose((dx * y).sum(axis=axes, keepdims=True), expect, atol=1e-10)


def test_adam_and_cross_formulas():
    """gpu_op.cu:4461-4506 (Adam) and :4538-4573 (cross) written out by hand."""
    rng = np.random.RandomState(14)
    w, m, v, g = (rng.uniform(0.1, 1, 9) for _ in range(4))
    m2, v2 = O.adam_mv(m, v, g, 0.9, 0.999)
    np.testing.assert_allclose(m2, 0.9 * m + 0.1 * g)
    np.testing.assert_allclose(v2, 0.999 * v + 0.001 * g * g)
    np.testing.assert_allclose(O.adam_update(w, m, v, 0.9, 0.999, 1e-8, 0.01),
                               w - 0.01 * (m / 0.1) / (np.sqrt(v / 0.001) + 1e-8))
    x, y = rng.uniform(0.1, 1, (4, 3)), np.eye(3)[[0, 2, 1, 1]]
    np.testing.assert_allclose(O.cross(x, y, 0.5), -0.5 * y * np.log(x))
    np.testing.assert_allclose(O.cross_backward(x, y, np.ones_like(x), 0.5), -0.5 * y / x)


# ------------------------------------------------------- dropout, concatenation

PHILOX_KAT = [
    # counter, key, output: known-answer vectors of philox4x32-10 published with the Random123 library
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


def test_philox_known_answers():
    for ctr, key, want in PHILOX_KAT:
        got = O.philox4x32_10(np.array(ctr, dtype=np.uint32), key)
        assert tuple(int(v) for v in got) == want
    # vectorised over a leading axis
    ctrs = np.array([k[0] for k in PHILOX_KAT[:1]] * 3, dtype=np.uint32)
    assert O.philox4x32_10(ctrs, (0, 0)).shape == (3, 4)


@pytest.mark.parametrize("p", [0.0, 0.1, 0.5, 0.9])
def test_dropout_mask_rate_scale_and_backward(p):
    rng = np.random.RandomState(3)
    x = rng.normal(0, 1, (64, 1000)).astype(np.float32)
    out, keep = O.dropout_forward(x, p, seed=11)
    n = x.size
    assert abs(keep.mean() - (1 - p)) < 4 * np.sqrt(p * (1 - p) / n) + 1e-12
    assert np.array_equal(out != 0, keep & (x != 0))
    np.testing.assert_array_equal(out[keep], x[keep] * (np.float32(1) / (np.float32(1) - np.float32(p))))
    dy = rng.normal(0, 1, x.shape).astype(np.float32)
    dx = O.dropout_backward(dy, keep, p)
    # same mask, same scale: <dropout(x), dy> == <x, dropout_backward(dy)>
    assert abs(np.vdot(out.astype(np.float64), dy) - np.vdot(x.astype(np.float64), dx)) < 1e-6 * n
    # a different seed gives a different mask, the same seed the same mask
    assert np.array_equal(keep, O.dropout_forward(x, p, seed=11)[1])
    if 0 < p < 1:
        assert not np.array_equal(keep, O.dropout_forward(x, p, seed=12)[1])


def test_concat_and_its_gradients():
    rng = np.random.RandomState(4)
    a = rng.normal(0, 1, (3, 2, 4, 5)).astype(np.float32)
    b = rng.normal(0, 1, (3, 7, 4, 5)).astype(np.float32)
    out = O.concat_forward(a, b)
    assert out.shape == (3, 9, 4, 5)
    # the reference kernel's index arithmetic (gpu_op.cu:967-979), element by element
    count1, count2 = a[0].size, b[0].size
    flat = out.reshape(-1)
    for index in range(0, flat.size, 37):
        i1, i2 = index % (count1 + count2), index // (count1 + count2)
        want = a.reshape(-1)[i2 * count1 + i1] if i1 < count1 else b.reshape(-1)[i2 * count2 + i1 - count1]
        assert flat[index] == want
    da, db = O.concat_backward(a, b, out)
    assert np.array_equal(da, a) and np.array_equal(db, b)
