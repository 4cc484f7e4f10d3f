"""Known-answer vectors held by the reference's own tests (tests/golden/reference_vectors.json):
the oracle is checked against them on the CPU, the HIP library through the C-ABI on the GPU."""
import json
import os

import numpy as np
import pytest

from oracle import ops as O

with open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")) as f:
    GOLDEN = json.load(f)


def _make(spec, dtype=np.float32):
    if "linspace" in spec:
        a = np.linspace(*spec["linspace"])
    else:
        a = np.full(int(np.prod(spec["shape"])), spec["full"])
    return a.reshape(spec["shape"]).astype(dtype)


def _window_sums(x, r, s):
    n, c, h, w = x.shape
    out = np.zeros((n, 1, h - r + 1, w - s + 1), np.float64)
    for p in range(out.shape[2]):
        for q in range(out.shape[3]):
            out[:, 0, p, q] = x[:, :, p:p + r, q:q + s].astype(np.float64).sum(axis=(1, 2, 3))
    return out


# ----------------------------------------------------------------------- CPU: oracle

def test_oracle_conv1d_vector():
    g = GOLDEN["conv1d_upstream_gradient"]
    y = O.conv2d_forward(_make(g["x"]), _make(g["w"]), 0, 0, 1, 1)
    np.testing.assert_allclose(0.4 * y.reshape(-1), np.array(g["stored"], np.float32), rtol=2e-6)


def test_oracle_conv2d_tiny():
    g = GOLDEN["conv2d_tiny"]
    x, w = _make(g["x"], np.float64), _make(g["w"], np.float64)
    np.testing.assert_allclose(O.conv2d_forward(x, w, 0, 0, 1, 1), 0.001 * _window_sums(x, 3, 3), rtol=1e-12)


def test_oracle_matmul_grad():
    g = GOLDEN["matmul_grad"]
    x2, x3 = np.array(g["x2"], np.float32), np.array(g["x3"], np.float32)
    y = O.matmul(x2, False, x3, False)
    assert np.array_equal(y, np.array(g["y"], np.float32))
    ones = np.ones_like(y)
    assert np.array_equal(O.matmul(ones, False, x3, True), np.array(g["grad_x2"], np.float32))
    assert np.array_equal(O.matmul(x2, True, ones, False), np.array(g["grad_x3"], np.float32))


# ----------------------------------------------------------------- GPU: HIP library

def _conv_on_gpu(rt, x, w, padding):
    from tinyflow_amd import gpu_op, ndarray
    out_shape, cudnnlist = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", padding, 1, 1)
    dx, dw, dy = (ndarray.array(a, rt.ctx) for a in (x, w, np.zeros(out_shape, np.float32)))
    assert gpu_op.convolution_2d_forward(dx, dw, dy, cudnnlist, rt.cudnn, rt.stream) == 0
    return dy.asnumpy()


@pytest.mark.gpu
def test_hip_conv1d_vector(rt):
    g = GOLDEN["conv1d_upstream_gradient"]
    y = _conv_on_gpu(rt, _make(g["x"]), _make(g["w"]), g["padding"])
    np.testing.assert_allclose(0.4 * y.reshape(-1), np.array(g["stored"], np.float32), rtol=1e-5)


@pytest.mark.gpu
def test_hip_conv2d_tiny(rt):
    g = GOLDEN["conv2d_tiny"]
    x = _make(g["x"])
    y = _conv_on_gpu(rt, x, _make(g["w"]), g["padding"])
    np.testing.assert_allclose(y, 0.001 * _window_sums(x, 3, 3), rtol=1e-5)


@pytest.mark.gpu
def test_hip_matmul_grad_and_shapes(rt):
    from tinyflow_amd import gpu_op, ndarray

    def mm(a, ta, b, tb):
        m = a.shape[1] if ta else a.shape[0]
        n = b.shape[0] if tb else b.shape[1]
        out = ndarray.empty((m, n), rt.ctx)
        gpu_op.matrix_multiply(ndarray.array(a, rt.ctx), ta, ndarray.array(b, rt.ctx), tb, out, rt.cublas, rt.stream)
        return out.asnumpy()

    g = GOLDEN["matmul_grad"]
    x2, x3 = np.array(g["x2"], np.float32), np.array(g["x3"], np.float32)
    y = mm(x2, False, x3, False)
    assert np.array_equal(y, np.array(g["y"], np.float32))
    ones = np.ones_like(y)
    assert np.array_equal(mm(ones, False, x3, True), np.array(g["grad_x2"], np.float32))
    assert np.array_equal(mm(x2, True, ones, False), np.array(g["grad_x3"], np.float32))
    rng = np.random.RandomState(0)
    for case in GOLDEN["matmul_shapes"]["cases"]:
        a = rng.uniform(0, 10, case["A"]).astype(np.float32)
        b = rng.uniform(0, 10, case["B"]).astype(np.float32)
        want = (a.T if case["transA"] else a).astype(np.float64) @ (b.T if case["transB"] else b).astype(np.float64)
        np.testing.assert_allclose(mm(a, case["transA"], b, case["transB"]), want, rtol=GOLDEN["matmul_shapes"]["rtol"])
