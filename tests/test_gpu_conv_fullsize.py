"""Convolution forward / grad-data / grad-filter at the full layer shapes of the
ResNet-50 (batch 64) and VGG-16 (batch 32) configurations.

The CPU oracle cannot evaluate these shapes inside a unit test, so parity is
checked on a random sample of output elements: each sampled element is computed
by brute force from the definition in float64 (the same definition
oracle/conv_direct.c and oracle.ops.conv2d_* implement) and compared with the HIP
result within rtol 1e-3 / atol 1e-5 (relative to the largest sampled magnitude).
Each sampled element is also evaluated in float32 on the CPU in two ways, and the
HIP error against float64 is held to a multiple of each evaluation's own error:
  * a plain loop, acc += a*b term after term (numpy's sequential float32 cumsum):
    factor K_SEQ for the direct form, K_SEQ_WINOGRAD where the planner picked a
    Winograd form.  This is the arithmetic of one fp32 accumulator, which is also
    what a matrix-core contraction keeps per output element;
  * one BLAS dot product over the same terms (how numpy's fp32 matmul accumulates):
    factors K_BLAS / K_BLAS_WINOGRAD.  BLAS spreads a reduction over 16-32 SIMD
    partial sums, so its rounding error grows with the square root of a 16-32 times
    shorter chain; a single-accumulator reduction of the same length cannot match
    it, hence the larger factor.
The tile shapes and split counts the library picks depend on the problem size, so
these are not the code paths the reduced-size cases take.

RESNET50_REFERENCE_STEM holds the layer shapes the reference's own ResNet-50 script
produces (pycode/tinyflow/ResNet50_test_leo.py:219-226: a pad-3 1x1 max-pool in front
of an unpadded 7x7/2 stem and a pad-0 3x3/2 pool give 55x55 stage-2 maps): odd row
lengths, so no 16-byte loaders, Winograd edge tiles on every map and a 55 -> 28
stride-2 grid.
"""
import numpy as np
import pytest

from oracle import ops as O
import parity

K_SEQ, K_SEQ_WINOGRAD = 3.0, 4.0
K_BLAS, K_BLAS_WINOGRAD = 20.0, 32.0

# (N, C, HW, K, R, stride, padding)
RESNET50_B64 = [
    (64, 3, 224, 64, 7, 2, "SAME"), (64, 64, 56, 64, 1, 1, "VALID"), (64, 64, 56, 64, 3, 1, "SAME"),
    (64, 64, 56, 256, 1, 1, "VALID"), (64, 256, 56, 64, 1, 1, "VALID"), (64, 256, 56, 128, 1, 2, "VALID"),
    (64, 128, 28, 128, 3, 1, "SAME"), (64, 128, 28, 512, 1, 1, "VALID"), (64, 256, 56, 512, 1, 2, "VALID"),
    (64, 512, 28, 128, 1, 1, "VALID"), (64, 512, 28, 256, 1, 2, "VALID"), (64, 256, 14, 256, 3, 1, "SAME"),
    (64, 256, 14, 1024, 1, 1, "VALID"), (64, 512, 28, 1024, 1, 2, "VALID"), (64, 1024, 14, 256, 1, 1, "VALID"),
    (64, 1024, 14, 512, 1, 2, "VALID"), (64, 512, 7, 512, 3, 1, "SAME"), (64, 512, 7, 2048, 1, 1, "VALID"),
    (64, 1024, 14, 2048, 1, 2, "VALID"), (64, 2048, 7, 512, 1, 1, "VALID"),
]
# 230x230 padded image -> 7x7/2 unpadded -> 112x112 -> 3x3/2 unpadded pool -> 55x55
RESNET50_REFERENCE_STEM = [
    (64, 3, 230, 64, 7, 2, "VALID"), (64, 64, 55, 64, 1, 1, "VALID"), (64, 64, 55, 64, 3, 1, "SAME"),
    (64, 64, 55, 256, 1, 1, "VALID"), (64, 256, 55, 64, 1, 1, "VALID"), (64, 256, 55, 128, 1, 2, "VALID"),
    (64, 256, 55, 512, 1, 2, "VALID"),
]
VGG16_B32 = [
    (32, 3, 224, 64, 3, 1, "SAME"), (32, 64, 224, 64, 3, 1, "SAME"), (32, 64, 112, 128, 3, 1, "SAME"),
    (32, 128, 112, 128, 3, 1, "SAME"), (32, 128, 56, 256, 3, 1, "SAME"), (32, 256, 56, 256, 3, 1, "SAME"),
    (32, 256, 28, 512, 3, 1, "SAME"), (32, 512, 28, 512, 3, 1, "SAME"), (32, 512, 14, 512, 3, 1, "SAME"),
]


def _dot(a, b, dtype):
    """One dot product over the given terms, accumulated in `dtype` (BLAS for float32);
    dtype "seq32": float32 products added one after the other into one accumulator."""
    if dtype == "seq32":
        prod = np.ascontiguousarray(a, dtype=np.float32).ravel() * np.ascontiguousarray(b, dtype=np.float32).ravel()
        return float(np.cumsum(prod, dtype=np.float32)[-1]) if prod.size else 0.0
    return float(np.dot(np.ascontiguousarray(a, dtype=dtype).ravel(), np.ascontiguousarray(b, dtype=dtype).ravel()))


def _sampled_references(x, w, dy, pad, u, rng, n_out=400, n_dx=400, n_dw=48, dtype=np.float64):
    """Brute-force values, accumulated in `dtype`, of randomly chosen elements of y, dx and dw."""
    N, C, H, W = x.shape
    K, _, R, S = w.shape
    P, Q = dy.shape[2], dy.shape[3]
    xp = np.pad(x, ((0, 0), (0, 0), (pad, pad + u), (pad, pad + u)))   # zero border, room for strided slices
    w64 = w.astype(np.float32 if dtype == "seq32" else dtype)

    y_idx = np.stack([rng.randint(0, m, n_out) for m in (N, K, P, Q)], axis=1)
    y_ref = np.empty(n_out)
    for i, (n, k, p, q) in enumerate(y_idx):
        y_ref[i] = _dot(xp[n, :, p * u:p * u + R, q * u:q * u + S], w64[k], dtype)

    dx_idx = np.stack([rng.randint(0, m, n_dx) for m in (N, C, H, W)], axis=1)
    dx_ref = np.zeros(n_dx)
    for i, (n, c, h, ww) in enumerate(dx_idx):
        lhs, rhs = [], []
        for r in range(R):
            ph = h + pad - r
            if ph % u or not 0 <= ph // u < P:
                continue
            for s in range(S):
                qw = ww + pad - s
                if qw % u or not 0 <= qw // u < Q:
                    continue
                lhs.append(dy[n, :, ph // u, qw // u])
                rhs.append(w64[:, c, r, s])
        dx_ref[i] = _dot(np.concatenate(lhs), np.concatenate(rhs), dtype) if lhs else 0.0

    dw_idx = np.stack([rng.randint(0, m, n_dw) for m in (K, C, R, S)], axis=1)
    dw_ref = np.empty(n_dw)
    for i, (k, c, r, s) in enumerate(dw_idx):
        taps = xp[:, c, r:r + u * P:u, s:s + u * Q:u]
        dw_ref[i] = _dot(dy[:, k], taps, dtype)
    return (y_idx, y_ref), (dx_idx, dx_ref), (dw_idx, dw_ref)


def _check(got, idx, ref, ref_blas32, ref_seq32, what, plan, case):
    picked = got[tuple(idx.T)]
    scale = max(1.0, float(np.abs(ref).max()))
    np.testing.assert_allclose(picked, ref, rtol=1e-3, atol=1e-5 * scale, err_msg=what)
    form = "winograd F(4x4)" if "winograd4x4" in plan else "winograd F(2x2)" if "winograd" in plan else "direct"
    family = "conv %s, %s, full-size layers" % (what, form)
    parity.compare(picked, ref, ref_seq32, family + ", vs sequential fp32 loop", "%s %s" % (what, (case,)),
                   K_SEQ if form == "direct" else K_SEQ_WINOGRAD)
    parity.compare(picked, ref, ref_blas32, family + ", vs fp32 BLAS dot", "%s %s" % (what, (case,)),
                   K_BLAS if form == "direct" else K_BLAS_WINOGRAD)


def _plan(lst, which):
    import ctypes
    from tinyflow_amd import _base
    buf = ctypes.create_string_buffer(256)
    assert _base._LIB.DLGpuConvolutionDescribeKernel(lst, which, buf, 256, None) == 0
    return buf.value.decode()


@pytest.mark.gpu
@pytest.mark.parametrize("case", RESNET50_B64 + RESNET50_REFERENCE_STEM + VGG16_B32,
                         ids=lambda c: "x".join(str(v) for v in c))
def test_full_size_layer_against_sampled_brute_force(rt, case):
    from tinyflow_amd import gpu_op, ndarray
    N, C, HW, K, R, u, padding = case
    gen = np.random.default_rng(parity.stable_seed(case))
    rng = np.random.RandomState(parity.stable_seed(case))
    x = gen.standard_normal((N, C, HW, HW), dtype=np.float32)
    w = gen.standard_normal((K, C, R, R), dtype=np.float32) * np.float32(np.sqrt(2.0 / (C * R * R)))
    pad = O.conv_pad(R, padding)
    out_shape, lst = gpu_op.convolution_2d_forward_get_out_shape(x.shape, w.shape, "NCHW", padding, u, u)
    assert out_shape == (N, K, O.conv_out_extent(HW, R, pad, u), O.conv_out_extent(HW, R, pad, u))
    dy = gen.standard_normal(out_shape, dtype=np.float32)

    gx, gw, gdy = (ndarray.array(a, rt.ctx) for a in (x, w, dy))
    gy, gdx, gdw = ndarray.empty(out_shape, rt.ctx), ndarray.empty(x.shape, rt.ctx), ndarray.empty(w.shape, rt.ctx)
    for arr in (gy, gdx, gdw):
        gpu_op.array_set(arr, np.nan, rt.stream)   # every element must be written
    assert gpu_op.convolution_2d_forward(gx, gw, gy, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, rt.cudnn, rt.stream) == 0
    assert gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, rt.cudnn, rt.stream) == 0
    y, dx, dw = gy.asnumpy(), gdx.asnumpy(), gdw.asnumpy()
    assert not np.isnan(y).any() and not np.isnan(dx).any() and not np.isnan(dw).any()

    refs = _sampled_references(x, w, dy, pad, u, rng)
    # the same sample accumulated in float32: by BLAS, and term after term
    refs32 = _sampled_references(x, w, dy, pad, u, np.random.RandomState(parity.stable_seed(case)), dtype=np.float32)
    seq32 = _sampled_references(x, w, dy, pad, u, np.random.RandomState(parity.stable_seed(case)), dtype="seq32")
    for which, (got, what) in enumerate(((y, "forward"), (dx, "grad-data"), (dw, "grad-filter"))):
        assert np.array_equal(refs[which][0], refs32[which][0]) and np.array_equal(refs[which][0], seq32[which][0])
        _check(got, refs[which][0], refs[which][1], refs32[which][1], seq32[which][1], what, _plan(lst, which), case)


def test_sampled_brute_force_agrees_with_the_oracle():
    """The sampler itself, against oracle.ops on a shape the oracle can evaluate."""
    rng = np.random.RandomState(0)
    for (N, C, HW, K, R, u, padding) in [(2, 3, 9, 4, 3, 1, "SAME"), (2, 4, 11, 3, 1, 2, "VALID"),
                                         (1, 2, 12, 3, 7, 2, "SAME")]:
        x = rng.normal(0, 1, (N, C, HW, HW)).astype(np.float32)
        w = rng.normal(0, 1, (K, C, R, R)).astype(np.float32)
        pad = O.conv_pad(R, padding)
        y = O.conv2d_forward(x.astype(np.float64), w.astype(np.float64), pad, pad, u, u)
        dy = rng.normal(0, 1, y.shape).astype(np.float32)
        dx = O.conv2d_backward_data(dy.astype(np.float64), w.astype(np.float64), x.shape, pad, pad, u, u)
        dw = O.conv2d_backward_filter(x.astype(np.float64), dy.astype(np.float64), w.shape, pad, pad, u, u)
        refs = _sampled_references(x, w, dy, pad, u, rng, 50, 50, 20)
        for full, (idx, ref) in zip((y, dx, dw), refs):
            np.testing.assert_allclose(full[tuple(idx.T)], ref, rtol=1e-12, atol=1e-12)
