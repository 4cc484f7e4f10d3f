"""CPU oracle for the training hot path -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

A numpy restatement of the arithmetic that tinyflow's backward pass performs,
one function per operator.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import this package; nothing under
tinyflow_amd/ does, and the product has no CPU fallback.

Where the reference has a numpy branch the function follows it line by line;
where the reference only calls cuDNN/cuBLAS (convolution, pooling, batch norm,
activation, cudnnReduceTensor) the function restates the published definition
of that library call as the reference configures it.  Each docstring cites the
reference lines it follows.  All functions compute in the dtype of their inputs
(float32 reproduces the reference; float64 gives a high-precision yardstick).

What pins each function (see tests/test_oracle_*.py):
  matmul, ew ops, relu, softmax, xent   reference tests' closed forms and shapes
                                        (tests/test_gpu_op.py:5-182,
                                        tests/autodiff_test.py:188-208)
  conv fwd / dgrad / wgrad              brute-force 7-loop C (oracle/conv_direct.c),
                                        adjoint identities, 1x1 == matmul, torch CPU,
                                        the conv1d vector of tests/test_gpu_op.py:223
  pooling                               brute-force loops, sum(dx) == sum(dy), torch CPU
  batch norm                            closed form, sum(dx) = 0, sum(dx*xhat) = 0, torch CPU
  softmax activation backward           Jacobian by finite differences
  dropout generator (Philox4x32-10)     the known-answer vectors published with Random123;
                                        keep rate; forward/backward share one mask
  concatenation                         numpy.concatenate and its slices

Parity unpinned (only real cuDNN 7.6.5 could pin them bit-for-bit): the
summation order inside the cuDNN/cuBLAS kernels, cudnnPoolingBackward's choice
among tied maxima, cudnnActivationBackward's value at x == 0, and which elements
cudnnDropoutForward drops for a given seed (its generator is private to cuDNN).
The tie and zero rules used here are stated in max_pool_backward and relu_gradient,
the dropout mask definition in dropout_keep_mask.
"""
import numpy as np

BN_EPS = 1e-5  # reference src/gpu_op.cu:4333, 4442


# ----------------------------------------------------------------- elementwise

def add(a, b):
    """reference autodiff.py:314 (AddOp numpy branch); gpu_op.cu:193-198"""
    return a + b


def add_by_const(a, c):
    """reference autodiff.py:362; gpu_op.cu:200-205"""
    return a + a.dtype.type(c)


def multiply(a, b):
    """reference autodiff.py:386; gpu_op.cu:207-212"""
    return a * b


def multiply_by_const(a, c):
    """reference autodiff.py:427; gpu_op.cu:214-219"""
    return a * a.dtype.type(c)


def relu(x):
    """out = x, except 0 where x < 0: the CUDA kernel (gpu_op.cu:221-228), which
    leaves a negative zero as it is.  The numpy branch (autodiff.py:754,
    np.maximum(x, 0)) differs from it only in that sign of zero."""
    return np.where(x < 0, np.zeros_like(x), x)


def relu_gradient(x, grad):
    """dx = grad where x > 0 else 0.

    Follows the CUDA kernel (gpu_op.cu:230-235) and the reference's own unit test
    (tests/test_gpu_op.py:145-155), NOT the numpy branch, which yields 0.5*grad at
    x == 0 (autodiff.py:777-779)."""
    return np.where(x > 0, grad, np.zeros_like(grad))


def array_set(shape, value, dtype=np.float32):
    """reference gpu_op.cu:39-45"""
    return np.full(shape, value, dtype=dtype)


def broadcast_to_trailing(b, out_shape):
    """out[i] = b[i % b.size]: b matches the trailing dims (FC bias).
    reference gpu_op.cu:47-52, 343-367"""
    return np.ascontiguousarray(np.broadcast_to(b, out_shape))


def broadcast_to_channel(b, out_shape):
    """out[n, c, ...] = b[c] (conv bias).  reference gpu_op.cu:108-123, 450-471"""
    shape = [1] * len(out_shape)
    shape[1] = out_shape[1]
    return np.ascontiguousarray(np.broadcast_to(b.reshape(shape), out_shape))


def reduce_sum_axis_zero(x):
    """reference autodiff.py:601; gpu_op.cu:179-189"""
    return np.sum(x, axis=0)


def bias_gradient(dy, dataformat):
    """Gradient of a broadcast bias = sum over all non-channel dims.

    "NCHW": (N, C, H, W) -> (C,); "NHWC" on a 2-D (N, C) array -> (C,).
    reference autodiff.py:648-678 + gpu_op.py:83-119 (shapes handed to
    cudnnReduceTensor ADD, gpu_op.cu:812-881)."""
    if dataformat == "NCHW":
        axes = (0,) + tuple(range(2, dy.ndim))
        return dy.sum(axis=axes)
    return dy.reshape(-1, dy.shape[-1]).sum(axis=0)


def sgd_update(w, g, lr):
    """w - lr*g.  reference gpu_op.cu:4600-4605"""
    return w - w.dtype.type(lr) * g


def adam_mv(m, v, g, b1, b2):
    """reference gpu_op.cu:4495-4506"""
    t = m.dtype.type
    return m * t(b1) + g * t(1 - b1), v * t(b2) + g * g * t(1 - b2)


def adam_update(w, m, v, b1t, b2t, e, lr):
    """reference gpu_op.cu:4461-4467"""
    t = w.dtype.type
    return w - t(lr) * m / t(1 - b1t) / (np.sqrt(v / t(1 - b2t)) + t(e))


# ---------------------------------------------------------------------- matmul

def matmul(a, trans_a, b, trans_b):
    """reference autodiff.py:452-467 (four transpose cases of np.matmul)"""
    return np.matmul(a.T if trans_a else a, b.T if trans_b else b)


def matmul_gradients(a, trans_a, b, trans_b, dy):
    """(dA, dB) of Y = op(A) op(B).  reference autodiff.py:477-506"""
    if not trans_a and not trans_b:
        return matmul(dy, False, b, True), matmul(a, True, dy, False)
    if trans_a and not trans_b:
        return matmul(b, False, dy, True), matmul(a, False, dy, False)
    if not trans_a and trans_b:
        return matmul(dy, False, b, False), matmul(dy, True, a, False)
    return matmul(b, True, dy, True), matmul(dy, True, a, True)


# --------------------------------------------------- softmax / cross entropy

def softmax(y):
    """Row softmax, max-subtracted.  reference autodiff.py:681-686 (softmax_func)"""
    b = y - np.max(y, axis=1, keepdims=True)
    e = np.exp(b)
    return e / np.sum(e, axis=1, keepdims=True)


def softmax_cross_entropy(y, y_):
    """mean_n(-sum_c y_ * log softmax(y)), shape (1,).  reference autodiff.py:701-704"""
    return np.mean(-np.sum(y_ * np.log(softmax(y)), axis=1), keepdims=True)


def softmax_cross_entropy_gradient(y, y_, upstream=1.0):
    """(softmax(y) + -1*y_) * upstream -- NOT divided by the batch size although
    the loss is a batch mean.  reference autodiff.py:710-713"""
    return (softmax(y) + y.dtype.type(-1) * y_) * y.dtype.type(upstream)


def cross(x, y, scale):
    """-scale * y * log(x).  reference gpu_op.cu:4538-4543"""
    return np.log(x) * y * x.dtype.type(-1) * x.dtype.type(scale)


def cross_backward(x, y, dout, scale):
    """reference gpu_op.cu:4568-4573"""
    t = x.dtype.type
    return y * t(-1) * t(scale) * (t(1) / x) * dout


# ----------------------------------------------------------------- convolution

def conv_pad(filter_extent, padding):
    """"SAME" = symmetric k//2, "VALID" = 0.  reference gpu_op.cu:2081-2087"""
    return filter_extent // 2 if padding == "SAME" else 0


def conv_out_extent(in_extent, filter_extent, pad, stride):
    """cudnnGetConvolution2dForwardOutputDim with dilation 1 (gpu_op.cu:2121-2135)"""
    return 1 + (in_extent + 2 * pad - filter_extent) // stride


def _strided_taps(xp, r, s, P, Q, u, v):
    return xp[:, :, r:r + (P - 1) * u + 1:u, s:s + (Q - 1) * v + 1:v]


def conv2d_forward(x, w, pad_h, pad_w, u, v):
    """y[n,k,p,q] = sum_{c,r,s} x[n,c,p*u+r-pad_h,q*v+s-pad_w] * w[k,c,r,s]

    NCHW x, KCRS w, cross-correlation, dilation 1 -- cudnnConvolutionForward as
    configured at gpu_op.cu:2094-2125, 2019-2031."""
    N, C, H, W = x.shape
    K, C2, R, S = w.shape
    assert C == C2
    P = conv_out_extent(H, R, pad_h, u)
    Q = conv_out_extent(W, S, pad_w, v)
    xp = np.pad(x, ((0, 0), (0, 0), (pad_h, pad_h), (pad_w, pad_w)))
    # im2col: [N, C, R, S, P, Q] -> one GEMM with w viewed as [K, C*R*S]
    cols = np.empty((N, C, R, S, P, Q), dtype=x.dtype)
    for r in range(R):
        for s in range(S):
            cols[:, :, r, s] = _strided_taps(xp, r, s, P, Q, u, v)
    y = np.matmul(w.reshape(K, C * R * S), cols.reshape(N, C * R * S, P * Q))
    return y.reshape(N, K, P, Q)


def conv2d_backward_filter(x, dy, filter_shape, pad_h, pad_w, u, v):
    """dw[k,c,r,s] = sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*u+r-pad_h,q*v+s-pad_w]

    cudnnConvolutionBackwardFilter, beta = 0 (gpu_op.cu:1715-1728)."""
    N, C, H, W = x.shape
    K, _, R, S = filter_shape
    _, _, P, Q = dy.shape
    xp = np.pad(x, ((0, 0), (0, 0), (pad_h, pad_h), (pad_w, pad_w)))
    cols = np.empty((N, C, R, S, P, Q), dtype=x.dtype)
    for r in range(R):
        for s in range(S):
            cols[:, :, r, s] = _strided_taps(xp, r, s, P, Q, u, v)
    # sum over n of dy_n [K, PQ] @ cols_n^T [PQ, CRS]
    dw = np.tensordot(dy.reshape(N, K, P * Q), cols.reshape(N, C * R * S, P * Q), axes=([0, 2], [0, 2]))
    return dw.reshape(K, C, R, S).astype(x.dtype, copy=False)


def conv2d_backward_data(dy, w, input_shape, pad_h, pad_w, u, v):
    """dx[n,c,h,w] = sum_{k,r,s} dy[n,k,p,q] * w[k,c,r,s] with h = p*u+r-pad_h

    cudnnConvolutionBackwardData, beta = 0 (gpu_op.cu:1803-1816)."""
    N, C, H, W = input_shape
    K, _, R, S = w.shape
    _, _, P, Q = dy.shape
    # col gradient [N, CRS, PQ] = w^T [CRS, K] @ dy_n [K, PQ], then col2im (scatter-add)
    dcols = np.matmul(w.reshape(K, C * R * S).T, dy.reshape(N, K, P * Q)).reshape(N, C, R, S, P, Q)
    dxp = np.zeros((N, C, H + 2 * pad_h, W + 2 * pad_w), dtype=dy.dtype)
    for r in range(R):
        for s in range(S):
            dxp[:, :, r:r + (P - 1) * u + 1:u, s:s + (Q - 1) * v + 1:v] += dcols[:, :, r, s]
    return np.ascontiguousarray(dxp[:, :, pad_h:pad_h + H, pad_w:pad_w + W])


# --------------------------------------------------------------------- pooling

def pool_out_extent(in_extent, window, pad, stride):
    """cudnnGetPooling2dForwardOutputDim (gpu_op.cu:2941-2947)"""
    return 1 + (in_extent + 2 * pad - window) // stride


def _pool_windows(x, fh, fw, pad_h, pad_w, u, v, fill):
    N, C, H, W = x.shape
    P = pool_out_extent(H, fh, pad_h, u)
    Q = pool_out_extent(W, fw, pad_w, v)
    xp = np.full((N, C, H + 2 * pad_h, W + 2 * pad_w), fill, dtype=x.dtype)
    xp[:, :, pad_h:pad_h + H, pad_w:pad_w + W] = x
    win = np.empty((N, C, P, Q, fh, fw), dtype=x.dtype)
    for r in range(fh):
        for s in range(fw):
            win[..., r, s] = xp[:, :, r:r + (P - 1) * u + 1:u, s:s + (Q - 1) * v + 1:v]
    return win, P, Q


def max_pool_forward(x, fh, fw, pad_h, pad_w, u, v):
    """CUDNN_POOLING_MAX; padding never wins (gpu_op.cu:2921-2927, 2865-2872)."""
    win, P, Q = _pool_windows(x, fh, fw, pad_h, pad_w, u, v, -np.inf)
    return win.reshape(win.shape[:4] + (fh * fw,)).max(axis=-1)


def max_pool_backward(x, dy, fh, fw, pad_h, pad_w, u, v):
    """dy[n,c,p,q] goes to the FIRST maximum of window (p,q) in row-major scan
    order (numpy argmax); overlapping windows accumulate.

    cudnnPoolingBackward MAX (gpu_op.cu:3007-3018); the tie rule is this build's
    stated convention -- cuDNN's own choice among equal maxima is unpinned."""
    N, C, H, W = x.shape
    win, P, Q = _pool_windows(x, fh, fw, pad_h, pad_w, u, v, -np.inf)
    arg = win.reshape(N, C, P, Q, fh * fw).argmax(axis=-1)
    r, s = arg // fw, arg % fw
    p_idx = np.arange(P).reshape(1, 1, P, 1)
    q_idx = np.arange(Q).reshape(1, 1, 1, Q)
    h = p_idx * u + r - pad_h
    w_ = q_idx * v + s - pad_w
    n_idx = np.arange(N).reshape(N, 1, 1, 1)
    c_idx = np.arange(C).reshape(1, C, 1, 1)
    dx = np.zeros_like(x)
    np.add.at(dx, (np.broadcast_to(n_idx, arg.shape), np.broadcast_to(c_idx, arg.shape), h, w_), dy)
    return dx


def max_pool_argmax(x, fh, fw, pad_h, pad_w, u, v):
    """Flat input index h*W + w of the first maximum of every window."""
    N, C, H, W = x.shape
    win, P, Q = _pool_windows(x, fh, fw, pad_h, pad_w, u, v, -np.inf)
    arg = win.reshape(N, C, P, Q, fh * fw).argmax(axis=-1)
    h = np.arange(P).reshape(1, 1, P, 1) * u + arg // fw - pad_h
    w_ = np.arange(Q).reshape(1, 1, 1, Q) * v + arg % fw - pad_w
    return h * W + w_


def avg_pool_forward(x, fh, fw, pad_h, pad_w, u, v):
    """CUDNN_POOLING_AVERAGE_COUNT_INCLUDE_PADDING: always divide by fh*fw
    (gpu_op.py:610-613, gpu_op.cu:2921-2927)."""
    win, P, Q = _pool_windows(x, fh, fw, pad_h, pad_w, u, v, 0)
    return win.reshape(win.shape[:4] + (fh * fw,)).sum(axis=-1) / x.dtype.type(fh * fw)


def avg_pool_backward(x_shape, dy, fh, fw, pad_h, pad_w, u, v):
    N, C, H, W = x_shape
    _, _, P, Q = dy.shape
    dxp = np.zeros((N, C, H + 2 * pad_h, W + 2 * pad_w), dtype=dy.dtype)
    share = dy / dy.dtype.type(fh * fw)
    for r in range(fh):
        for s in range(fw):
            dxp[:, :, r:r + (P - 1) * u + 1:u, s:s + (Q - 1) * v + 1:v] += share
    return np.ascontiguousarray(dxp[:, :, pad_h:pad_h + H, pad_w:pad_w + W])


# ------------------------------------------------------------------ activation

def activation_forward(x, mode):
    """cudnnActivationForward (sigmoid/relu/tanh) and cudnnSoftmaxForward over
    c*h*w per instance for "softmax" (gpu_op.cu:3237-3260)."""
    if mode == "relu":
        return np.maximum(x, 0)
    if mode == "sigmoid":
        return 1 / (1 + np.exp(-x))
    if mode == "tanh":
        return np.tanh(x)
    if mode == "softmax":
        return softmax(x.reshape(x.shape[0], -1)).reshape(x.shape)
    raise ValueError(mode)


def activation_backward(x, y, dy, mode):
    """cudnnActivationBackward / cudnnSoftmaxBackward (gpu_op.cu:3505-3531).
    relu: dx = dy where x > 0 (equivalently y > 0); softmax: y*(dy - sum(dy*y))."""
    if mode == "relu":
        return np.where(x > 0, dy, np.zeros_like(dy))
    if mode == "sigmoid":
        return dy * y * (1 - y)
    if mode == "tanh":
        return dy * (1 - y * y)
    if mode == "softmax":
        y2 = y.reshape(y.shape[0], -1)
        dy2 = dy.reshape(y2.shape)
        return (y2 * (dy2 - np.sum(dy2 * y2, axis=1, keepdims=True))).reshape(x.shape)
    raise ValueError(mode)


# ---------------------------------------------------------- batch normalisation

def _bn_axes(x, mode):
    # "pre_activation" = CUDNN_BATCHNORM_PER_ACTIVATION: one statistic per (c,h,w), over N
    # "spatial"        = CUDNN_BATCHNORM_SPATIAL: one statistic per c, over (N,H,W)
    return (0,) if mode == "pre_activation" else (0,) + tuple(range(2, x.ndim))


def batch_norm_forward(x, mode):
    """y = (x - mean) * istd with gamma = 1, beta = 0, eps = 1e-5, biased
    variance; returns (y, mean, istd).  cudnnBatchNormalizationForwardTraining as
    called at gpu_op.cu:4245-4250, 4319-4337."""
    axes = _bn_axes(x, mode)
    mean = x.mean(axis=axes, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=axes, keepdims=True)
    istd = 1 / np.sqrt(var + x.dtype.type(BN_EPS))
    return (x - mean) * istd, mean, istd


def batch_norm_backward(x, dy, mode, mean=None, istd=None):
    """dx = istd/m * (m*dy - sum(dy) - xhat*sum(dy*xhat)), gamma = 1.
    cudnnBatchNormalizationBackward as called at gpu_op.cu:4426-4445 (the scale
    and bias gradients it also produces are discarded by the reference)."""
    axes = _bn_axes(x, mode)
    if mean is None or istd is None:
        _, mean, istd = batch_norm_forward(x, mode)
    m = x.dtype.type(np.prod([x.shape[a] for a in axes]))
    xhat = (x - mean) * istd
    sum_dy = dy.sum(axis=axes, keepdims=True)
    sum_dy_xhat = (dy * xhat).sum(axis=axes, keepdims=True)
    return istd / m * (m * dy - sum_dy - xhat * sum_dy_xhat)


# ------------------------------------------------------- dropout, concatenation

def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
    as 1, 2, 3", SC'11).  ``counter``: uint32 array [..., 4]; ``key``: two uint32.
    Returns uint32 [..., 4].  Pinned by the known-answer vectors published with the
    Random123 library (tests/test_oracle_ops.py)."""
    c = np.array(counter, dtype=np.uint64) & np.uint64(0xFFFFFFFF)
    c0, c1, c2, c3 = c[..., 0], c[..., 1], c[..., 2], c[..., 3]
    k0, k1 = np.uint64(int(key[0]) & 0xFFFFFFFF), np.uint64(int(key[1]) & 0xFFFFFFFF)
    m0, m1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0, p1 = m0 * c0, m1 * c2
        hi0, lo0 = p0 >> np.uint64(32), p0 & mask
        hi1, lo1 = p1 >> np.uint64(32), p1 & mask
        c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return np.stack([c0, c1, c2, c3], axis=-1).astype(np.uint32)


def dropout_keep_mask(count, dropout, seed):
    """Boolean keep-mask of ``count`` elements: element i uses word i % 4 of the
    Philox block with counter (i // 4, 0, 0, 0) and key (seed, 0) and is kept when
    that word is >= dropout * 2**32.  This is this build's definition (cuDNN's
    generator, reference gpu_op.cu:3606-3625, is not reproducible outside cuDNN):
    parity with the reference's mask bits is unpinned; what is pinned is the
    generator (known-answer vectors), the keep rate and the fwd/bwd mask identity."""
    blocks = (count + 3) // 4
    idx = np.arange(blocks, dtype=np.uint64)
    ctr = np.stack([idx & np.uint64(0xFFFFFFFF), idx >> np.uint64(32), np.zeros_like(idx), np.zeros_like(idx)], axis=-1)
    words = philox4x32_10(ctr, (seed, 0)).reshape(-1)[:count]
    t = float(dropout) * 4294967296.0
    threshold = np.uint32(0xFFFFFFFF) if t >= 4294967295.0 else np.uint32(int(t))
    return words >= threshold


def dropout_forward(x, dropout, seed):
    """out = x * keep / (1 - dropout) (cudnnDropoutForward semantics, reference
    gpu_op.cu:3547-3640); returns (out, keep)."""
    keep = dropout_keep_mask(x.size, dropout, seed).reshape(x.shape)
    scale = x.dtype.type(1.0) / (x.dtype.type(1.0) - x.dtype.type(dropout))
    return np.where(keep, x * scale, np.zeros_like(x)), keep


def dropout_backward(dy, keep, dropout):
    """dx = dy * keep / (1 - dropout) (reference gpu_op.cu:3647-3693)"""
    scale = dy.dtype.type(1.0) / (dy.dtype.type(1.0) - dy.dtype.type(dropout))
    return np.where(keep, dy * scale, np.zeros_like(dy))


def concat_forward(a, b):
    """reference gpu_op.cu:967-1003: concatenation along axis 1"""
    return np.concatenate([a, b], axis=1)


def concat_backward(a, b, dout):
    """reference gpu_op.cu:1006-1084: the two axis-1 slices of dout"""
    ca = a.shape[1]
    return np.ascontiguousarray(dout[:, :ca]), np.ascontiguousarray(dout[:, ca:ca + b.shape[1]])
