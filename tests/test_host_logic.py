"""Host-side logic without a GPU: the C-ABI surface, descriptor/shape helpers,
graph construction, reverse-mode differentiation and update placement.

Graphs are evaluated with tests/graph_eval.py (numpy, oracle ops) so that the
product's ``Op.gradient`` methods, ``gradients``, ``sum_node_list`` and ``swapsgd``
are exercised on the CPU and compared with the closed forms the reference's own
autodiff tests assert (tests/autodiff_test.py:8-208) and with the independent
layer-by-layer oracle networks.
"""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import models as OM
from oracle import ops as O
from tinyflow_amd import autodiff as ad
from tinyflow_amd import gpu_op, models
from tinyflow_amd._base import _LIB, LIB_PATH
from tinyflow_amd.TrainExecute import getcomputelist, swapsgd

from graph_eval import evaluate

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------------- C-ABI surface

def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "c_runtime_api.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\bint\s+([A-Za-z_][A-Za-z0-9_]*)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 50 and "DLGpuConvolutionBackwardFilter" in names and "DLArrayAlloc" in names
    lib = ctypes.CDLL(LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, "declared in include/c_runtime_api.h but not exported: %s" % missing


def test_streamed_copy_waits_unless_the_stream_orders_its_readers():
    """DLArrayCopyFromTo with a stream: copies that touch host memory always wait (the
    reference syncs after every streamed copy, src/c_runtime_api.cc:148-158); a
    device-to-device copy may stay asynchronous only on a stream that op entry points
    launch on, because nothing else would order a later reader behind it."""
    H2D, D2H, D2D = 0, 1, 2
    f = _LIB.DLArrayCopyWaitsForCompletion
    for runs_kernels in (0, 1):
        for sync in (0, 1):
            assert f(H2D, runs_kernels, sync) == 1
            assert f(D2H, runs_kernels, sync) == 1
    assert f(D2D, 1, 0) == 0      # compute stream: later kernels are enqueued behind the copy
    assert f(D2D, 0, 0) == 1      # copy-only side stream: wait, as the reference does
    assert f(D2D, 1, 1) == 1 and f(D2D, 0, 1) == 1


def test_no_alloc_column_sum_scratch_rule():
    """The partial sums the column sum keeps in the library's built-in 1.5 MiB area: on a
    256-unit part every chunked sum of up to 131 072 columns fits, single-chunk sums want
    nothing, wider chunked sums are refused; a part with more units wants more (the rule
    aims at four workgroups per unit), so there narrower sums are refused too."""
    def wanted(rows, cols, cus):
        w, lim = ctypes.c_int64(-1), ctypes.c_int64(-1)
        assert _LIB.DLGpuReduceSumAxisZeroNoAllocBytes(ctypes.c_int64(rows), ctypes.c_int64(cols), cus,
                                                       ctypes.byref(w), ctypes.byref(lim)) == 0
        assert lim.value == 3 << 19
        return w.value, lim.value
    worst = 0
    for rows in (1, 7, 8, 9, 64, 1000, 100000):
        for cols in list(range(1, 70)) + [255, 256, 257, 1000, 3000, 4097, 65536, 100000, 131072]:
            w, lim = wanted(rows, cols, 256)
            assert w % (4 * cols) == 0 and w // (4 * cols) != 1      # whole chunks; one chunk needs no scratch
            assert w // (4 * cols) <= max(1, (rows + 7) // 8)       # at least eight rows per chunk
            assert w <= lim, (rows, cols, w)
            worst = max(worst, w)
    assert worst > lim // 2                                          # the bound is not vacuous
    assert wanted(64, 200000, 256)[0] == 2 * 200000 * 4 > lim        # refused by the entry point
    assert wanted(8, 200000, 256)[0] == 0                            # eight rows: one chunk
    assert wanted(64, 300000, 256)[0] == 0                           # wide enough to fill the part unsplit
    assert wanted(100000, 100000, 512)[0] > lim                      # a larger part splits further
    assert wanted(0, 5, 256)[0] == 0 and wanted(5, 0, 256)[0] == 0


def test_struct_layout_matches_the_abi():
    """DLContext is 8 bytes, DLArray 32 (src/dlarray.h:21-52)."""
    from tinyflow_amd import ndarray
    assert ctypes.sizeof(ndarray.DLContext) == 8
    assert ctypes.sizeof(ndarray.DLArray) == 32
    assert ndarray.DLArray.ctx.offset == 8 and ndarray.DLArray.ndim.offset == 16 and ndarray.DLArray.shape.offset == 24
    assert ndarray.cpu().device_type == 1 and ndarray.gpu().device_type == 2
    assert _LIB.getInt(ctypes.byref(ctypes.c_int(41))) == 41


@pytest.mark.parametrize("case", [
    ((64, 3, 224, 224), (64, 3, 7, 7), "SAME", 2, 2), ((64, 64, 56, 56), (256, 64, 1, 1), "VALID", 1, 1),
    ((64, 256, 56, 56), (512, 256, 1, 1), "VALID", 2, 2), ((32, 64, 224, 224), (64, 64, 3, 3), "SAME", 1, 1),
    ((64, 6, 14, 14), (16, 6, 5, 5), "VALID", 1, 1), ((2, 3, 9, 10), (4, 3, 2, 2), "SAME", 1, 1)], ids=str)
def test_conv_out_shape_descriptor(case):
    x_shape, w_shape, padding, u, v = case
    out, lst = gpu_op.convolution_2d_forward_get_out_shape(x_shape, w_shape, "NCHW", padding, u, v)
    ph, pw = O.conv_pad(w_shape[2], padding), O.conv_pad(w_shape[3], padding)
    assert out == (x_shape[0], w_shape[0], O.conv_out_extent(x_shape[2], w_shape[2], ph, u),
                   O.conv_out_extent(x_shape[3], w_shape[3], pw, v))
    name = ctypes.create_string_buffer(256)
    flops = ctypes.c_double()
    for which in range(3):
        assert _LIB.DLGpuConvolutionDescribeKernel(lst, which, name, 256, ctypes.byref(flops)) == 0
        assert b" | gemm_kernel<" in name.value
        expect = 2.0 * np.prod(out, dtype=np.float64) * w_shape[1] * w_shape[2] * w_shape[3]
        variant = name.value.decode().split()[0]
        if "winograd" in variant:   # flops the batched transformed-domain products execute
            m = 4 if variant.endswith("4x4") else 2
            rows, cols = (x_shape[2], x_shape[3]) if which == 1 else (out[2], out[3])
            tiles = x_shape[0] * -(-rows // m) * -(-cols // m)
            expect = 2.0 * (m + 2) ** 2 * w_shape[0] * w_shape[1] * tiles
        assert flops.value == expect


def _variants(x_shape, w_shape, padding="SAME", stride=1):
    _, lst = gpu_op.convolution_2d_forward_get_out_shape(x_shape, w_shape, "NCHW", padding, stride, stride)
    name = ctypes.create_string_buffer(256)
    out = []
    for which in range(3):
        assert _LIB.DLGpuConvolutionDescribeKernel(lst, which, name, 256, None) == 0
        out.append(name.value.decode().split()[0])
    return out


def test_planner_picks_winograd_forms_by_shape(monkeypatch):
    """3x3 / stride-1 layers of the ResNet-50 batch-64 configuration: 4x4 tiles up to 512
    channels, 2x2 tiles above; other filters and strides stay direct; the environment
    overrides what the cost model would pick."""
    monkeypatch.delenv("TINYFLOW_WINOGRAD", raising=False)
    monkeypatch.delenv("TINYFLOW_WINOGRAD_MAX_TILE", raising=False)
    four = ["fwd_winograd4x4", "dgrad_winograd4x4", "wgrad_winograd4x4"]
    assert _variants((64, 64, 56, 56), (64, 64, 3, 3)) == four
    assert _variants((64, 128, 28, 28), (128, 128, 3, 3)) == four
    assert _variants((64, 256, 14, 14), (256, 256, 3, 3)) == four
    assert _variants((64, 512, 7, 7), (512, 512, 3, 3)) == four
    assert _variants((16, 640, 14, 14), (640, 640, 3, 3)) == ["fwd_winograd", "dgrad_winograd", "wgrad_winograd"]
    for shapes in (((64, 64, 56, 56), (256, 64, 1, 1), "VALID", 1), ((64, 3, 224, 224), (64, 3, 7, 7), "SAME", 2),
                   ((64, 128, 56, 56), (128, 128, 3, 3), "SAME", 2)):
        assert not any("winograd" in v for v in _variants(*shapes))
    monkeypatch.setenv("TINYFLOW_WINOGRAD_MAX_TILE", "2")
    assert not any("4x4" in v for v in _variants((64, 128, 28, 28), (128, 128, 3, 3)))
    assert "fwd_winograd" in _variants((64, 128, 28, 28), (128, 128, 3, 3))
    monkeypatch.setenv("TINYFLOW_WINOGRAD", "0")
    assert not any("winograd" in v for v in _variants((64, 256, 14, 14), (256, 256, 3, 3)))


def test_descriptor_calls_reject_bad_arguments():
    with pytest.raises(RuntimeError):
        gpu_op.convolution_2d_forward_get_out_shape((2, 3, 8, 8), (4, 5, 3, 3), "NCHW", "SAME", 1, 1)  # channel mismatch
    with pytest.raises(RuntimeError):
        gpu_op.convolution_2d_forward_get_out_shape((2, 8, 8, 3), (4, 3, 3, 3), "NHWC", "SAME", 1, 1)  # layout
    with pytest.raises(RuntimeError):
        gpu_op.pooling_2d_forward_get_out_shape((2, 3, 4, 4), "NCHW", "max", 0, 0, 2, 2, 9, 9)         # window > input
    with pytest.raises(AssertionError):
        gpu_op.pooling_2d_forward_get_out_shape((2, 3, 4, 4), "NCHW", "median", 0, 0, 2, 2, 2, 2)


def test_pool_out_shape_descriptor():
    out, _ = gpu_op.pooling_2d_forward_get_out_shape((64, 64, 112, 112), "NCHW", "max", 1, 1, 2, 2, 3, 3)
    assert out == (64, 64, 56, 56)
    out, _ = gpu_op.pooling_2d_forward_get_out_shape((64, 64, 112, 112), "NCHW", "max", 0, 0, 2, 2, 3, 3)
    assert out == (64, 64, 55, 55)
    out, _ = gpu_op.pooling_2d_forward_get_out_shape((64, 2048, 7, 7), "NCHW", "mean", 0, 0, 1, 1, 7, 7)
    assert out == (64, 2048, 1, 1)


def test_reduce_sum_real_shapes():
    """gpu_op.py:83-119 of the reference."""
    f = gpu_op.reduce_sum_get_real_shape
    assert f((64, 6, 28, 28), (6,), "NCHW") == ((64, 6, 28, 28), (1, 6, 1, 1))
    assert f((128, 256), (256,), "NHWC") == ((1, 128, 256), (1, 1, 256))
    assert f((128, 10), (1,), "NHWC") == ((1, 128, 10), (1, 1, 1))
    assert f((4, 5, 6), (6,), "NHWC") == ((4, 5, 6), (1, 1, 6))


# ----------------------------------------------------- autodiff algebra (reference cases)

def _grad_values(y, wrt, feed):
    grads = ad.gradients(y, wrt)
    vals = evaluate([y] + grads, feed)
    return vals[y], [vals[g] for g in grads]


def test_identity_and_constants():
    """autodiff_test.py:8-60"""
    x2 = ad.Variable("x2")
    x2v = 2 * np.ones(3)
    y, (g,) = _grad_values(x2, [x2], {x2: x2v})
    assert np.array_equal(y, x2v) and np.array_equal(g, np.ones_like(x2v))
    y, (g,) = _grad_values(5 + x2, [x2], {x2: x2v})
    assert np.array_equal(y, x2v + 5) and np.array_equal(g, np.ones_like(x2v))
    y, (g,) = _grad_values(5 * x2, [x2], {x2: x2v})
    assert np.array_equal(y, x2v * 5) and np.array_equal(g, np.ones_like(x2v) * 5)


def test_add_mul_and_mixed_expressions():
    """autodiff_test.py:62-150"""
    x1, x2, x3 = ad.Variable("x1"), ad.Variable("x2"), ad.Variable("x3")
    v1, v2, v3 = 1 * np.ones(3), 2 * np.ones(3), 3 * np.ones(3)
    feed = {x1: v1, x2: v2, x3: v3}
    y, (g2, g3) = _grad_values(x2 + x3, [x2, x3], feed)
    assert np.array_equal(y, v2 + v3) and np.array_equal(g2, np.ones(3)) and np.array_equal(g3, np.ones(3))
    y, (g2, g3) = _grad_values(x2 * x3, [x2, x3], feed)
    assert np.array_equal(y, v2 * v3) and np.array_equal(g2, v3) and np.array_equal(g3, v2)
    y, (g1, g2, g3) = _grad_values(x1 + x2 * x3 * x1, [x1, x2, x3], feed)
    assert np.array_equal(y, v1 + v2 * v3)
    assert np.array_equal(g1, np.ones(3) + v2 * v3) and np.array_equal(g2, v3 * v1) and np.array_equal(g3, v2 * v1)
    # a node used several times: partial adjoints are accumulated
    y, (g2, g3) = _grad_values(x2 * x2 + x2 + x3 + 3, [x2, x3], feed)
    assert np.array_equal(y, v2 * v2 + v2 + v3 + 3)
    assert np.array_equal(g2, 2 * v2 + 1) and np.array_equal(g3, np.ones(3))


def test_scalar_operand_shapes():
    """A (1,)-shaped operand (the upstream-gradient scalar) is applied as a constant:
    the result has the other operand's shape whichever side the scalar is on.  (The
    reference's AddOp.infer_shape returns the second operand's shape for any unequal
    pair, autodiff.py:335-348, which under-allocates the result of ``x + scalar``.)"""
    x, s = ad.Placeholder("x"), ad.Placeholder("s")
    for node in (x + s, s + x, x * s, s * x):
        shapes = {x: (4, 5), s: (1,)}
        assert tuple(node.op.infer_shape(node, [shapes[i] for i in node.inputs], None)) == (4, 5)
    both = x + x
    assert tuple(both.op.infer_shape(both, [(4, 5), (4, 5)], None)) == (4, 5)


def test_gradient_of_gradient():
    """autodiff_test.py:152-186: y = x2*x2 + x2*x3, z = dy/dx2 + dy/dx3, then dz/dx."""
    x2, x3 = ad.Variable("x2"), ad.Variable("x3")
    v2, v3 = 2 * np.ones(3), 3 * np.ones(3)
    y = x2 * x2 + x2 * x3
    g2, g3 = ad.gradients(y, [x2, x3])
    gg2, gg3 = ad.gradients(g2 + g3, [x2, x3])
    vals = evaluate([y, g2, g3, gg2, gg3], {x2: v2, x3: v3})
    assert np.array_equal(vals[y], v2 * v2 + v2 * v3)
    assert np.array_equal(vals[g2], 2 * v2 + v3) and np.array_equal(vals[g3], v2)
    assert np.array_equal(vals[gg2], 3 * np.ones(3)) and np.array_equal(vals[gg3], np.ones(3))


def test_matmul_gradient_nodes():
    """autodiff_test.py:188-208 plus the other three transpose combinations."""
    rng = np.random.RandomState(0)
    for ta in (False, True):
        for tb in (False, True):
            A, B = ad.Variable("A"), ad.Variable("B")
            a = rng.normal(0, 1, (4, 3) if ta else (3, 4))
            b = rng.normal(0, 1, (5, 4) if tb else (4, 5))
            y = ad.matmul_op(A, B, ta, tb)
            val, (ga, gb) = _grad_values(y, [A, B], {A: a, B: b})
            da, db = O.matmul_gradients(a, ta, b, tb, np.ones((3, 5)))
            np.testing.assert_allclose(val, O.matmul(a, ta, b, tb))
            np.testing.assert_allclose(ga, da)
            np.testing.assert_allclose(gb, db)


def test_topo_sort_handles_deep_graphs_and_shared_nodes():
    x = ad.Variable("x")
    h = x
    for _ in range(5000):   # far beyond the default recursion limit
        h = h + 1
    order = ad.find_topo_sort([h, x])
    assert order[0] is x and order[-1] is h and len(order) == 5001
    a = x * x
    order = ad.find_topo_sort([a + a])
    assert order.count(a) == 1


# ------------------------------------------- whole networks: graph autodiff vs layer oracle

def _network_case(name):
    if name == "mlp":
        model, X, y = models.build("mlp", batch=16)
        return model, X, y, OM.network("mlp")
    if name == "lenet5":
        model, X, y = models.build("lenet5", batch=4)
        return model, X, y, OM.network("lenet5")
    if name == "vgg16":
        model, X, y = models.build("vgg16", batch=2, image=32, n_class=10, fc_width=32)
        return model, X, y, OM.network("vgg16")
    blocks, mode = [2, 1, 1, 1], name.split(":")[1]
    rng = np.random.RandomState(4)
    X, y = models.synthetic_batch(rng, (8, 3, 32, 32), 10, "normal")
    model = models.resnet(rng, blocks, 8, image=32, n_class=10, bn_mode=mode, width=4)
    return model, X, y, OM.resnet_layers(blocks, mode, 1)


@pytest.mark.parametrize("name", ["mlp", "lenet5", "vgg16", "resnet:pre_activation", "resnet:spatial"])
def test_graph_gradients_and_sgd_step_match_the_layer_oracle(name):
    model, X, y, net = _network_case(name)
    lr = 0.05
    variables = list(model.variables)
    params = {v.name: val.astype(np.float64) for v, val in model.variables.items()}
    loss_ref, grads_ref, new_params, logits_ref = OM.train_step(net, params, X.astype(np.float64),
                                                                y.astype(np.float64), lr)
    # same step through the product's graph: gradients(), sgd nodes, swapsgd order
    var_list = list(reversed(ad.get_Variable_node_list(model.loss)))
    assert set(var_list) == set(variables)
    grads = ad.gradients(model.loss, var_list)
    order = swapsgd(ad.find_topo_sort(getcomputelist(var_list, grads, lr)))
    feed = {model.X: X.astype(np.float64), model.y_: y.astype(np.float64)}
    feed.update({v: params[v.name] for v in variables})
    val = dict(feed)
    for node in order:                     # execute exactly in the executor's order
        if node in val:
            continue
        sub = evaluate([node], val)
        if node.issgd:
            val[node.inputs[0]] = sub[node.inputs[0]]
        val[node] = sub[node]
    np.testing.assert_allclose(val[model.loss], loss_ref, rtol=1e-10)
    np.testing.assert_allclose(val[model.logits], logits_ref, rtol=1e-8, atol=1e-10)
    for v, g in zip(var_list, grads):
        np.testing.assert_allclose(val[g], grads_ref[v.name].reshape(val[g].shape), rtol=1e-7, atol=1e-10,
                                   err_msg=v.name)
        np.testing.assert_allclose(val[v], new_params[v.name], rtol=1e-7, atol=1e-10, err_msg=v.name)


@pytest.mark.parametrize("config,kw", [("lenet5", {}), ("resnet50", dict(batch=2, image=32, n_class=10, width=4))])
def test_updates_are_placed_behind_the_last_reader(config, kw):
    """swapsgd: no node that reads a parameter runs after that parameter's update."""
    model, _, _ = models.build(config, **kw)
    var_list = list(reversed(ad.get_Variable_node_list(model.loss)))
    order = swapsgd(ad.find_topo_sort(getcomputelist(var_list, ad.gradients(model.loss, var_list), 0.1)))
    pos = {n: i for i, n in enumerate(order)}
    updates = [n for n in order if n.issgd]
    assert len(updates) == len(var_list)
    for upd in updates:
        param = upd.inputs[0]
        readers = [n for n in order if not n.issgd and param in n.inputs]
        assert readers and max(pos[r] for r in readers) < pos[upd]
        assert all(pos[i] < pos[upd] for i in upd.inputs)      # still topological
    for n in order:                                             # whole order stays topological
        assert all(pos[i] < pos[n] for i in n.inputs)


def test_adam_updates_are_placed_behind_the_last_reader():
    """The Adam step graph: one update node per variable reading (w, m, v, grad), two
    zero-initialised moment variables per variable, updates behind the last reader."""
    from tinyflow_amd import TrainExecuteAdam as A
    model, _, _ = models.build("lenet5")
    var_list = list(reversed(ad.get_Variable_node_list(model.loss)))
    b1t, b2t = [0.9], [0.999]
    updates, mv, var_to_mv = A.getcomputelist(var_list, ad.gradients(model.loss, var_list), 0.9, 0.999, b1t, b2t,
                                              1e-8, 0.001)
    assert len(updates) == len(var_list) and len(mv) == 2 * len(var_list)
    for upd, var in zip(updates, var_list):
        m, v = var_to_mv[var]
        assert upd.inputs[:3] == [var, m, v] and upd.issgd == 1
        assert (m.name, v.name, m.isw, v.isw) == (var.name + "m", var.name + "v", 1, 1)
        assert upd.b1t is b1t and upd.b2t is b2t          # shared with the executor, which advances them
    order = A.swapadam(ad.find_topo_sort(updates))
    pos = {n: i for i, n in enumerate(order)}
    for upd in updates:
        readers = [n for n in order if not n.issgd and upd.inputs[0] in n.inputs]
        assert readers and max(pos[r] for r in readers) < pos[upd]
    for n in order:
        assert all(pos[i] < pos[n] for i in n.inputs)


def test_resnet50_graph_census():
    """ResNet-50 as the reference builds it: 53 convolutions and 53 batch norms, 49
    ReLUs, 16 residual adds; the first convolution's grad-data node is never reached
    from the optimizer nodes, so 52 grad-data and 53 grad-filter nodes execute."""
    model, _, _ = models.build("resnet50", batch=2, image=32, n_class=10, width=4)
    var_list = list(reversed(ad.get_Variable_node_list(model.loss)))
    assert len(var_list) == 55   # 53 filters + fc weight + fc bias
    order = ad.find_topo_sort(getcomputelist(var_list, ad.gradients(model.loss, var_list), 0.1))
    count = lambda pred: sum(1 for n in order if pred(n))
    assert count(lambda n: isinstance(n.op, ad.Convolution2DForwardOp)) == 53
    assert count(lambda n: isinstance(n.op, ad.BNForwardOp)) == 53
    assert count(lambda n: isinstance(n.op, ad.BNBackwardOp)) == 53
    assert count(lambda n: isinstance(n.op, ad.ActivationForwardOp)) == 49
    assert count(lambda n: isinstance(n.op, ad.Convolution2DBackwardOp) and n.type == 1) == 53
    assert count(lambda n: isinstance(n.op, ad.Convolution2DBackwardOp) and n.type == 0) == 52
    n_params = sum(int(np.prod(v.shape)) for v in model.variables.values())
    assert n_params > 0


def test_resnet50_parameter_count_at_full_width():
    """25 503 912 trainable parameters: 53 filters + 2048x1000 + 1000 (BN has none)."""
    shapes = []
    rng = np.random.RandomState(0)

    class Recorder(models._Builder):
        def var(self, name, shape, zero=False):
            shapes.append(shape)
            return ad.Variable(name)
    orig = models._Builder
    models._Builder = Recorder
    try:
        models.resnet50(rng, batch=1)
    finally:
        models._Builder = orig
    assert sum(int(np.prod(s)) for s in shapes) == 25503912


# ------------------------------------------------------------- swap schedule

def test_swap_schedule_orders_every_transfer_around_its_uses():
    """plan_schedule on the LeNet training graph: every offloaded value is a
    forward value with a backward use; it leaves after its last forward use, comes
    back before its first backward use and is released only after its last use."""
    from tinyflow_amd import autodiff as ad, models
    from tinyflow_amd.SwapExecute import plan_schedule
    from tinyflow_amd.TrainExecute import getcomputelist, swapsgd
    rng = np.random.RandomState(0)
    model = models.build("lenet", rng=rng) if hasattr(models, "CONFIGS") and "lenet" in models.CONFIGS \
        else models.lenet5(rng, 8)
    variables = ad.get_Variable_node_list(model.loss)
    variables.reverse()
    grads = ad.gradients(model.loss, variables)
    topo = swapsgd(ad.find_topo_sort(getcomputelist(variables, grads, 0.1)))
    forward = set(ad.find_topo_sort([model.loss]))
    keep = set(variables) | {model.X, model.y_, model.loss}
    swap_out, swap_in, release, recompute = plan_schedule(topo, forward, keep, lambda n: True, 2)
    assert recompute == {}
    pos = {n: i for i, n in enumerate(topo)}
    uses = {}
    for n in topo:
        for inp in n.inputs:
            uses.setdefault(inp, []).append(pos[n])
    out_at = {n: t for t, ns in swap_out.items() for n in ns}
    in_at = {n: t for t, ns in swap_in.items() for n in ns}
    rel_at = {n: t for t, ns in release.items() for n in ns}
    assert out_at and set(out_at) == set(in_at)
    first_backward = min(pos[n] for n in topo if n not in forward and n.isw not in (1, 2))
    for n, t_out in out_at.items():
        assert n in forward and n not in keep
        fwd = [u for u in uses[n] if u < first_backward]
        bwd = [u for u in uses[n] if u >= first_backward]
        assert bwd, "offloaded value without a backward use"
        assert t_out >= max(fwd + [pos[n]])
        assert t_out < in_at[n] < bwd[0]
        assert rel_at[n] == max(uses[n])
    for n in keep:
        assert n not in rel_at and n not in out_at
    # every value that is not kept is released exactly once, never before its last use
    for n in topo:
        if n in keep or n.issgd:
            continue
        assert rel_at[n] == max(uses.get(n, [pos[n]]))


def test_prefetch_points_placed_by_time():
    """plan_schedule with node and copy times: every prefetch still lies between the
    tensor's last forward and first backward use; a slower link moves the points
    earlier; and the copies, laid out back to back on one engine with the last
    needed last, each fit between their point and the first use."""
    from tinyflow_amd.SwapExecute import plan_schedule
    from tinyflow_amd.TrainExecute import getcomputelist, swapsgd
    model, _, _ = models.build("resnet50", batch=2, image=32, n_class=10, width=4)
    variables = list(reversed(ad.get_Variable_node_list(model.loss)))
    topo = swapsgd(ad.find_topo_sort(getcomputelist(variables, ad.gradients(model.loss, variables), 0.1)))
    forward = set(ad.find_topo_sort([model.loss]))
    keep = set(variables) | {model.X, model.y_, model.loss}
    pos = {n: i for i, n in enumerate(topo)}
    uses = {}
    for n in topo:
        for inp in n.inputs:
            uses.setdefault(inp, []).append(pos[n])
    first_backward = min(pos[n] for n in topo if n not in forward and n.isw not in (1, 2))
    node_seconds = 1e-3
    clock = lambda i: i * node_seconds                     # device time at which node i starts

    movable = lambda n: pos[n] % 5 == 0                    # a fifth of the values: a load the link can carry

    def points(copy_seconds):
        out, inn, _, _ = plan_schedule(topo, forward, keep, movable, 2, seconds_of=lambda n: node_seconds,
                                       copy_seconds_of=lambda n: copy_seconds, copy_slack=1.0)
        return ({n: t for t, ns in out.items() for n in ns}, {n: t for t, ns in inn.items() for n in ns})
    out_fast, in_fast = points(0.5e-3)
    out_slow, in_slow = points(2e-3)
    assert in_fast and set(in_fast) == set(in_slow) == set(out_fast)
    earlier = 0
    for n in in_fast:
        first_use = min(u for u in uses[n] if u >= first_backward)
        for table in (in_fast, in_slow):
            assert max(out_fast[n], first_backward - 2) < table[n] < first_use
        assert in_slow[n] <= in_fast[n]
        earlier += in_slow[n] < in_fast[n]
    assert earlier > 0
    # the slow link's copies, started when the device passes their point and run one after
    # the other in order of need, are all in time -- unless the point is already the earliest possible
    engine_free = 0.0
    for n in sorted(in_slow, key=lambda n: min(u for u in uses[n] if u >= first_backward)):
        first_use = min(u for u in uses[n] if u >= first_backward)
        start = max(engine_free, clock(in_slow[n] + 1))
        engine_free = start + 2e-3
        at_floor = in_slow[n] == max(out_slow[n] + 1, first_backward - 1)
        assert engine_free <= clock(first_use) + 1e-9 or at_floor, (n.name, engine_free, clock(first_use))


def test_budget_recomputes_cheap_convolution_outputs_instead_of_moving_them():
    """plan_schedule with a budget and ``recompute_instead``: of the tensors the budget
    would send over the link, the convolution outputs that hang on a short chain are
    recomputed; fewer bytes move, the simulated footprint still fits, a chain holds at
    most one such value and five evaluations, and without the option (or without a
    budget) the plan is the old one."""
    from tinyflow_amd.SwapExecute import plan_schedule
    from tinyflow_amd.TrainExecute import getcomputelist, swapsgd
    rng = np.random.RandomState(0)
    model = models.resnet(rng, [2, 2, 1, 1], 4, image=32, n_class=10, width=8)
    variables = list(reversed(ad.get_Variable_node_list(model.loss)))
    topo = swapsgd(ad.find_topo_sort(getcomputelist(variables, ad.gradients(model.loss, variables), 0.1)))
    forward = set(ad.find_topo_sort([model.loss]))
    keep = set(n for n in topo if n.isw in (1, 2)) | {model.loss}
    shapes = {}
    feed = {model.X: (4, 3, 32, 32), model.y_: (4, 10)}
    for n in topo:
        if n in feed:
            shapes[n] = feed[n]
        elif n.isw == 1:
            shapes[n] = tuple(np.shape(dict(model.variables)[n]))
        else:
            shapes[n] = tuple(n.op.infer_shape(n, [shapes[i] for i in n.inputs], None))
    nbytes = lambda n: 4 * int(np.prod(shapes[n]))
    cheap = lambda n: isinstance(n.op, (ad.BNForwardOp, ad.ActivationForwardOp))
    conv = lambda n: isinstance(n.op, ad.Convolution2DForwardOp)
    args = (topo, forward, keep, lambda n: True, 2)
    common = dict(nbytes_of=nbytes, recomputable=cheap)
    # the footprint with recomputation only, then a budget a fifth below its peak
    pos = {n: i for i, n in enumerate(topo)}

    def peak_of(plan, budget_for_lag=0):
        out, inn, rel, rec = plan
        live = np.zeros(len(topo) + 1, dtype=np.int64)
        persistent = sum(nbytes(n) for n in keep)
        last = {n: max(t for t, ns in rel.items() if n in ns) for n in topo if n not in keep and not n.issgd}
        for n, l in last.items():
            live[pos[n]] += nbytes(n)
            live[l + 1] -= nbytes(n)
        live = np.cumsum(live)[:len(topo)] + persistent
        first_rel = {n: min(t for t, ns in rel.items() if n in ns) for n in last}
        for t, ns in rec.items():
            for n in ns:
                live[first_rel[n] + 1:t] -= nbytes(n)
        in_at = {n: t for t, ns in inn.items() for n in ns}
        for t, ns in out.items():
            for n in ns:
                live[t + 2 + 1:in_at[n]] -= nbytes(n)
        return int(live.max())

    free = plan_schedule(*args, budget=1 << 40, **common)
    assert not free[0], "nothing has to move under a huge budget"
    budget = int(peak_of(free) * 0.8)
    plain = plan_schedule(*args, budget=budget, **common)
    hybrid = plan_schedule(*args, budget=budget, recompute_instead=conv, **common)
    assert plan_schedule(*args, budget=budget, recompute_instead=lambda n: False, **common) == plain
    moved = lambda plan: sum(nbytes(n) for ns in plan[0].values() for n in ns)
    rec_of = lambda plan: {n for ns in plan[3].values() for n in ns}
    assert moved(plain) > 0
    heavy = {n for n in rec_of(hybrid) if conv(n)}
    assert heavy and not any(conv(n) for n in rec_of(plain))
    assert heavy <= {n for ns in plain[0].values() for n in ns}, "only tensors the budget would have moved"
    assert moved(hybrid) < moved(plain)
    assert peak_of(hybrid) <= budget

    rec_at = {n: t for t, ns in hybrid[3].items() for n in ns}

    def chain(n):
        if n not in rec_at:
            return 0, 0
        below = [chain(i) for i in n.inputs]
        return 1 + max(d for d, _ in below), int(conv(n)) + max(h for _, h in below)

    for n, t in rec_at.items():
        d, h = chain(n)
        assert (h == 0 and d <= 2) or (h == 1 and d <= 5), (n.name, d, h)
        for inp in n.inputs:
            if inp in rec_at:
                assert rec_at[inp] <= t


def test_planner_wire_format_round_trip():
    """schedule_to_wire / schedule_from_wire: the planner's list format
    (reference Scheduler.py:304-331) carries the same schedule as the dicts."""
    from tinyflow_amd.SwapExecute import schedule_from_wire, schedule_to_wire
    swap_out = {3: [1, 2], 7: [5]}
    swap_in = {7: [1], 20: [2, 5]}
    release = {4: [0], 25: [1, 2, 5]}
    swaps, releases = schedule_to_wire(swap_out, swap_in, release)
    assert all(len(m) == 5 and m[1] == 0 and m[4] == 1 for m in swaps)
    assert [m[2] for m in swaps] == sorted(m[2] for m in swaps)          # issue order = trigger order
    assert swaps[0] == [1, 0, 3, 0, 1] and [5, 0, 20, 1, 1] in swaps
    assert releases == [(4, 0), (25, 1), (25, 2), (25, 5)]
    out2, in2, rel2, rec2 = schedule_from_wire(swaps, releases, [(9, 4, True)])
    assert out2 == swap_out and in2 == swap_in and rel2 == release and rec2 == {9: [4]}


def test_planner_message_format():
    """Executor -> planner report (reference autodiff.py:2473-2510): one entry per node,
    ids are topological positions, update nodes list the tensors they rewrite under
    id + node count, parameters and the loss carry the flag."""
    from tinyflow_amd import TrainExecuteAdam as A
    from tinyflow_amd.SwapExecute import planner_message
    from tinyflow_amd.TrainExecute import getcomputelist, swapsgd
    model, X, y = models.build("lenet5")
    variables = list(reversed(ad.get_Variable_node_list(model.loss)))
    grads = ad.gradients(model.loss, variables)
    for optimizer in ("sgd", "adam"):
        if optimizer == "sgd":
            updates = getcomputelist(variables, grads, 0.1)
            fed = {}
        else:
            updates, mv, var_to_mv = A.getcomputelist(variables, grads, 0.9, 0.999, [0.9], [0.999], 1e-8, 0.001)
            fed = {n: np.shape(model.variables[v]) for v, pair in var_to_mv.items() for n in pair}
        topo = swapsgd(ad.find_topo_sort(updates))
        shapes = {model.X: X.shape, model.y_: y.shape}
        shapes.update({v: np.shape(val) for v, val in model.variables.items()})
        shapes.update(fed)
        for n in topo:
            if n not in shapes:
                shapes[n] = tuple(n.op.infer_shape(n, [shapes[i] for i in n.inputs], None))
        some = topo[len(topo) // 2]
        msg = planner_message(topo, shapes, model.loss, {some: 2.5e-4})
        assert len(msg) == len(topo)
        total = len(topo)
        for i, (node, entry) in enumerate(zip(topo, msg)):
            tensors, inputs, name, op_id, flag, empty, runtime = entry
            assert (name, op_id, empty) == (node.name, i, [])
            assert inputs == [topo.index(p) for p in node.inputs]
            assert flag == (1 if (node.isw == 1 or node is model.loss) else 0)
            assert runtime == (2.5e-4 if node is some else 1e-8)
            if node.issgd:
                want = 3 if optimizer == "adam" else 1
                assert [t[0] for t in tensors] == [topo.index(p) + total for p in node.inputs[:want]]
                assert all(t[1] == 4 * int(np.prod(shapes[p])) for t, p in zip(tensors, node.inputs))
            else:
                assert tensors == [(i, 4 * int(np.prod(shapes[node])), tuple(shapes[node]))]


def test_recompute_schedule_invariants():
    """plan_schedule with recomputation on a shallow bottleneck ResNet: batch-norm and
    activation outputs are rebuilt instead of moved, every recomputation comes no
    later than the first backward use, its inputs are back on the device by then,
    chains are at most two long, and producers are rebuilt before their consumers."""
    from tinyflow_amd import autodiff as ad, models
    from tinyflow_amd.SwapExecute import plan_schedule
    from tinyflow_amd.TrainExecute import getcomputelist, swapsgd
    rng = np.random.RandomState(0)
    model = models.resnet(rng, [1, 1, 1, 1], 4, image=32, n_class=10, width=8)
    variables = ad.get_Variable_node_list(model.loss)
    variables.reverse()
    grads = ad.gradients(model.loss, variables)
    topo = swapsgd(ad.find_topo_sort(getcomputelist(variables, grads, 0.1)))
    forward = set(ad.find_topo_sort([model.loss]))
    keep = set(n for n in topo if n.isw in (1, 2)) | {model.loss}
    cheap = lambda n: isinstance(n.op, (ad.BNForwardOp, ad.ActivationForwardOp))
    swap_out, swap_in, release, recompute = plan_schedule(topo, forward, keep, lambda n: True, 4, recomputable=cheap)
    pos = {n: i for i, n in enumerate(topo)}
    uses = {n: [] for n in topo}
    for n in topo:
        for inp in n.inputs:
            uses[inp].append(pos[n])
    first_backward = min(pos[n] for n in topo if n not in forward and n.isw not in (1, 2))
    rec_at = {n: t for t, ns in recompute.items() for n in ns}
    out_at = {n: t for t, ns in swap_out.items() for n in ns}
    in_at = {n: t for t, ns in swap_in.items() for n in ns}
    assert rec_at, "nothing is recomputed"
    assert not set(rec_at) & set(out_at), "a recomputed value is also swapped"
    n_bn = sum(isinstance(n.op, ad.BNForwardOp) for n in rec_at)
    n_act = sum(isinstance(n.op, ad.ActivationForwardOp) for n in rec_at)
    assert n_bn > 0 and n_act > 0

    def chain(n):
        return 0 if n not in rec_at else 1 + max(chain(i) for i in n.inputs)

    for n, t in rec_at.items():
        assert cheap(n) and n in forward and n not in keep
        bwd = [u for u in uses[n] if u >= first_backward]
        assert t >= first_backward and t <= min(bwd)
        assert 1 <= chain(n) <= 2
        for inp in n.inputs:
            if inp in rec_at:
                assert rec_at[inp] <= t
                if rec_at[inp] == t:   # same trigger: the producer is listed first
                    order = recompute[t]
                    assert order.index(inp) < order.index(n)
            if inp in in_at:
                assert in_at[inp] < t, "input is prefetched only after the recomputation needs it"
        # released once after the forward pass and once for good
        rel = sorted(t2 for t2, ns in release.items() if n in ns)
        assert len(rel) == 2 and rel[0] < first_backward <= rel[1] and rel[0] < t <= rel[1]
