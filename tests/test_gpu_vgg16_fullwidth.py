"""VGG-16 at its real width (64 ... 512 channels, 25088-4096-4096-1000 classifier) and
resolution (3x224x224), batch 2, one training step end to end against the CPU oracle.

tests/test_gpu_conv_fullsize.py holds every VGG-16 layer to the oracle at batch 32 one
layer at a time, and tests/test_gpu_train_step.py runs a narrow VGG; this is the whole
graph at the widths and map sizes of the benchmark configuration (so with the tile
shapes, split counts and Winograd forms the launch planner picks there -- all thirteen
convolutions but the first are 3x3 / stride-1 layers with at least 64 channels), with
only the batch reduced so that the float64 oracle finishes in half a minute.

Checked: the loss within rtol 1e-5 of the float64 oracle; the classifier's gradients
(nothing but matrix products between them and the loss) within 3 x the float32 CPU
oracle's own distance from float64; every convolution gradient in relative L2 within
2e-2.  The convolution bound is not a rounding bound.  Fed with the oracle's own
tensors, every one of these layers' grad-data and grad-filter is within 4e-7 (direct
form) / 2e-6 (F(4x4)) of float64, like the float32 CPU evaluation.  End to end, the
forward activations differ from float64 by fp32 rounding, and among the 25 million
ReLU inputs and 6 million pooling windows a handful (measured: 0-4 per layer) lie
closer to zero, or to their window's runner-up, than that rounding: there the ReLU
mask or the arg-max flips, one element of the upstream gradient moves by its whole
value, and the relative L2 distance of everything below jumps by about sqrt(1 / elements)
of that tensor's energy share (3e-4 at the first flip, 4e-3 after the third pooling
layer).  Which elements flip depends on the rounding of the evaluation, so a float32
CPU evaluation flips others (or, in this sample, none).  Distances are recorded per
tensor (tests/parity.py).
"""
import ctypes

import numpy as np
import pytest

from oracle import models as OM
import parity

pytestmark = pytest.mark.gpu


def _rel(got, ref):
    ref = np.asarray(ref, dtype=np.float64).ravel()
    diff = np.asarray(got, dtype=np.float64).ravel() - ref
    return float(np.sqrt(np.dot(diff, diff)) / max(1e-30, np.sqrt(np.dot(ref, ref))))


def test_vgg16_full_width_step_matches_oracle():
    from tinyflow_amd import _base, models
    from tinyflow_amd import autodiff as ad
    from tinyflow_amd.TrainExecute import TrainExecutor
    lr = 0.01
    model, X, y = models.build("vgg16", batch=2)
    shapes = sorted(tuple(v.shape) for v in model.variables.values())
    assert X.shape == (2, 3, 224, 224) and (512, 512, 3, 3) in shapes and (25088, 4096) in shapes
    ex = TrainExecutor(model.loss, lr)
    ex.init_Variable(dict(model.variables))
    out = ex.run({model.X: X, model.y_: y})
    loss = out[0].asnumpy()

    forms = []
    for node in ex.topo_order:
        if isinstance(node.op, ad.Convolution2DForwardOp) and getattr(node, "cudnnlist", None):
            buf = ctypes.create_string_buffer(256)
            for which in range(3):
                assert _base._LIB.DLGpuConvolutionDescribeKernel(node.cudnnlist[0], which, buf, 256, None) == 0
                forms.append(buf.value.decode())
    n_wino = sum("winograd" in f for f in forms)

    net = OM.network("vgg16", image=224)
    p64 = {v.name: val.astype(np.float64) for v, val in model.variables.items()}
    p32 = {v.name: val for v, val in model.variables.items()}
    loss64, grads64, new64 = OM.train_step(net, p64, X.astype(np.float64), y.astype(np.float64), lr)[:3]
    loss32, grads32, new32 = OM.train_step(net, p32, X, y, lr)[:3]
    np.testing.assert_allclose(loss, loss64, rtol=1e-5)
    grad_nodes = dict(zip(ex.Variable_node_list, ex.Variable_node_grad_list))
    worst = 0.0
    family = "train step vgg16 full width b2"
    for var, g in grad_nodes.items():
        got = ex.value_of(g).asnumpy()
        cpu_gap = _rel(grads32[var.name], grads64[var.name])
        err = _rel(got, grads64[var.name])
        worst = max(worst, err)
        parity.compare(got, grads64[var.name], grads32[var.name], family + ", gradients", var.name, 3.0,
                       assert_ratio=False)
        bound = 3 * cpu_gap if var.name.startswith("fc") else 2e-2
        assert err <= bound, "gradient of %s: relative L2 %.3g, fp32 CPU oracle %.3g" % (var.name, err, cpu_gap)
    for arr, var in zip(out[1:], model.variables):
        old = model.variables[var].astype(np.float64)
        bound = 3 * _rel(grads32[var.name], grads64[var.name]) if var.name.startswith("fc") else 2e-2
        assert _rel(arr.asnumpy().astype(np.float64) - old, new64[var.name] - old) <= bound + 1e-5, var.name
    print("%d of %d conv launches in a Winograd form, loss %.6f (oracle %.6f), worst gradient relative L2 %.2e"
          % (n_wino, len(forms), float(loss[0]), float(loss64[0]), worst))
    ex.close()


def test_vgg16_every_convolution_gradient_on_the_oracles_own_tensors():
    """The same network, one layer at a time: each convolution's grad-data and grad-filter
    evaluated by the library on the float64 oracle's own input, filter and upstream
    gradient (cast to float32), so that no ReLU mask or pooling arg-max lies between the
    two evaluations.  Bound: 24 x the distance of the float32 CPU evaluation of the same
    call from float64 (the planner runs these layers in a Winograd form; 16 x where it
    does not), which at these sizes is 1e-7 ... 4e-7."""
    from tinyflow_amd import _base, gpu_op, models, ndarray
    from oracle import ops as O
    model, X, y = models.build("vgg16", batch=2)
    net = OM.network("vgg16", image=224)
    p64 = {v.name: val.astype(np.float64) for v, val in model.variables.items()}
    logits = net.forward(X.astype(np.float64), p64)
    dy = O.softmax_cross_entropy_gradient(logits, y.astype(np.float64), 1.0)
    ctx = ndarray.gpu(0)
    stream = gpu_op.create_cudaStream()
    handle = gpu_op.create_cudnnHandle(stream)
    grads, checked = {}, 0
    for layer in reversed(net.layers):
        dx = layer.backward(dy, grads, True)
        if isinstance(layer, OM.Conv):
            x32, w32, dy32 = layer.x.astype(np.float32), layer.w.astype(np.float32), dy.astype(np.float32)
            _, lst = gpu_op.convolution_2d_forward_get_out_shape(x32.shape, w32.shape, "NCHW", layer.padding,
                                                                 layer.stride, layer.stride)
            gx, gw, gdy = ndarray.array(x32, ctx), ndarray.array(w32, ctx), ndarray.array(dy32, ctx)
            gdx, gdw = ndarray.empty(x32.shape, ctx), ndarray.empty(w32.shape, ctx)
            assert gpu_op.convolution_backward_data(gx, gdy, gw, gdx, lst, handle, stream) == 0
            assert gpu_op.convolution_backward_filter(gx, gdy, gw, gdw, lst, handle, stream) == 0
            cpu_dx = O.conv2d_backward_data(dy32, w32, x32.shape, layer.ph, layer.pw, layer.stride, layer.stride)
            cpu_dw = O.conv2d_backward_filter(x32, dy32, w32.shape, layer.ph, layer.pw, layer.stride, layer.stride)
            for which, got, ref, cpu in ((1, gdx.asnumpy(), dx, cpu_dx), (2, gdw.asnumpy(), grads[layer.name + "_W"], cpu_dw)):
                buf = ctypes.create_string_buffer(256)
                assert _base._LIB.DLGpuConvolutionDescribeKernel(lst, which, buf, 256, None) == 0
                k = 24.0 if "winograd" in buf.value.decode() else 16.0
                err, gap = _rel(got, ref), _rel(cpu, ref)
                parity.compare(got, ref, cpu, "vgg16 b2 layer gradients on the oracle's tensors", "%s %s" % (
                    layer.name, "grad-data" if which == 1 else "grad-filter"), k, assert_ratio=False)
                assert err <= k * gap, "%s %s: relative L2 %.3g, fp32 CPU oracle %.3g" % (
                    layer.name, "grad-data" if which == 1 else "grad-filter", err, gap)
                checked += 1
        dy = dx
    assert checked == 26
