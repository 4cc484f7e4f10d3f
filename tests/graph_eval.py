"""Numpy evaluator of a tinyflow_amd.autodiff graph -- test helper.

Walks any list of graph nodes in topological order and computes each node with
the CPU oracle's per-op functions, dispatching on the op's class.  It lets the
CPU test-suite run the product's graph construction (ops' ``gradient`` methods,
``gradients``, ``swapsgd``) without a GPU and compare the result with the
layer-by-layer oracle networks, which share no code with it.
"""
import numpy as np

from oracle import ops as O
from tinyflow_amd import autodiff as ad


def _conv_geometry(node, w_shape):
    return O.conv_pad(w_shape[2], node.padding), O.conv_pad(w_shape[3], node.padding), node.u, node.v


def evaluate(nodes, feed):
    """{node: value} for every node reachable from ``nodes``; ``feed`` gives the
    placeholders.  SGD nodes update their parameter's entry in place."""
    val = dict(feed)
    for node in nodes if isinstance(nodes, list) and getattr(nodes, "_ordered", False) else ad.find_topo_sort(nodes):
        if node in val:
            continue
        op, ins = node.op, [val[i] for i in node.inputs]
        if isinstance(op, ad.AddOp):
            out = O.add(ins[0], ins[1]) if ins[0].shape == ins[1].shape else ins[0] + ins[1].reshape(())
        elif isinstance(op, ad.AddByConstOp):
            out = O.add_by_const(ins[0], node.const_attr)
        elif isinstance(op, ad.MulOp):
            if ins[0].shape == ins[1].shape:
                out = O.multiply(ins[0], ins[1])
            else:
                big, small = (ins[0], ins[1]) if ins[1].shape == (1,) else (ins[1], ins[0])
                out = O.multiply_by_const(big, small[0])
        elif isinstance(op, ad.MulByConstOp):
            out = O.multiply_by_const(ins[0], node.const_attr)
        elif isinstance(op, ad.MatMulOp):
            out = O.matmul(ins[0], node.matmul_attr_trans_A, ins[1], node.matmul_attr_trans_B)
        elif isinstance(op, ad.ZerosLikeOp):
            out = np.zeros_like(ins[0])
        elif isinstance(op, ad.OnesLikeOp):
            out = np.ones_like(ins[0])
        elif isinstance(op, ad.ReduceSumAxisZeroOp):
            out = O.reduce_sum_axis_zero(ins[0]).reshape(-1) if ins[0].ndim == 1 else O.reduce_sum_axis_zero(ins[0])
        elif isinstance(op, ad.BroadcastToOp):
            out = (O.broadcast_to_channel(ins[0], ins[1].shape) if node.type == "NCHW"
                   else O.broadcast_to_trailing(ins[0], ins[1].shape))
        elif isinstance(op, ad.BroadcastToGradientOp):
            out = O.bias_gradient(ins[0], node.type).reshape(ins[1].shape)
        elif isinstance(op, ad.SoftmaxCrossEntropyOp):
            out = O.softmax_cross_entropy(ins[0], ins[1])
        elif isinstance(op, ad.SoftmaxOp):
            out = O.softmax(ins[0])
        elif isinstance(op, ad.ReluOp):
            out = O.relu(ins[0])
        elif isinstance(op, ad.ReluGradientOp):
            out = O.relu_gradient(ins[0], ins[1])
        elif isinstance(op, ad.CrossOp):
            scale = 1.0 / ins[0].size if node.ismean else 1.0
            out = O.cross(ins[0], ins[1], scale)
        elif isinstance(op, ad.CrossBackwardOp):
            # the scale cell is filled by infer_shape in the product; recompute it here
            out = O.cross_backward(ins[0], ins[1], ins[2].reshape(()) * np.ones_like(ins[0])
                                   if ins[2].shape == (1,) else ins[2], node.meanfloat[0])
        elif isinstance(op, ad.ReduceSumOp):
            out = np.sum(ins[0]).reshape(1)
        elif isinstance(op, ad.Convolution2DForwardOp):
            ph, pw, u, v = _conv_geometry(node, ins[1].shape)
            out = O.conv2d_forward(ins[0], ins[1], ph, pw, u, v)
        elif isinstance(op, ad.Convolution2DBackwardOp):
            ph, pw, u, v = _conv_geometry(node, ins[1].shape)
            if node.type == 0:
                out = O.conv2d_backward_data(ins[2], ins[1], ins[0].shape, ph, pw, u, v)
            else:
                out = O.conv2d_backward_filter(ins[0], ins[2], ins[1].shape, ph, pw, u, v)
        elif isinstance(op, ad.FlattenOp):
            out = ins[0].reshape(ins[0].shape[0], -1)
        elif isinstance(op, ad.FlattenGradientOp):
            out = ins[1].reshape(ins[0].shape)
        elif isinstance(op, ad.ActivationForwardOp):   # also FullyActivationForwardOp
            out = O.activation_forward(ins[0], node.activationMode)
        elif isinstance(op, ad.ActivationBackwardOp):
            out = O.activation_backward(ins[0], ins[2], ins[1], node.activationMode)
        elif isinstance(op, ad.Pooling2DForwardOp):
            f = (O.max_pool_forward if node.poolingMode == "max" else O.avg_pool_forward)
            out = f(ins[0], node.filter_h, node.filter_w, node.pad_h, node.pad_w, node.u, node.v)
        elif isinstance(op, ad.Pooling2DBackwardOp):
            fwd = node.inputs[2]
            geo = (fwd.filter_h, fwd.filter_w, fwd.pad_h, fwd.pad_w, fwd.u, fwd.v)
            if fwd.poolingMode == "max":
                out = O.max_pool_backward(ins[0], ins[1], *geo)
            else:
                out = O.avg_pool_backward(ins[0].shape, ins[1], *geo)
        elif isinstance(op, ad.BNForwardOp):           # also FullyBNForwardOp
            out = O.batch_norm_forward(ins[0], node.batchNormMode)[0]
        elif isinstance(op, ad.BNBackwardOp):
            out = O.batch_norm_backward(ins[0], ins[1], node.batchNormMode)
        elif isinstance(op, ad.SgdOp):
            val[node.inputs[0]] = O.sgd_update(ins[0], ins[1], node.learning_rate)
            out = None
        else:
            raise NotImplementedError(type(op).__name__)
        val[node] = out
    return val


def evaluate_in_order(order, feed):
    """Like ``evaluate`` but follows a given execution order (e.g. the executor's
    ``topo_order``), so in-place updates happen exactly where the product does them."""
    val = dict(feed)
    for node in order:
        if node in val:
            continue
        sub = evaluate([node], {k: v for k, v in val.items() if k is not node})
        for k, v in sub.items():
            if k not in val or isinstance(k.op, ad.PlaceholderOp):
                val[k] = v
        if node.issgd:
            val[node.inputs[0]] = sub[node.inputs[0]]
    return val
