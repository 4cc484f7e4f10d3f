"""Computation graph, reverse-mode differentiation and the operators of the
training hot path.

Host-side counterpart of the reference ``pycode/tinyflow/autodiff.py`` for the
path this package accelerates.  It keeps the reference's public names and
conventions -- op singletons (``matmul_op``, ``convolution_2d_forward_op``, ...),
``Variable`` / ``Placeholder``, ``Op.compute(node, input_vals, output_val,
cudnnHandle, cublasHandle, cudaStream)``, ``Op.gradient`` emitting backward
nodes, ``Op.infer_shape`` creating the C-side descriptors, ``gradients`` and
``find_topo_sort`` -- so model code written for the reference builds the same
graph, which decides which C entry points run, in which order, on which shapes.

Every ``compute`` goes through ``gpu_op`` into libc_runtime_api.so; there is no
numpy branch (the reference keeps one for a subset of ops, autodiff.py:312-779).
"""
import random
from functools import reduce
from operator import add

from . import gpu_op, ndarray


class Node(object):
    """A value in the graph: the op that produces it and its input nodes."""

    def __init__(self):
        self.inputs = []
        self.op = None
        self.const_attr = None
        self.name = ""
        self.index = 0
        # 1: trainable Variable, 2: fed Placeholder, 3: optimizer node already
        # moved behind the last reader of its parameter (reference autodiff.py:218-237)
        self.isw = 0
        self.issgd = 0

    def __add__(self, other):
        if isinstance(other, Node):
            return add_op(self, other)
        return add_byconst_op(self, other)

    def __mul__(self, other):
        if isinstance(other, Node):
            return mul_op(self, other)
        return mul_byconst_op(self, other)

    __radd__ = __add__
    __rmul__ = __mul__

    def __str__(self):
        return self.name

    __repr__ = __str__


def Variable(name):
    """Trainable parameter (fed once, then updated in place by the optimizer)."""
    node = placeholder_op()
    node.name = name
    node.isw = 1
    return node


def Placeholder(name):
    """Per-step input (data, labels)."""
    node = placeholder_op()
    node.name = name
    node.isw = 2
    return node


class Op(object):
    """Operator: creates nodes, computes them, differentiates them."""

    def __call__(self):
        node = Node()
        node.op = self
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        """Write the node's value into ``output_val``; returns 0, or the number of
        scratch bytes that could not be allocated."""
        raise NotImplementedError

    def gradient(self, node, output_grad):
        """Nodes computing the gradient with respect to each input."""
        raise NotImplementedError

    def infer_shape(self, node, input_shapes, cudnnHandle):
        raise NotImplementedError


def _no_numpy(use_numpy):
    assert not use_numpy, "this build has no CPU path: ops run on the GPU only"


# ------------------------------------------------------------------ arithmetic

class AddOp(Op):
    """reference autodiff.py:302-348"""

    def __call__(self, node_A, node_B):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "+"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        a, b = input_vals
        if a.shape == b.shape:
            gpu_op.matrix_elementwise_add(a, b, output_val, cudaStream)
        elif b.shape == (1,):
            # a (1,) operand is read back to the host and applied as a constant
            gpu_op.matrix_elementwise_add_by_const(a, b.asnumpy()[0], output_val, cudaStream)
        elif a.shape == (1,):
            gpu_op.matrix_elementwise_add_by_const(b, a.asnumpy()[0], output_val, cudaStream)
        else:
            raise ValueError("add: incompatible shapes %s and %s" % (a.shape, b.shape))
        return 0

    def gradient(self, node, output_grad):
        return [output_grad, output_grad]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        a, b = input_shapes
        if a == b:
            return a
        return b if a == (1,) else a


class AddByConstOp(Op):
    """reference autodiff.py:351-373"""

    def __call__(self, node_A, const_val):
        node = Op.__call__(self)
        node.const_attr = const_val
        node.inputs = [node_A]
        node.name = "+"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.matrix_elementwise_add_by_const(input_vals[0], node.const_attr, output_val, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [output_grad]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class MulOp(Op):
    """reference autodiff.py:376-413"""

    def __call__(self, node_A, node_B):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "*"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        a, b = input_vals
        if a.shape == b.shape:
            gpu_op.matrix_elementwise_multiply(a, b, output_val, cudaStream)
        elif b.shape == (1,):
            gpu_op.matrix_elementwise_multiply_by_const(a, b.asnumpy()[0], output_val, cudaStream)
        elif a.shape == (1,):
            gpu_op.matrix_elementwise_multiply_by_const(b, a.asnumpy()[0], output_val, cudaStream)
        else:
            raise ValueError("mul: incompatible shapes %s and %s" % (a.shape, b.shape))
        return 0

    def gradient(self, node, output_grad):
        return [node.inputs[1] * output_grad, node.inputs[0] * output_grad]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        a, b = input_shapes
        if a == b:
            return a
        return b if a == (1,) else a


class MulByConstOp(Op):
    """reference autodiff.py:416-438"""

    def __call__(self, node_A, const_val):
        node = Op.__call__(self)
        node.const_attr = const_val
        node.inputs = [node_A]
        node.name = "*"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.matrix_elementwise_multiply_by_const(input_vals[0], node.const_attr, output_val, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [node.const_attr * output_grad]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class MatMulOp(Op):
    """C = op(A) op(B) and its two gradients (reference autodiff.py:441-516)."""

    def __call__(self, node_A, node_B, trans_A=False, trans_B=False):
        node = Op.__call__(self)
        node.matmul_attr_trans_A = trans_A
        node.matmul_attr_trans_B = trans_B
        node.inputs = [node_A, node_B]
        node.name = "MatMul"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.matrix_multiply(input_vals[0], node.matmul_attr_trans_A, input_vals[1],
                               node.matmul_attr_trans_B, output_val, cublasHandle, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        A, B = node.inputs
        tA, tB = node.matmul_attr_trans_A, node.matmul_attr_trans_B
        if not tA and not tB:    # Y = A B:      dA = dY B^T,     dB = A^T dY
            return [matmul_op(output_grad, B, False, True), matmul_op(A, output_grad, True, False)]
        if tA and not tB:        # Y = A^T B:    dA = B dY^T,     dB = A dY
            return [matmul_op(B, output_grad, False, True), matmul_op(A, output_grad, False, False)]
        if not tA and tB:        # Y = A B^T:    dA = dY B,       dB = dY^T A
            return [matmul_op(output_grad, B, False, False), matmul_op(output_grad, A, True, False)]
        # Y = A^T B^T:           dA = B^T dY^T,  dB = dY^T A^T
        return [matmul_op(B, output_grad, True, True), matmul_op(output_grad, A, True, True)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        a, b = input_shapes
        rows = a[1] if node.matmul_attr_trans_A else a[0]
        cols = b[0] if node.matmul_attr_trans_B else b[1]
        return (rows, cols)


class PlaceholderOp(Op):
    def __call__(self):
        return Op.__call__(self)

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        assert False, "placeholder %s values provided by feed_dict" % node.name

    def gradient(self, node, output_grad):
        return None

    def infer_shape(self, node, input_shapes, cudnnHandle):
        assert False, "placeholder %s shape provided by feed_shape" % node.name


class ZerosLikeOp(Op):
    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "Zeroslike"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.array_set(output_val, 0, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [zeroslike_op(node.inputs[0])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class OnesLikeOp(Op):
    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "Oneslike"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.array_set(output_val, 1, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [zeroslike_op(node.inputs[0])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class ReduceSumAxisZeroOp(Op):
    """reference autodiff.py:587-618"""

    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "ReduceSumAxisZero"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.reduce_sum_axis_zero(input_vals[0], output_val)
        return 0

    def gradient(self, node, output_grad):
        return [broadcastto_op(output_grad, node.inputs[0])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        if len(input_shapes[0]) == 1:
            return (1,)
        return tuple(input_shapes[0][1:])


class BroadcastToOp(Op):
    """Bias broadcast: "NHWC" = along the trailing dims (FC bias), "NCHW" = per
    channel (conv bias).  reference autodiff.py:621-645"""

    def __call__(self, node_A, node_B, type="NHWC"):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "BroadcastTo"
        node.type = type
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.broadcast_to(input_vals[0], output_val, node.type, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [broadcastto_gradient_op(output_grad, node.inputs[0], node.type), zeroslike_op(node.inputs[1])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[1]


class BroadcastToGradientOp(Op):
    """Bias gradient: sum of the upstream gradient over every non-bias dim.
    reference autodiff.py:648-678"""

    def __call__(self, node_A, node_B, type):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "BroadcastToGradient"
        node.type = type
        node.cudnnlist = [0]
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        return gpu_op.reduce_sum_new(input_vals[0], output_val, node.cudnnlist[0], cudnnHandle, cudaStream)

    def infer_shape(self, node, input_shapes, cudnnHandle):
        in_shape, out_shape = gpu_op.reduce_sum_get_real_shape(input_shapes[0], input_shapes[1], node.type)
        node.cudnnlist[0] = gpu_op.reduce_sum_get_cudnnlist(in_shape, out_shape, node.type, cudnnHandle)
        return input_shapes[1]


# ------------------------------------------------------- softmax / cross entropy

class SoftmaxCrossEntropyOp(Op):
    """loss = mean_n(-sum_c y_ log softmax(y)); its gradient is
    (softmax(y) + -1*y_) * upstream, i.e. NOT divided by the batch size
    (reference autodiff.py:689-716)."""

    def __call__(self, node_A, node_B):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "SoftmaxXEntropy"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.softmax_cross_entropy(input_vals[0], input_vals[1], output_val, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        grad_A = (softmax_op(node.inputs[0]) + -1 * node.inputs[1]) * output_grad
        return [grad_A, zeroslike_op(node.inputs[1])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return (1,)


class SoftmaxOp(Op):
    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "Softmax"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.softmax(input_vals[0], output_val, cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class ReluOp(Op):
    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "Relu"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.relu(input_vals[0], output_val)
        return 0

    def gradient(self, node, output_grad):
        return [relu_gradient_op(node.inputs[0], output_grad)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class ReluGradientOp(Op):
    def __call__(self, node_A, node_B):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "ReluGradient"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.relu_gradient(input_vals[0], input_vals[1], output_val)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class CrossOp(Op):
    """-b * y_ * log(x); b = 1 / (number of elements of x) when ismean, else 1
    (reference autodiff.py:2079-2103)."""

    def __call__(self, node_A, node_B, ismean=True):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "CrossOp"
        node.ismean = ismean
        node.meanfloat = [1.0]  # shared with the backward node, filled by infer_shape
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.cross(input_vals[0], input_vals[1], output_val, node.meanfloat[0], cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [cross_backward_op(node.inputs[0], node.inputs[1], output_grad, node.meanfloat),
                zeroslike_op(node.inputs[1])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        if node.ismean:
            count = 1
            for extent in input_shapes[0]:
                count *= extent
            node.meanfloat[0] = 1.0 / count
        return input_shapes[0]


class CrossBackwardOp(Op):
    """inputs: x, y_, upstream (reference autodiff.py:2106-2123)"""

    def __call__(self, node_A, node_B, node_C, meanfloat):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B, node_C]
        node.name = "CrossBackwardOp"
        node.meanfloat = meanfloat
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.cross_backward(input_vals[0], input_vals[1], input_vals[2], output_val, node.meanfloat[0],
                              cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class ReduceSumOp(Op):
    """Sum of all elements to a (1,) array (reference autodiff.py:1503-1532)."""

    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "ReduceSumOp"
        node.type = "NHWC"
        node.cudnnlist = [0]
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        return gpu_op.reduce_sum_new(input_vals[0], output_val, node.cudnnlist[0], cudnnHandle, cudaStream)

    def gradient(self, node, output_grad):
        return [broadcastto_op(output_grad, node.inputs[0])]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        in_shape, out_shape = gpu_op.reduce_sum_get_real_shape(input_shapes[0], (1,), node.type)
        node.cudnnlist[0] = gpu_op.reduce_sum_get_cudnnlist(in_shape, out_shape, node.type, cudnnHandle)
        return (1,)


# ------------------------------------------------------------------ convolution

class Convolution2DForwardOp(Op):
    """reference autodiff.py:944-973"""

    def __call__(self, node_A, node_B, dataformat, padding, u, v):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "Convolution2DForward"
        node.dataformat = dataformat
        node.padding = padding
        node.u = u
        node.v = v
        node.cudnnlist = [0]  # shared (same list object) with both gradient nodes
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        return gpu_op.convolution_2d_forward(input_vals[0], input_vals[1], output_val, node.cudnnlist[0],
                                             cudnnHandle, cudaStream)

    def gradient(self, node, output_grad):
        x, w = node.inputs
        return [convolution_2d_backward_op(x, w, output_grad, 0, node.padding, node.u, node.v, node.cudnnlist),
                convolution_2d_backward_op(x, w, output_grad, 1, node.padding, node.u, node.v, node.cudnnlist)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        out_shape, node.cudnnlist[0] = gpu_op.convolution_2d_forward_get_out_shape(
            input_shapes[0], input_shapes[1], node.dataformat, node.padding, node.u, node.v)
        return out_shape


class Convolution2DBackwardOp(Op):
    """type 0: gradient w.r.t. the input, type 1: w.r.t. the filter
    (reference autodiff.py:976-1012)."""

    def __call__(self, node_A, node_B, node_C, type, padding, u, v, cudnnlist):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B, node_C]
        node.name = "Convolution2DBackward"
        node.type = type
        node.padding = padding
        node.u = u
        node.v = v
        node.cudnnlist = cudnnlist
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        x, w, dy = input_vals
        if node.type == 0:
            return gpu_op.convolution_backward_data(x, dy, w, output_val, node.cudnnlist[0], cudnnHandle,
                                                    cudaStream)
        return gpu_op.convolution_backward_filter(x, dy, w, output_val, node.cudnnlist[0], cudnnHandle,
                                                  cudaStream)

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0] if node.type == 0 else input_shapes[1]


class FlattenOp(Op):
    """(N, ...) -> (N, prod(...)) as a device copy (reference autodiff.py:1081-1102)."""

    def __call__(self, node_A):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "Flatten"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        input_vals[0].copyto(output_val, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [flatten_gradient_op(node.inputs[0], output_grad)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        inner = 1
        for extent in input_shapes[0][1:]:
            inner *= extent
        return (input_shapes[0][0], inner)


class FlattenGradientOp(Op):
    def __call__(self, node_A, node_B):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "FlattenGradient"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        input_vals[1].copyto(output_val, cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


# ------------------------------------------------------------------- activation

class ActivationForwardOp(Op):
    """reference autodiff.py:1124-1145"""

    def __call__(self, node_A, dataformat, activationMode):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "ActivationForward"
        node.dataformat = dataformat
        node.activationMode = activationMode
        node.cudnnlist = [0]
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.activation_forward(input_vals[0], output_val, node.activationMode, node.cudnnlist[0],
                                  cudnnHandle, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [activation_backward_op(node.inputs[0], output_grad, node, node.activationMode, node.cudnnlist)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        node.cudnnlist[0] = gpu_op.activation_get_cudnnlist(self._descriptor_shape(input_shapes[0]),
                                                            node.dataformat, node.activationMode)
        return input_shapes[0]

    @staticmethod
    def _descriptor_shape(shape):
        return shape


class ActivationBackwardOp(Op):
    """inputs: x, dy, y (reference autodiff.py:1148-1168)"""

    def __call__(self, node_A, node_B, node_C, activationMode, cudnnlist):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B, node_C]
        node.name = "ActivationBackward"
        node.activationMode = activationMode
        node.cudnnlist = cudnnlist
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        x, dy, y = input_vals
        gpu_op.activation_backward(x, output_val, y, dy, node.activationMode, node.cudnnlist[0], cudnnHandle,
                                   cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class FullyActivationForwardOp(ActivationForwardOp):
    """Activation of a 2-D (N, F) array, described to the C side as (N, 1, F)
    (reference autodiff.py:1447-1473)."""

    def __call__(self, node_A, dataformat, activationMode):
        node = ActivationForwardOp.__call__(self, node_A, dataformat, activationMode)
        node.name = "FullyActivationForward"
        return node

    def gradient(self, node, output_grad):
        return [fullyactivation_backward_op(node.inputs[0], output_grad, node, node.activationMode,
                                            node.cudnnlist)]

    @staticmethod
    def _descriptor_shape(shape):
        return (shape[0], 1, shape[1])


class FullyActivationBackwardOp(ActivationBackwardOp):
    def __call__(self, node_A, node_B, node_C, activationMode, cudnnlist):
        node = ActivationBackwardOp.__call__(self, node_A, node_B, node_C, activationMode, cudnnlist)
        node.name = "FullyActivationBackward"
        return node


# ---------------------------------------------------------------------- pooling

class Pooling2DForwardOp(Op):
    """reference autodiff.py:1223-1255"""

    def __call__(self, node_A, dataformat, poolingMode, pad_h, pad_w, u, v, filter_h, filter_w):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "Pooling2DForward"
        node.dataformat = dataformat
        node.poolingMode = poolingMode
        node.pad_h, node.pad_w = pad_h, pad_w
        node.u, node.v = u, v
        node.filter_h, node.filter_w = filter_h, filter_w
        node.cudnnlist = [0]
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.pooling_2d_forward(input_vals[0], output_val, node.cudnnlist[0], cudnnHandle, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [pooling_2d_backward_op(node.inputs[0], output_grad, node, node.cudnnlist)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        out_shape, node.cudnnlist[0] = gpu_op.pooling_2d_forward_get_out_shape(
            input_shapes[0], node.dataformat, node.poolingMode, node.pad_h, node.pad_w, node.u, node.v,
            node.filter_h, node.filter_w)
        return out_shape


class Pooling2DBackwardOp(Op):
    """inputs: x, dy, y (reference autodiff.py:1258-1276)"""

    def __call__(self, node_A, node_B, node_C, cudnnlist):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B, node_C]
        node.name = "Pooling2DBackward"
        node.cudnnlist = cudnnlist
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        x, dy, y = input_vals
        gpu_op.pooling_2d_backward(x, y, dy, output_val, node.cudnnlist[0], cudnnHandle, cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


# ----------------------------------------------------------- batch normalisation

class BNForwardOp(Op):
    """gamma = 1, beta = 0 batch normalisation; ``batchNormMode`` is
    "pre_activation" (per-activation statistics) or "spatial"
    (reference autodiff.py:1820-1850)."""

    def __call__(self, node_A, dataformat, batchNormMode):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "BNForward"
        node.dataformat = dataformat
        node.batchNormMode = batchNormMode
        node.Save_p = [0, 0]   # cells holding the saved mean / inverse std, shared with the backward node
        node.n = 0
        node.cudnnlist = [0]
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        wanted = gpu_op.bn_forward(input_vals[0], output_val, node.batchNormMode, node.n, node.Save_p[0],
                                   node.Save_p[1], node.cudnnlist[0], cudnnHandle, cudaStream)
        node.n += 1
        return wanted

    def gradient(self, node, output_grad):
        return [bn_backward_op(node.inputs[0], output_grad, node.batchNormMode, node.Save_p, node.cudnnlist)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        node.Save_p[0], node.Save_p[1], node.cudnnlist[0] = gpu_op.bn_get_cudnnlist(
            self._descriptor_shape(input_shapes[0]), node.dataformat, node.batchNormMode)
        return input_shapes[0]

    @staticmethod
    def _descriptor_shape(shape):
        return shape


class BNBackwardOp(Op):
    """inputs: x, dy (reference autodiff.py:1853-1875)"""

    def __call__(self, node_A, node_B, batchNormMode, Save_p, cudnnlist):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "BNBackward"
        node.Save_p = Save_p
        node.batchNormMode = batchNormMode
        node.cudnnlist = cudnnlist
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        return gpu_op.bn_backward(input_vals[0], input_vals[1], output_val, node.batchNormMode, node.Save_p[0],
                                  node.Save_p[1], node.cudnnlist[0], cudnnHandle, cudaStream)

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class FullyBNForwardOp(BNForwardOp):
    """Per-activation batch norm of a 2-D (N, F) array, described to the C side
    as (N, 1, F) (reference autodiff.py:1878-1909)."""

    def __call__(self, node_A, dataformat):
        node = BNForwardOp.__call__(self, node_A, dataformat, "pre_activation")
        node.name = "FullyBNForward"
        return node

    @staticmethod
    def _descriptor_shape(shape):
        return (shape[0], 1, shape[1])


# -------------------------------------------------------------------- optimizer

class SgdOp(Op):
    """In-place w -= lr * g; produces no value of its own (reference autodiff.py:2028-2047)."""

    def __call__(self, node_A, node_B, learning_rate):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "SgdOp"
        node.learning_rate = learning_rate
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.sgd_update(input_vals[0], input_vals[1], node.learning_rate, cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class AdamOp(Op):
    """In-place Adam update of a parameter and its two moment variables; produces no
    value of its own (reference autodiff.py:2050-2076).  Inputs: parameter, m, v,
    gradient.  ``b1t`` / ``b2t`` are one-element lists shared with the executor,
    which multiplies them by b1 / b2 after every step."""

    def __call__(self, node_A, node_B, node_C, node_D, b1, b2, b1t, b2t, e, learning_rate):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B, node_C, node_D]
        node.name = "AdamOp"
        node.b1, node.b2, node.b1t, node.b2t, node.e = b1, b2, b1t, b2t, e
        node.learning_rate = learning_rate
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.adam_mv(input_vals[1], input_vals[2], input_vals[3], node.b1, node.b2, cudaStream)
        gpu_op.adam_compute(input_vals[0], input_vals[1], input_vals[2], node.b1t[0], node.b2t[0], node.e,
                            node.learning_rate, cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


# ------------------------------------------------------------------- composites

def dense(X, W, b):
    """X W + broadcast(b)   (reference autodiff.py:2126-2129)"""
    xw = matmul_op(X, W)
    return xw + broadcastto_op(b, xw)


def conv2withbias(input, filter, bias, dataformat, padding, strideh, stridew):
    """conv(input, filter) + per-channel bias   (reference autodiff.py:2139-2143)"""
    c = convolution_2d_forward_op(input, filter, dataformat, padding, strideh, stridew)
    return c + broadcastto_op(bias, c, dataformat)


def crossEntropy_loss(input, y_, ismean=True):
    """sum(-b * y_ * log(input)): the loss head of the reference's model scripts,
    applied to softmax probabilities (reference autodiff.py:2153-2156)"""
    return reduce_sum_op(cross_op(input, y_, ismean))


# ------------------------------------------------------------------- singletons

add_op = AddOp()
mul_op = MulOp()
add_byconst_op = AddByConstOp()
mul_byconst_op = MulByConstOp()
matmul_op = MatMulOp()
placeholder_op = PlaceholderOp()
oneslike_op = OnesLikeOp()
zeroslike_op = ZerosLikeOp()
# ------------------------------------------------------- dropout, concatenation

class DropoutForwardOp(Op):
    """reference autodiff.py:1337-1365.  A fresh seed is drawn from Python's
    ``random`` module on every evaluation, as there."""

    def __call__(self, node_A, dataformat, dropout):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "DropoutForward"
        node.dataformat = dataformat
        node.dropout = dropout
        node.seed = [0]
        node.reserveSpace_p = [0]
        node.cudnnlist = [0]
        node.inputd = [0]
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        node.seed[0] = random.randint(0, 100)
        node.reserveSpace_p[0], node.cudnnlist[0], wanted = gpu_op.dropout_forward(
            input_vals[0], output_val, node.dataformat, node.dropout, node.seed[0], node.inputd[0], cudnnHandle,
            cudaStream)
        return wanted

    def gradient(self, node, output_grad):
        return [dropout_backward_op(output_grad, node.dropout, node.reserveSpace_p, node.cudnnlist)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        node.inputd[0] = gpu_op.get_input_descriptor(self._descriptor_shape(input_shapes[0]), node.dataformat)
        return input_shapes[0]

    @staticmethod
    def _descriptor_shape(shape):
        return shape


class DropoutBackwardOp(Op):
    """reference autodiff.py:1368-1387"""

    def __call__(self, node_A, dropout, reserveSpace_p, cudnnlist):
        node = Op.__call__(self)
        node.inputs = [node_A]
        node.name = "DropoutBackward"
        node.dropout = dropout
        node.reserveSpace_p = reserveSpace_p
        node.cudnnlist = cudnnlist
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.dropout_backward(input_vals[0], output_val, node.reserveSpace_p[0], node.cudnnlist[0], cudnnHandle,
                                cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[0]


class FullyDropoutForwardOp(DropoutForwardOp):
    """Dropout on an (N, F) matrix, described as (N, 1, F) (reference autodiff.py:1390-1422)."""

    def __call__(self, node_A, dataformat, dropout):
        node = DropoutForwardOp.__call__(self, node_A, dataformat, dropout)
        node.name = "FullyDropoutForward"
        return node

    def gradient(self, node, output_grad):
        return [fullydropout_backward_op(output_grad, node.dropout, node.reserveSpace_p, node.cudnnlist)]

    @staticmethod
    def _descriptor_shape(shape):
        return (shape[0], 1, shape[1])


class FullyDropoutBackwardOp(DropoutBackwardOp):
    """reference autodiff.py:1425-1445"""

    def __call__(self, node_A, dropout, reserveSpace_p, cudnnlist):
        node = DropoutBackwardOp.__call__(self, node_A, dropout, reserveSpace_p, cudnnlist)
        node.name = "FullyDropoutBackward"
        return node


class ConcatForwardOp(Op):
    """Concatenation along axis 1 (reference autodiff.py:1935-1956)."""

    def __call__(self, node_A, node_B):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B]
        node.name = "ConcatForward"
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        gpu_op.concat_forward(input_vals[0], input_vals[1], output_val, cudaStream)
        return 0

    def gradient(self, node, output_grad):
        return [concat_backward_op(node.inputs[0], node.inputs[1], output_grad, 0),
                concat_backward_op(node.inputs[0], node.inputs[1], output_grad, 1)]

    def infer_shape(self, node, input_shapes, cudnnHandle):
        shape = list(input_shapes[0])
        shape[1] = input_shapes[0][1] + input_shapes[1][1]
        return tuple(shape)


class ConcatBackwardOp(Op):
    """inputs: a, b, d(concat); type 0 / 1 selects the slice for a / b
    (reference autodiff.py:1959-1984)."""

    def __call__(self, node_A, node_B, node_C, type):
        node = Op.__call__(self)
        node.inputs = [node_A, node_B, node_C]
        node.name = "Concatbackward"
        node.type = type
        return node

    def compute(self, node, input_vals, output_val, cudnnHandle, cublasHandle, cudaStream, use_numpy=False):
        _no_numpy(use_numpy)
        fn = gpu_op.concat_a_backward if node.type == 0 else gpu_op.concat_b_backward
        fn(input_vals[0], input_vals[1], input_vals[2], output_val, cudaStream)
        return 0

    def infer_shape(self, node, input_shapes, cudnnHandle):
        return input_shapes[node.type]


reducesumaxiszero_op = ReduceSumAxisZeroOp()
broadcastto_op = BroadcastToOp()
broadcastto_gradient_op = BroadcastToGradientOp()
softmaxcrossentropy_op = SoftmaxCrossEntropyOp()
softmax_op = SoftmaxOp()
relu_op = ReluOp()
relu_gradient_op = ReluGradientOp()
cross_op = CrossOp()
cross_backward_op = CrossBackwardOp()
reduce_sum_op = ReduceSumOp()
convolution_2d_forward_op = Convolution2DForwardOp()
convolution_2d_backward_op = Convolution2DBackwardOp()
flatten_op = FlattenOp()
flatten_gradient_op = FlattenGradientOp()
activation_forward_op = ActivationForwardOp()
activation_backward_op = ActivationBackwardOp()
fullyactivation_forward_op = FullyActivationForwardOp()
fullyactivation_backward_op = FullyActivationBackwardOp()
pooling_2d_forward_op = Pooling2DForwardOp()
pooling_2d_backward_op = Pooling2DBackwardOp()
bn_forward_op = BNForwardOp()
bn_backward_op = BNBackwardOp()
fullybn_forward_op = FullyBNForwardOp()
sgd_op = SgdOp()
adam_op = AdamOp()
dropout_forward_op = DropoutForwardOp()
dropout_backward_op = DropoutBackwardOp()
fullydropout_forward_op = FullyDropoutForwardOp()
fullydropout_backward_op = FullyDropoutBackwardOp()
concat_forward_op = ConcatForwardOp()
concat_backward_op = ConcatBackwardOp()


# ---------------------------------------------------------------- autodiff core

def gradients(output_node, node_list):
    """Gradient nodes of ``output_node`` w.r.t. each node of ``node_list``.

    Reverse topological sweep; the partial adjoints of a node with several
    consumers are combined by a left-to-right chain of add nodes, which fixes the
    fp32 summation order (reference autodiff.py:2894-2925, 3024-3028)."""
    node_to_output_grads_list = {output_node: [oneslike_op(output_node)]}
    node_to_output_grad = {}
    for node in reversed(find_topo_sort([output_node])):
        output_grad = sum_node_list(node_to_output_grads_list[node])
        node_to_output_grad[node] = output_grad
        input_grads = node.op.gradient(node, output_grad)
        for i, inp in enumerate(node.inputs):
            node_to_output_grads_list.setdefault(inp, []).append(input_grads[i])
    return [node_to_output_grad[node] for node in node_list]


def find_topo_sort(node_list):
    """Post-order DFS over input edges: every node appears after its inputs."""
    visited = set()
    topo_order = []
    for root in node_list:
        # iterative DFS: deep networks would exhaust the recursion limit
        stack = [(root, 0)]
        while stack:
            node, next_input = stack.pop()
            if next_input == 0:
                if node in visited:
                    continue
                visited.add(node)
            if next_input < len(node.inputs):
                stack.append((node, next_input + 1))
                child = node.inputs[next_input]
                if child not in visited:
                    stack.append((child, 0))
            else:
                topo_order.append(node)
    return topo_order


def sum_node_list(node_list):
    return reduce(add, node_list)


def get_Variable_node_list(node):
    """Trainable variables below ``node`` in first-use (post-order) order."""
    return [n for n in find_topo_sort([node]) if n.isw == 1]
