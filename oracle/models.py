"""CPU oracle: whole training steps of the benchmark networks -- TEST
INFRASTRUCTURE, NOT PRODUCT CODE (see oracle/ops.py for the rules).

An independent, layer-by-layer numpy implementation (explicit forward caches and
hand-written backward passes, no graph, no autodiff) of the same networks that
tinyflow_amd.models builds as graphs, so that a step of the product -- graph
construction, reverse-mode differentiation, gradient accumulation at residual
joins, update placement, every kernel -- can be compared end to end with
something that shares none of that machinery.  The arithmetic of each layer is
oracle.ops; the topologies restate the reference's model scripts
(tests/mnist_dlsys.py:165-191, tests/LeNet5/LeNet5_mnist_test.py:72-106,
pycode/tinyflow/VGG16_test_leo.py:196-254,
pycode/tinyflow/ResNet50_test_leo.py:29-108, 205-261).

Parameters are passed in by name ("conv1_W", "s2b0_c1_W", "fc_b", ...) so the
caller decides the initial values; nothing here draws random numbers.
"""
import numpy as np

from . import ops as O


class Conv(object):
    def __init__(self, name, padding, stride, bias=False):
        self.name, self.padding, self.stride, self.bias = name, padding, stride, bias

    def forward(self, x, params):
        w = params[self.name + "_W"]
        self.x, self.w = x, w
        self.ph, self.pw = O.conv_pad(w.shape[2], self.padding), O.conv_pad(w.shape[3], self.padding)
        y = O.conv2d_forward(x, w, self.ph, self.pw, self.stride, self.stride)
        if self.bias:
            y = O.add(y, O.broadcast_to_channel(params[self.name + "_b"], y.shape))
        return y

    def backward(self, dy, grads, need_dx=True):
        grads[self.name + "_W"] = O.conv2d_backward_filter(self.x, dy, self.w.shape, self.ph, self.pw,
                                                           self.stride, self.stride)
        if self.bias:
            grads[self.name + "_b"] = O.bias_gradient(dy, "NCHW")
        if not need_dx:
            return None
        return O.conv2d_backward_data(dy, self.w, self.x.shape, self.ph, self.pw, self.stride, self.stride)


class Dense(object):
    def __init__(self, name):
        self.name = name

    def forward(self, x, params):
        self.x, self.w = x, params[self.name + "_W"]
        z = O.matmul(x, False, self.w, False)
        return O.add(z, O.broadcast_to_trailing(params[self.name + "_b"], z.shape))

    def backward(self, dy, grads, need_dx=True):
        dx, dw = O.matmul_gradients(self.x, False, self.w, False, dy)
        grads[self.name + "_W"] = dw
        grads[self.name + "_b"] = O.bias_gradient(dy, "NHWC")
        return dx


class Relu(object):
    def forward(self, x, params):
        self.x = x
        return O.relu(x)

    def backward(self, dy, grads, need_dx=True):
        return O.relu_gradient(self.x, dy)


class BatchNorm(object):
    def __init__(self, mode):
        self.mode = mode

    def forward(self, x, params):
        self.x = x
        y, self.mean, self.istd = O.batch_norm_forward(x, self.mode)
        return y

    def backward(self, dy, grads, need_dx=True):
        return O.batch_norm_backward(self.x, dy, self.mode, self.mean, self.istd)


class MaxPool(object):
    def __init__(self, window, stride, pad):
        self.f, self.s, self.p = window, stride, pad

    def forward(self, x, params):
        self.x = x
        return O.max_pool_forward(x, self.f, self.f, self.p, self.p, self.s, self.s)

    def backward(self, dy, grads, need_dx=True):
        return O.max_pool_backward(self.x, dy, self.f, self.f, self.p, self.p, self.s, self.s)


class AvgPool(object):
    def __init__(self, window, stride, pad):
        self.f, self.s, self.p = window, stride, pad

    def forward(self, x, params):
        self.shape = x.shape
        return O.avg_pool_forward(x, self.f, self.f, self.p, self.p, self.s, self.s)

    def backward(self, dy, grads, need_dx=True):
        return O.avg_pool_backward(self.shape, dy, self.f, self.f, self.p, self.p, self.s, self.s)


class Flatten(object):
    def forward(self, x, params):
        self.shape = x.shape
        return x.reshape(x.shape[0], -1)

    def backward(self, dy, grads, need_dx=True):
        return dy.reshape(self.shape)


class Dropout(object):
    """Inverted dropout at rate ``rate`` (reference autodiff.py:1337-1445).  The caller
    sets ``seed`` before every forward pass: the reference draws a fresh one per
    evaluation, so a comparison has to hand over the seed the product drew."""

    def __init__(self, rate):
        self.rate, self.seed = rate, 0

    def forward(self, x, params):
        y, self.keep = O.dropout_forward(x, self.rate, self.seed)
        return y

    def backward(self, dy, grads, need_dx=True):
        return O.dropout_backward(dy, self.keep, self.rate)


class Sequential(object):
    def __init__(self, layers):
        self.layers = layers

    def forward(self, x, params):
        for layer in self.layers:
            x = layer.forward(x, params)
        return x

    def backward(self, dy, grads, need_dx=True):
        for i in range(len(self.layers) - 1, -1, -1):
            dy = self.layers[i].backward(dy, grads, need_dx or i > 0)
        return dy


class Bottleneck(object):
    """conv1x1(stride)-BN-ReLU, conv3x3-BN-ReLU, conv1x1-BN, plus identity or a
    conv1x1(stride)-BN projection, add, ReLU
    (reference ResNet50_test_leo.py:29-108)."""

    def __init__(self, name, stride, project, bn_mode):
        self.branch = Sequential([
            Conv(name + "_c1", "VALID", stride), BatchNorm(bn_mode), Relu(),
            Conv(name + "_c2", "SAME", 1), BatchNorm(bn_mode), Relu(),
            Conv(name + "_c3", "VALID", 1), BatchNorm(bn_mode)])
        self.shortcut = Sequential([Conv(name + "_sc", "VALID", stride), BatchNorm(bn_mode)]) if project else None
        self.relu = Relu()

    def forward(self, x, params):
        main = self.branch.forward(x, params)
        side = self.shortcut.forward(x, params) if self.shortcut else x
        return self.relu.forward(O.add(main, side), params)

    def backward(self, dy, grads, need_dx=True):
        d = self.relu.backward(dy, grads)
        d_main = self.branch.backward(d, grads)
        d_side = self.shortcut.backward(d, grads) if self.shortcut else d
        return O.add(d_main, d_side)


def mlp_layers():
    return Sequential([Dense("fc1"), Relu(), Dense("fc2"), Relu(), Dense("fc3")])


def lenet5_layers():
    return Sequential([Conv("conv1", "SAME", 1, bias=True), Relu(), MaxPool(2, 2, 0),
                       Conv("conv2", "VALID", 1, bias=True), Relu(), MaxPool(2, 2, 0), Flatten(),
                       Dense("fc3"), Relu(), Dense("fc4"), Relu(), Dense("fc5")])


def vgg16_layers(dropout=None):
    """``dropout``: rate of the two dropout layers behind fc6 and fc7 of the reference's
    model script (pycode/tinyflow/VGG16_test_leo.py:240-247), None for the plain network."""
    layers = []
    for stage, count in enumerate([2, 2, 3, 3, 3], start=1):
        for i in range(1, count + 1):
            layers += [Conv("conv%d_%d" % (stage, i), "SAME", 1), Relu()]
        layers.append(MaxPool(2, 2, 0))
    drop = [] if dropout is None else [Dropout(dropout)]
    layers += [Flatten(), Dense("fc6"), Relu()] + drop + [Dense("fc7"), Relu()]
    layers += ([] if dropout is None else [Dropout(dropout)]) + [Dense("fc8")]
    return Sequential(layers)


def resnet_layers(blocks, bn_mode, final_pool):
    layers = [Conv("stem", "SAME", 2), BatchNorm(bn_mode), Relu(), MaxPool(3, 2, 1)]
    for stage, count in enumerate(blocks):
        for i in range(count):
            stride = 2 if (i == 0 and stage > 0) else 1
            layers.append(Bottleneck("s%db%d" % (stage + 2, i), stride, i == 0, bn_mode))
    layers += [AvgPool(final_pool, 1, 0), Flatten(), Dense("fc")]
    return Sequential(layers)


def network(config, bn_mode="pre_activation", image=224):
    if config == "mlp":
        return mlp_layers()
    if config == "lenet5":
        return lenet5_layers()
    if config == "vgg16":
        return vgg16_layers()
    if config == "resnet50":
        return resnet_layers([3, 4, 6, 3], bn_mode, image // 32)
    if config == "resnet152":
        return resnet_layers([3, 8, 36, 3], bn_mode, image // 32)
    raise ValueError(config)


def loss_and_gradients(net, params, X, y_onehot, head="softmax_xent"):
    """Forward + backward of ``net`` under one of the two loss heads.

    ``"softmax_xent"``: mean softmax cross-entropy; the logit gradient is softmax - y
    WITHOUT the 1/N factor, times the upstream gradient 1 (reference autodiff.py:701-713).
    ``"cross"``: the head of the reference's ``*_leo`` model scripts
    (pycode/tinyflow/VGG16_test_leo.py:250-254) on top of the logits: per-feature batch
    norm over the batch, softmax per instance, loss = sum(-y_ * log(p)) / p.size
    (reference autodiff.py:2079-2103, 2153-2156), differentiated link by link: cross
    backward (gpu_op.cu:4568-4573), softmax backward (gpu_op.cu:3521-3531), batch-norm
    backward, then the network.  Returns (loss, grads, logits)."""
    logits = net.forward(X, params)
    grads = {}
    if head == "softmax_xent":
        loss = O.softmax_cross_entropy(logits, y_onehot)
        dlogits = O.softmax_cross_entropy_gradient(logits, y_onehot, 1.0)
    else:
        assert head == "cross", head
        z, mean, istd = O.batch_norm_forward(logits, "pre_activation")
        p = O.activation_forward(z, "softmax")
        scale = 1.0 / p.size
        loss = np.sum(O.cross(p, y_onehot, scale)).reshape(1)
        dp = O.cross_backward(p, y_onehot, np.ones_like(p), scale)
        dz = O.activation_backward(z, p, dp, "softmax")
        dlogits = O.batch_norm_backward(logits, dz, "pre_activation", mean, istd)
    net.backward(dlogits, grads, need_dx=False)
    return loss, grads, logits


def train_step(net, params, X, y_onehot, lr):
    """One forward + backward + SGD step.

    Returns (loss, grads, new_params, logits).  The loss is the batch mean; the
    logit gradient is softmax - y WITHOUT the 1/N factor, times the upstream
    gradient 1 (reference autodiff.py:701-713); new = old - lr * grad
    (reference gpu_op.cu:4600-4605)."""
    loss, grads, logits = loss_and_gradients(net, params, X, y_onehot)
    new_params = {k: O.sgd_update(v, grads[k], lr) for k, v in params.items()}
    return loss, grads, new_params, logits


def train_step_adam(net, params, moments, X, y_onehot, lr, step, b1=0.9, b2=0.999, e=1e-8, head="softmax_xent"):
    """One forward + backward + Adam step; ``step`` counts from 1.

    ``moments`` maps a parameter name to (m, v).  Returns (loss, grads, new_params,
    new_moments).  m, v update: reference gpu_op.cu:4495-4506; parameter update with
    the bias corrections 1 - b1**step, 1 - b2**step: reference gpu_op.cu:4461-4467 and
    TrainExecuteAdam.py:16-21, 196-198 (the powers start at b1, b2 and are multiplied
    once after every step).  ``head``: see ``loss_and_gradients``."""
    loss, grads, _ = loss_and_gradients(net, params, X, y_onehot, head)
    new_params, new_moments = {}, {}
    for k, w in params.items():
        m, v = O.adam_mv(moments[k][0], moments[k][1], grads[k], b1, b2)
        new_moments[k] = (m, v)
        new_params[k] = O.adam_update(w, m, v, b1 ** step, b2 ** step, e, lr)
    return loss, grads, new_params, new_moments


def train_step_cross_head(net, params, X, y_onehot, lr):
    """One forward + backward + SGD step with the loss head of the reference's
    ``*_leo`` model scripts (pycode/tinyflow/VGG16_test_leo.py:250-254) on top of
    ``net``'s logits (see ``loss_and_gradients``).  Returns (loss, grads, new_params)."""
    loss, grads, _ = loss_and_gradients(net, params, X, y_onehot, "cross")
    new_params = {k: O.sgd_update(v, grads[k], lr) for k, v in params.items()}
    return loss, grads, new_params
