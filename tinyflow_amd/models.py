"""Model graphs of the benchmark configurations, built from the autodiff ops.

Each builder returns a ``Model``: the loss node, the data/label placeholders and
an ordered ``{Variable node: initial numpy value}`` dict.  Topologies follow the
reference's own model scripts:

  mlp        tests/mnist_dlsys.py:165-191 (784-256-100-10, relu_op, softmax xent)
  lenet5     tests/LeNet5/LeNet5_mnist_test.py:72-106 (conv2withbias + max pool + dense),
             with the classic 6/16/120/84 channel counts
  vgg16      pycode/tinyflow/VGG16_test_leo.py:196-254 (13 bias-free 3x3 "SAME" convs,
             five 2x2 max pools, three dense layers; dropout and the final fully-BN
             are left out: dropout is non-deterministic in the reference)
  resnet     pycode/tinyflow/ResNet50_test_leo.py:29-108, 205-261 (bottleneck blocks with
             the stride on the first 1x1 and on the 1x1 shortcut, batch norm after every
             convolution, ReLU after BN1/BN2 and after the residual add), block counts
             [3,4,6,3] (ResNet-50) or [3,8,36,3] (ResNet-152, tests/ResNet152_test.py:92-149).
             The stem is a padded 7x7 stride-2 "SAME" convolution and the stem pool is
             3x3 stride 2 pad 1, i.e. the standard 56x56 stage-2 maps.
All of them end in ``softmaxcrossentropy_op`` and are trained with plain SGD.
"""
from collections import OrderedDict

import numpy as np

from . import autodiff as ad


class Model(object):
    def __init__(self, name, loss, logits, X, y_, variables, input_shape, n_class):
        self.name = name
        self.loss = loss
        self.logits = logits
        self.X = X
        self.y_ = y_
        self.variables = variables  # OrderedDict: Variable node -> initial value (numpy, fp32)
        self.input_shape = input_shape
        self.n_class = n_class

    def variable_by_name(self):
        return {v.name: v for v in self.variables}


def he_normal(rng, shape):
    """N(0, sqrt(2 / fan_in)); fan_in = C*R*S for filters, rows for matrices."""
    fan_in = int(np.prod(shape[1:])) if len(shape) == 4 else shape[0]
    return rng.normal(0.0, np.sqrt(2.0 / fan_in), shape).astype(np.float32)


class _Builder(object):
    def __init__(self, rng, init=he_normal):
        self.rng = rng
        self.init = init
        self.variables = OrderedDict()

    def var(self, name, shape, zero=False):
        node = ad.Variable(name)
        self.variables[node] = np.zeros(shape, np.float32) if zero else self.init(self.rng, shape)
        return node

    def conv(self, x, name, in_ch, out_ch, k, padding, stride, bias=False):
        w = self.var(name + "_W", (out_ch, in_ch, k, k))
        if bias:
            b = self.var(name + "_b", (out_ch,), zero=True)
            return ad.conv2withbias(x, w, b, "NCHW", padding, stride, stride)
        return ad.convolution_2d_forward_op(x, w, "NCHW", padding, stride, stride)

    def dense(self, x, name, in_f, out_f):
        w = self.var(name + "_W", (in_f, out_f))
        b = self.var(name + "_b", (out_f,), zero=True)
        return ad.dense(x, w, b)


def synthetic_batch(rng, input_shape, n_class, distribution):
    """X ("uniform": U[0,1), "normal": N(0,1)) and uniformly random one-hot labels."""
    if distribution == "uniform":
        X = rng.uniform(0.0, 1.0, input_shape)
    else:
        X = rng.normal(0.0, 1.0, input_shape)
    labels = rng.randint(0, n_class, input_shape[0])
    y = np.zeros((input_shape[0], n_class), np.float32)
    y[np.arange(input_shape[0]), labels] = 1.0
    return X.astype(np.float32), y


def _loss_head(h, y_, head):
    """``"softmax_xent"``: the fused softmax cross-entropy node (the benchmark
    configurations).  ``"cross"``: the head of the reference's ``*_leo`` model scripts
    (pycode/tinyflow/VGG16_test_leo.py:250-254): batch norm of the logits, softmax
    activation, then ``crossEntropy_loss`` = sum(-y_ * log(p)) / p.size."""
    if head == "softmax_xent":
        return ad.softmaxcrossentropy_op(h, y_)
    assert head == "cross", head
    p = ad.fullyactivation_forward_op(ad.fullybn_forward_op(h, "NCHW"), "NCHW", "softmax")
    return ad.crossEntropy_loss(p, y_)


def mlp(rng, batch=128, head="softmax_xent"):
    b = _Builder(rng, init=lambda r, shape: r.normal(0.0, 0.01, shape).astype(np.float32))
    X, y_ = ad.Placeholder("X"), ad.Placeholder("y_")
    h = X
    sizes = [784, 256, 100, 10]
    for i in range(3):
        h = b.dense(h, "fc%d" % (i + 1), sizes[i], sizes[i + 1])
        if i < 2:
            h = ad.relu_op(h)
    loss = _loss_head(h, y_, head)
    return Model("mlp", loss, h, X, y_, b.variables, (batch, 784), 10)


def lenet5(rng, batch=64, head="softmax_xent"):
    b = _Builder(rng)
    X, y_ = ad.Placeholder("X"), ad.Placeholder("y_")
    h = b.conv(X, "conv1", 1, 6, 5, "SAME", 1, bias=True)
    h = ad.activation_forward_op(h, "NCHW", "relu")
    h = ad.pooling_2d_forward_op(h, "NCHW", "max", 0, 0, 2, 2, 2, 2)
    h = b.conv(h, "conv2", 6, 16, 5, "VALID", 1, bias=True)
    h = ad.activation_forward_op(h, "NCHW", "relu")
    h = ad.pooling_2d_forward_op(h, "NCHW", "max", 0, 0, 2, 2, 2, 2)
    h = ad.flatten_op(h)
    h = ad.fullyactivation_forward_op(b.dense(h, "fc3", 400, 120), "NCHW", "relu")
    h = ad.fullyactivation_forward_op(b.dense(h, "fc4", 120, 84), "NCHW", "relu")
    h = b.dense(h, "fc5", 84, 10)
    loss = _loss_head(h, y_, head)
    return Model("lenet5", loss, h, X, y_, b.variables, (batch, 1, 28, 28), 10)


VGG16_CHANNELS = [(64, 64), (128, 128), (256, 256, 256), (512, 512, 512), (512, 512, 512)]


def vgg16(rng, batch=32, image=224, n_class=1000, fc_width=4096, head="softmax_xent", dropout=None):
    """``head="cross"`` with ``dropout=0.5`` is the graph of the reference's model script
    as written (pycode/tinyflow/VGG16_test_leo.py:196-254): dropout behind fc6 and fc7,
    batch norm of the logits, softmax activation, ``crossEntropy_loss``."""
    b = _Builder(rng)
    X, y_ = ad.Placeholder("X"), ad.Placeholder("y_")
    h, in_ch = X, 3
    for stage, widths in enumerate(VGG16_CHANNELS, start=1):
        for i, out_ch in enumerate(widths, start=1):
            h = b.conv(h, "conv%d_%d" % (stage, i), in_ch, out_ch, 3, "SAME", 1)
            h = ad.activation_forward_op(h, "NCHW", "relu")
            in_ch = out_ch
        h = ad.pooling_2d_forward_op(h, "NCHW", "max", 0, 0, 2, 2, 2, 2)
    h = ad.flatten_op(h)
    flat = in_ch * (image // 32) ** 2
    h = ad.fullyactivation_forward_op(b.dense(h, "fc6", flat, fc_width), "NCHW", "relu")
    if dropout is not None:
        h = ad.fullydropout_forward_op(h, "NCHW", dropout)
    h = ad.fullyactivation_forward_op(b.dense(h, "fc7", fc_width, fc_width), "NCHW", "relu")
    if dropout is not None:
        h = ad.fullydropout_forward_op(h, "NCHW", dropout)
    h = b.dense(h, "fc8", fc_width, n_class)
    loss = _loss_head(h, y_, head)
    return Model("vgg16", loss, h, X, y_, b.variables, (batch, 3, image, image), n_class)


def _bottleneck(b, x, name, in_ch, widths, stride, project, bn_mode):
    f1, f2, f3 = widths

    def conv_bn(h, tag, cin, cout, k, padding, s, relu):
        h = b.conv(h, name + tag, cin, cout, k, padding, s)
        h = ad.bn_forward_op(h, "NCHW", bn_mode)
        return ad.activation_forward_op(h, "NCHW", "relu") if relu else h

    h = conv_bn(x, "_c1", in_ch, f1, 1, "VALID", stride, True)
    h = conv_bn(h, "_c2", f1, f2, 3, "SAME", 1, True)
    h = conv_bn(h, "_c3", f2, f3, 1, "VALID", 1, False)
    shortcut = conv_bn(x, "_sc", in_ch, f3, 1, "VALID", stride, False) if project else x
    return ad.activation_forward_op(ad.add_op(h, shortcut), "NCHW", "relu")


def resnet(rng, blocks, batch, image=224, n_class=1000, bn_mode="pre_activation", width=64, name="resnet"):
    """Bottleneck ResNet; ``width`` scales every channel count (64 = the real network)."""
    b = _Builder(rng)
    X, y_ = ad.Placeholder("X"), ad.Placeholder("y_")
    h = b.conv(X, "stem", 3, width, 7, "SAME", 2)
    h = ad.bn_forward_op(h, "NCHW", bn_mode)
    h = ad.activation_forward_op(h, "NCHW", "relu")
    h = ad.pooling_2d_forward_op(h, "NCHW", "max", 1, 1, 2, 2, 3, 3)
    in_ch = width
    for stage, count in enumerate(blocks):
        f = width * 2 ** stage
        for i in range(count):
            stride = 2 if (i == 0 and stage > 0) else 1
            h = _bottleneck(b, h, "s%db%d" % (stage + 2, i), in_ch, (f, f, 4 * f), stride, i == 0, bn_mode)
            in_ch = 4 * f
    final = image // 32
    h = ad.pooling_2d_forward_op(h, "NCHW", "mean", 0, 0, 1, 1, final, final)
    h = ad.flatten_op(h)
    h = b.dense(h, "fc", in_ch, n_class)
    loss = ad.softmaxcrossentropy_op(h, y_)
    return Model(name, loss, h, X, y_, b.variables, (batch, 3, image, image), n_class)


def resnet50(rng, batch=64, **kw):
    return resnet(rng, [3, 4, 6, 3], batch, name="resnet50", **kw)


def resnet152(rng, batch=128, **kw):
    return resnet(rng, [3, 8, 36, 3], batch, name="resnet152", **kw)


# the benchmark configurations: name -> (builder, seed, input distribution)
CONFIGS = OrderedDict([
    ("mlp", (mlp, 1, "uniform")),
    ("lenet5", (lenet5, 2, "uniform")),
    ("vgg16", (vgg16, 3, "normal")),
    ("resnet50", (resnet50, 4, "normal")),
    ("resnet152", (resnet152, 5, "normal")),
])


def build(config, **kw):
    """(model, X, y) of a named configuration: seeded data first, then the weights
    in network order, all from one ``numpy.random.RandomState(seed)``."""
    builder, seed, dist = CONFIGS[config]
    rng = np.random.RandomState(seed)
    input_shape = _input_shape(config, kw)
    n_class = kw.get("n_class", 10 if config in ("mlp", "lenet5") else 1000)
    X, y = synthetic_batch(rng, input_shape, n_class, dist)
    model = builder(rng, **kw)
    assert model.input_shape == input_shape and model.n_class == n_class
    return model, X, y


def _input_shape(config, kw):
    defaults = {"mlp": 128, "lenet5": 64, "vgg16": 32, "resnet50": 64, "resnet152": 128}
    batch = kw.get("batch", defaults[config])
    if config == "mlp":
        return (batch, 784)
    if config == "lenet5":
        return (batch, 1, 28, 28)
    image = kw.get("image", 224)
    return (batch, 3, image, image)
