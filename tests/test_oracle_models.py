"""Pins oracle/models.py -- the layer-by-layer networks the GPU step tests are compared
with -- against things that share none of its code:

* central finite differences of the loss: ``train_step`` returns hand-written backward
  passes, so for every parameter tensor the directional derivative of the float64 loss
  along a random direction must equal <gradient, direction> (a dropped term, a wrong
  sign, a transposed operand or a missed residual branch fails this).  The reference's
  softmax-cross-entropy gradient is softmax - y without the 1/N of the mean loss
  (reference autodiff.py:701-713), so the returned gradients are N x d(loss)/d(theta);
  the ``cross`` head (reference autodiff.py:2079-2103) divides by p.size in both
  directions, so there the factor is 1;
* torch autograd on the CPU (float64) for a small bottleneck ResNet, in both batch-norm
  modes: same parameters, same data, gradients compared tensor by tensor.

All CPU, float64, tiny shapes.
"""
import numpy as np
import pytest

from oracle import models as OM
from oracle import ops as O


def _params_for(net_name, rng, **kw):
    """(net, params, X, y) with He-normal weights drawn here (nothing of the product)."""
    def he(shape):
        fan_in = int(np.prod(shape[1:])) if len(shape) == 4 else shape[0]
        return rng.normal(0.0, np.sqrt(2.0 / fan_in), shape)

    def one_hot(n, classes):
        y = np.zeros((n, classes))
        y[np.arange(n), rng.randint(0, classes, n)] = 1.0
        return y

    if net_name == "mlp":
        n, dims = 6, [12, 9, 7, 5]
        params = {}
        for i, (a, b) in enumerate(zip(dims[:-1], dims[1:]), start=1):
            params["fc%d_W" % i] = he((a, b))
            params["fc%d_b" % i] = rng.normal(0, 0.1, (b,))
        return OM.mlp_layers(), params, rng.uniform(0, 1, (n, dims[0])), one_hot(n, dims[-1])
    if net_name == "lenet5":
        n = 3
        params = {"conv1_W": he((6, 1, 5, 5)), "conv1_b": rng.normal(0, 0.1, (6,)),
                  "conv2_W": he((16, 6, 5, 5)), "conv2_b": rng.normal(0, 0.1, (16,)),
                  "fc3_W": he((400, 120)), "fc3_b": rng.normal(0, 0.1, (120,)),
                  "fc4_W": he((120, 84)), "fc4_b": rng.normal(0, 0.1, (84,)),
                  "fc5_W": he((84, 10)), "fc5_b": rng.normal(0, 0.1, (10,))}
        return OM.lenet5_layers(), params, rng.uniform(0, 1, (n, 1, 28, 28)), one_hot(n, 10)
    assert net_name == "resnet"
    blocks, mode, width, n, image, classes = kw["blocks"], kw["mode"], 4, 6, 32, 5
    params = {"stem_W": he((width, 3, 7, 7))}
    in_ch = width
    for stage, count in enumerate(blocks):
        f = width * 2 ** stage
        for i in range(count):
            name = "s%db%d" % (stage + 2, i)
            params[name + "_c1_W"] = he((f, in_ch, 1, 1))
            params[name + "_c2_W"] = he((f, f, 3, 3))
            params[name + "_c3_W"] = he((4 * f, f, 1, 1))
            if i == 0:
                params[name + "_sc_W"] = he((4 * f, in_ch, 1, 1))
            in_ch = 4 * f
    params["fc_W"] = he((in_ch, classes))
    params["fc_b"] = rng.normal(0, 0.1, (classes,))
    final = image // (4 * 2 ** (len(blocks) - 1))
    return OM.resnet_layers(blocks, mode, final), params, rng.normal(0, 1, (n, 3, image, image)), one_hot(n, classes)


def _directional_check(step, net, params, X, y, factor, rng, h=1e-6, rtol=2e-5):
    """<grad, d> / factor against (loss(theta + h d) - loss(theta - h d)) / 2h for one
    random direction d per parameter tensor."""
    grads = step(net, params, X, y, 0.0)[1]
    assert set(grads) == set(params)
    worst = 0.0
    for name in sorted(params):
        d = rng.normal(0, 1, params[name].shape)
        d /= np.linalg.norm(d)
        plus, minus = dict(params), dict(params)
        plus[name] = params[name] + h * d
        minus[name] = params[name] - h * d
        lp = float(np.ravel(step(net, plus, X, y, 0.0)[0])[0])
        lm = float(np.ravel(step(net, minus, X, y, 0.0)[0])[0])
        numeric = (lp - lm) / (2 * h)
        analytic = float(np.sum(grads[name] * d)) / factor
        # scale: the gradient's norm, so that a direction nearly orthogonal to it is not held to its tiny
        # projection; the difference quotient itself is only known to a few roundings of the loss over 2h
        # (which is all there is for a gradient that is zero by construction: a bias in front of a batch norm)
        scale = max(abs(analytic), float(np.linalg.norm(grads[name])) / factor * 1e-2)
        noise = 8 * np.finfo(np.float64).eps * max(abs(lp), abs(lm)) / (2 * h)
        err = max(0.0, abs(numeric - analytic) - noise) / max(scale, 1e-300)
        worst = max(worst, err)
        assert err <= rtol, "%s: finite difference %.10g, hand-written backward %.10g (relative %.3g)" % (
            name, numeric, analytic, err)
    return worst


@pytest.mark.parametrize("case", ["mlp", "lenet5", "resnet:pre_activation", "resnet:spatial"])
def test_train_step_gradients_are_the_derivative_of_its_loss(case):
    rng = np.random.RandomState(11)
    if case.startswith("resnet"):
        net, params, X, y = _params_for("resnet", rng, blocks=[2, 1, 1, 1], mode=case.split(":")[1])
    else:
        net, params, X, y = _params_for(case, rng)
    # gradient = N x d(mean loss)/d(theta): the reference omits the 1/N in the backward
    _directional_check(OM.train_step, net, params, X, y, float(X.shape[0]), rng)


@pytest.mark.parametrize("case", ["mlp", "resnet:pre_activation"])
def test_cross_head_gradients_are_the_derivative_of_its_loss(case):
    rng = np.random.RandomState(12)
    if case.startswith("resnet"):
        net, params, X, y = _params_for("resnet", rng, blocks=[1, 1], mode="pre_activation")
    else:
        net, params, X, y = _params_for(case, rng)
    _directional_check(OM.train_step_cross_head, net, params, X, y, 1.0, rng)


def test_dropout_layer_and_cross_head_under_finite_differences():
    """A dense stack with the dropout layer of the reference's VGG-16 script under the
    batch-norm / softmax / cross head: with the seed held fixed the mask is a constant
    and the step must still be the derivative of its loss."""
    rng = np.random.RandomState(15)
    _, params, X, y = _params_for("mlp", rng)
    net = OM.Sequential([OM.Dense("fc1"), OM.Relu(), OM.Dropout(0.5), OM.Dense("fc2"), OM.Relu(), OM.Dropout(0.25),
                         OM.Dense("fc3")])
    for layer, seed in zip([l for l in net.layers if isinstance(l, OM.Dropout)], (3, 77)):
        layer.seed = seed
    _directional_check(OM.train_step_cross_head, net, params, X, y, 1.0, rng)
    kept = net.layers[2].keep
    assert 0 < kept.sum() < kept.size          # the mask really drops and keeps something

    def adam(net, params, X, y, lr):
        moments = {k: (np.zeros_like(v), np.zeros_like(v)) for k, v in params.items()}
        return OM.train_step_adam(net, params, moments, X, y, lr, 1, head="cross")
    _directional_check(adam, net, params, X, y, 1.0, rng)


def test_sgd_and_adam_steps_apply_their_update_rules_to_those_gradients():
    """new = old - lr * grad for SGD; Adam's first step moves every weight by
    lr * sign(grad) up to e (m / (1 - b1) = g, v / (1 - b2) = g^2)."""
    rng = np.random.RandomState(13)
    net, params, X, y = _params_for("mlp", rng)
    lr = 0.03
    _, grads, new, _ = OM.train_step(net, params, X, y, lr)
    for k in params:
        np.testing.assert_allclose(new[k], params[k] - lr * grads[k], rtol=1e-14, atol=0)
    moments = {k: (np.zeros_like(v), np.zeros_like(v)) for k, v in params.items()}
    _, grads_a, new_a, mom = OM.train_step_adam(net, params, moments, X, y, lr, 1)
    for k in params:
        np.testing.assert_array_equal(grads_a[k], grads[k])
        g = grads[k]
        np.testing.assert_allclose(mom[k][0], 0.1 * g, rtol=1e-12, atol=1e-18)
        np.testing.assert_allclose(mom[k][1], 0.001 * g * g, rtol=1e-9, atol=1e-24)
        big = np.abs(g) > 1e-4
        np.testing.assert_allclose((params[k] - new_a[k])[big], lr * np.sign(g)[big], rtol=1e-3)


@pytest.mark.parametrize("mode", ["pre_activation", "spatial"])
def test_resnet_oracle_matches_torch_autograd(mode):
    torch = pytest.importorskip("torch")
    F = torch.nn.functional
    rng = np.random.RandomState(14)
    blocks = [2, 1, 1]
    net, params, X, y = _params_for("resnet", rng, blocks=blocks, mode=mode)
    loss_ref, grads_ref, _, logits_ref = OM.train_step(net, params, X, y, 0.0)
    tp = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in params.items()}

    def bn(x):
        dims = (0,) if mode == "pre_activation" else (0, 2, 3)
        mean = x.mean(dim=dims, keepdim=True)
        var = ((x - mean) ** 2).mean(dim=dims, keepdim=True)   # biased, gamma = 1, beta = 0, eps = 1e-5
        return (x - mean) / torch.sqrt(var + 1e-5)

    x = torch.tensor(X, dtype=torch.float64)
    h = F.relu(bn(F.conv2d(x, tp["stem_W"], stride=2, padding=3)))
    h = F.max_pool2d(h, 3, 2, 1)
    for stage, count in enumerate(blocks):
        for i in range(count):
            name = "s%db%d" % (stage + 2, i)
            stride = 2 if (i == 0 and stage > 0) else 1
            m = F.relu(bn(F.conv2d(h, tp[name + "_c1_W"], stride=stride)))
            m = F.relu(bn(F.conv2d(m, tp[name + "_c2_W"], padding=1)))
            m = bn(F.conv2d(m, tp[name + "_c3_W"]))
            side = bn(F.conv2d(h, tp[name + "_sc_W"], stride=stride)) if i == 0 else h
            h = F.relu(m + side)
    h = F.avg_pool2d(h, h.shape[-1]).flatten(1)
    logits = h @ tp["fc_W"] + tp["fc_b"]
    yt = torch.tensor(y, dtype=torch.float64)
    loss = -(yt * F.log_softmax(logits, dim=1)).sum(dim=1).mean()
    loss.backward()
    np.testing.assert_allclose(logits.detach().numpy(), logits_ref, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(loss.item(), float(np.ravel(loss_ref)[0]), rtol=1e-12)
    n = X.shape[0]
    for k in params:
        np.testing.assert_allclose(n * tp[k].grad.numpy(), grads_ref[k], rtol=1e-7,
                                   atol=1e-9 * max(1.0, float(np.abs(grads_ref[k]).max())), err_msg=k)
