"""Pins of the oracle's training GRAPHS (oracle/nets.py), which compose the oracle operators
the way the reference applications do (apps/mnist_common.h:123-288,
owl/apps/imagenet_alexnet/alexnet.py:64-133).  The gradients they return must be the
derivative of the loss the graphs imply: with sens = prob - label at the output, that loss is
the cross entropy summed over the batch, L = -sum_n log prob[label_n, n].  Central finite
differences of L (evaluated in float64 from the oracle's fp32 probabilities) along random
directions and at single entries pin every layer's backward composition: a dropped term, a
transposed operand, a wrong pooling route or a missing ReLU gate changes the result by far
more than the tolerance.  CPU only."""
import numpy as np
import pytest

from oracle import nets


def _loss(prob, label, classes, batch):
    p = prob.reshape(batch, classes).astype(np.float64)
    lab = label.reshape(batch, classes).argmax(axis=1)
    return float(-np.log(p[np.arange(batch), lab]).sum())


def _directional_check(step, params, data, label, classes, batch, eps, tol, seed):
    """step(params) -> (grads dict, prob).  Compares <g, d> with the central difference of the
    loss along a random direction d of unit max-norm, one parameter tensor at a time, and at
    a few single entries of each tensor."""
    g, prob = step(params)
    rng = np.random.default_rng(seed)
    L = lambda p: _loss(step(p)[1], label, classes, batch)
    for name in sorted(params):
        w = params[name]
        d = rng.choice([-1.0, 1.0], size=w.size).astype(np.float32)
        plus, minus = dict(params), dict(params)
        plus[name] = w + np.float32(eps) * d
        minus[name] = w - np.float32(eps) * d
        # the step actually taken in fp32
        h = (plus[name].astype(np.float64) - minus[name].astype(np.float64))
        fd = L(plus) - L(minus)
        an = float(np.dot(g[name].astype(np.float64), h))
        scale = float(np.sum(np.abs(g[name].astype(np.float64) * h))) + 1e-12
        assert abs(fd - an) <= tol * scale, "%s: directional fd %.6e vs analytic %.6e (scale %.3e)" % (
            name, fd, an, scale)
        gmax = float(np.max(np.abs(g[name])))
        for idx in rng.choice(w.size, size=min(3, w.size), replace=False):
            plus, minus = dict(params), dict(params)
            plus[name] = w.copy()
            minus[name] = w.copy()
            plus[name][idx] += np.float32(eps)
            minus[name][idx] -= np.float32(eps)
            h1 = float(plus[name][idx]) - float(minus[name][idx])
            fd1 = (L(plus) - L(minus)) / h1
            assert abs(fd1 - float(g[name][idx])) <= 5 * tol * gmax + 1e-6, \
                "%s[%d]: fd %.6e vs analytic %.6e" % (name, idx, fd1, g[name][idx])


def test_mlp_graph_gradient_is_the_loss_derivative():
    din, hid, dout, batch = 12, 7, 5, 6
    rng = np.random.default_rng(3)
    params = {"w0": rng.standard_normal(hid * din).astype(np.float32) * np.float32(0.5),
              "b0": rng.standard_normal(hid).astype(np.float32) * np.float32(0.1),
              "w1": rng.standard_normal(dout * hid).astype(np.float32) * np.float32(0.5),
              "b1": rng.standard_normal(dout).astype(np.float32) * np.float32(0.1)}
    data = rng.random(din * batch, dtype=np.float32)
    label = np.zeros((batch, dout), np.float32)
    label[np.arange(batch), rng.integers(0, dout, batch)] = 1

    def step(p):
        _, res = nets.mlp_step(dict(p), data, label.ravel(), 0.01, batch, din, hid, dout)
        return {k: res["g_" + k] for k in p}, res["prob"]

    _directional_check(step, params, data, label, dout, batch, eps=2e-3, tol=2e-3, seed=4)


@pytest.mark.parametrize("variant", [0, 1])
def test_cnn_graph_gradient_is_the_loss_derivative(variant):
    batch = 2
    params, data, label = nets.make_inputs("cnn", batch, seed=5)
    rng = np.random.default_rng(6)
    # weights large enough that every layer's gradient is well above fp32 noise
    params = {k: (rng.standard_normal(v.size).astype(np.float32) *
                  np.float32(0.2 if k.startswith("w") else 0.05)) for k, v in params.items()}
    params["w2"] *= np.float32(0.1)
    kw = dict(pad2=2, pool2=3) if variant else {}

    def step(p):
        _, res = nets.cnn_step(dict(p), data, label, 0.01, batch, **kw)
        return {k: res["g_" + k] for k in p}, res["prob"]

    _directional_check(step, params, data, label.reshape(batch, 10), 10, batch, eps=1e-3,
                       tol=1e-2, seed=7)


def test_sgd_update_is_w_minus_lr_over_batch_times_gradient():
    batch = 4
    params, data, label = nets.make_inputs("mlp", batch, seed=8)
    newp, res = nets.mlp_step(dict(params), data, label, 0.05, batch)
    for k in params:
        want = params[k] - (np.float32(0.05) / np.float32(batch)) * res["g_" + k]
        np.testing.assert_array_equal(newp[k], want)


def test_alexnet_forward_is_the_forward_half_of_the_step():
    """alexnet_forward (used alone by the batch-256 prefix test) and alexnet_step share one
    forward pass; a tiny class count keeps this cheap."""
    batch, classes = 1, 10
    params, data, label = nets.make_inputs("alexnet", batch, classes=classes)
    acts, out = nets.alexnet_forward(params, data, batch, classes)
    _, res = nets.alexnet_step(dict(params), data, label, 0.01, batch, classes, keep=True)
    np.testing.assert_array_equal(out, res["prob"])
    assert all(np.array_equal(a, b) for a, b in zip(acts, res["acts"]))
    assert abs(float(out.sum()) - 1.0) < 1e-5


def test_caffe_style_graph_gradient_is_the_loss_derivative():
    """The owl.net-style unit chain (convolution, ReLU gated by its input, LRN, max pooling,
    inner product, dropout with its 1/(1-ratio) scale, softmax loss): central differences of
    the loss pin caffe_backward, including the LRN gradient and the dropout scale."""
    units = [("conv", "c1", 2, 4, 8, 8, 1, 1, 3), ("relu",), ("lrn", 4, 8, 8, 3, 0.5, 0.75),
             ("pool", 4, 8, 8, 3, 2, 0), ("fc", "f1", 64, 6), ("relu",), ("dropout", 6, 0.5),
             ("fc", "f2", 6, 3)]
    batch, classes = 3, 3
    rng = np.random.default_rng(11)
    shapes = nets.caffe_param_shapes(units)
    flat = {}
    for name, (ws, bs) in shapes.items():
        flat[name + ".w"] = (rng.standard_normal(int(np.prod(ws))) * 0.4).astype(np.float32)
        flat[name + ".b"] = (rng.standard_normal(int(np.prod(bs))) * 0.1).astype(np.float32)
    data = rng.standard_normal(batch * 2 * 8 * 8).astype(np.float32)
    labels = rng.integers(0, classes, batch)
    onehot = np.zeros((batch, classes), np.float32)
    onehot[np.arange(batch), labels] = 1
    masks = [(rng.random(6 * batch) < 0.5).astype(np.float32)]

    def step(p):
        params = {n: (p[n + ".w"], p[n + ".b"]) for n in shapes}
        acts, prob = nets.caffe_forward(units, params, data, batch, masks)
        g = nets.caffe_backward(units, params, data, acts, prob, labels, batch, masks)
        grads = {}
        for n in shapes:
            grads[n + ".w"], grads[n + ".b"] = g[n]
        return grads, prob

    _directional_check(step, flat, data, onehot, classes, batch, eps=1e-3, tol=1e-2, seed=12)


def test_caffe_update_rule():
    rng = np.random.default_rng(13)
    w, d, g = (rng.standard_normal(50).astype(np.float32) for _ in range(3))
    new_w, new_d = nets.caffe_update(w, d, g, 0.01, 2.0, 0.0005, 1.0, 0.9, 4)
    want_d = 0.9 * d.astype(np.float64) - 0.01 * 2 / 4 * g - 0.01 * 2 * 0.0005 * w
    assert np.max(np.abs(new_d - want_d)) < 1e-6 and np.max(np.abs(new_w - (w + want_d))) < 1e-6
