"""CPU restatement of the three training graphs, composed from the oracle operators.
TEST INFRASTRUCTURE ONLY (parity tests, smoke check, CPU-baseline timing).

Graphs: apps/mnist_common.h:123-288 (MLP, CNN) and
owl/apps/imagenet_alexnet/alexnet.py:64-133 (AlexNet without dropout), with the plain SGD
update w -= lr/batch * grad of apps/mnist_common.h:185-197.  ReluBackward has no
reference CPU implementation; the oracle's closed form dx = dy*[x>0] stands in for it.
All tensors are flat float32 buffers in Minerva's column-major layout.
"""
import numpy as np

from . import mnv_oracle as ora


def _fc(w, x, b, m, k, n):
    """W{m,k} * X{k,n} + b{m,1}"""
    y = ora.matmult(w, x, m, n, k, fast=True)
    return ora.norm_arithmetic(ora.ADD, y, [m, n], b, [1])


def _sgd(p, g, lr, batch):
    step = ora.arithmetic_const(ora.MUL, 0, np.float32(lr / np.float32(batch)), g)
    return ora.arithmetic(ora.SUB, p, step)


def _relu(x):
    return ora.activation_fwd(ora.RELU, x)


def _relu_bwd(dy, y):
    return ora.activation_bwd(ora.RELU, dy, y, y)


def mlp_step(p, data, label, lr, batch, din=784, hid=256, dout=10):
    """Returns (new params, results) for one step.  p: dict w0,b0,w1,b1."""
    a1 = _relu(_fc(p["w0"], data, p["b0"], hid, din, batch))
    a2 = _fc(p["w1"], a1, p["b1"], dout, hid, batch)
    a3 = ora.softmax_instance_fwd(a2, batch, dout, 1, 1)
    s2 = ora.arithmetic(ora.SUB, a3, label)
    w1t = ora.transpose(p["w1"], hid, dout)
    s1 = _relu_bwd(ora.matmult(w1t, s2, hid, batch, dout, fast=True), a1)
    g = {
        "w0": ora.matmult(s1, ora.transpose(data, batch, din), hid, din, batch, fast=True),
        "b0": ora.reduction(ora.SUM, s1, [hid, batch], [1]),
        "w1": ora.matmult(s2, ora.transpose(a1, batch, hid), dout, hid, batch, fast=True),
        "b1": ora.reduction(ora.SUM, s2, [dout, batch], [1]),
    }
    newp = {k: _sgd(p[k], g[k], lr, batch) for k in p}
    res = {"prob": a3}
    res.update({"g_" + k: v for k, v in g.items()})
    res["l1_b0"] = ora.reduction(ora.SUM, np.abs(s1), [hid, batch], [1])
    res["l1_b1"] = ora.reduction(ora.SUM, np.abs(s2), [dout, batch], [1])
    return newp, res


def cnn_step(p, data, label, lr, batch, pad2=0, pool2=2):
    N = batch
    c1 = (N, 1, 16, 28, 28, 0, 0, 1, 1, 5, 5)
    a1 = ora.conv_fwd(data, p["w0"], p["b0"], *c1)            # 16 x 24 x 24
    a2 = _relu(a1)
    pl1 = (N, 16, 24, 24, 2, 2, 2, 2, 0, 0)
    a3 = ora.pool_fwd(ora.POOL_MAX, a2, *pl1)                  # 16 x 12 x 12
    c2 = (N, 16, 32, 12, 12, pad2, pad2, 1, 1, 5, 5)
    h2 = 12 + 2 * pad2 - 4
    a4 = ora.conv_fwd(a3, p["w1"], p["b1"], *c2)
    a5 = _relu(a4)
    pl2 = (N, 32, h2, h2, pool2, pool2, pool2, pool2, 0, 0)
    a6 = ora.pool_fwd(ora.POOL_MAX, a5, *pl2)                  # 32 x 4 x 4
    assert a6.size == 512 * N
    a7 = _fc(p["w2"], a6, p["b2"], 10, 512, N)
    a8 = ora.softmax_instance_fwd(a7, N, 10, 1, 1)
    s7 = ora.arithmetic(ora.SUB, a8, label)
    s6 = ora.matmult(ora.transpose(p["w2"], 512, 10), s7, 512, N, 10, fast=True)
    s5 = ora.pool_bwd(ora.POOL_MAX, s6, a6, a5, *pl2)
    s4 = ora.activation_bwd(ora.RELU, s5, a5, a4)
    s3 = ora.conv_bwd_data(s4, p["w1"], *c2)
    s2 = ora.pool_bwd(ora.POOL_MAX, s3, a3, a2, *pl1)
    s1 = ora.activation_bwd(ora.RELU, s2, a2, a1)
    g = {
        "w0": ora.conv_bwd_filter(s1, data, *c1),
        "b0": ora.conv_bwd_bias(s1, N, 16, 24, 24),
        "w1": ora.conv_bwd_filter(s4, a3, *c2),
        "b1": ora.conv_bwd_bias(s4, N, 32, h2, h2),
        "w2": ora.matmult(s7, ora.transpose(a6, N, 512), 10, 512, N, fast=True),
        "b2": ora.reduction(ora.SUM, s7, [10, N], [1]),
    }
    newp = {k: _sgd(p[k], g[k], lr, batch) for k in p}
    res = {"prob": a8}
    res.update({"g_" + k: v for k, v in g.items()})
    res["l1_b0"] = ora.conv_bwd_bias(np.abs(s1), N, 16, 24, 24)
    res["l1_b1"] = ora.conv_bwd_bias(np.abs(s4), N, 32, h2, h2)
    res["l1_b2"] = ora.reduction(ora.SUM, np.abs(s7), [10, N], [1])
    return newp, res


ALEX_CONVS = [  # C, K, H, W, ph, pw, sv, sh, R, S
    (3, 96, 227, 227, 0, 0, 4, 4, 11, 11),
    (96, 256, 27, 27, 2, 2, 1, 1, 5, 5),
    (256, 384, 13, 13, 1, 1, 1, 1, 3, 3),
    (384, 384, 13, 13, 1, 1, 1, 1, 3, 3),
    (384, 256, 13, 13, 1, 1, 1, 1, 3, 3),
]


def alexnet_param_shapes(classes=1000):
    shapes = {}
    for i, (C, K, _, _, _, _, _, _, R, S) in enumerate(ALEX_CONVS):
        shapes["w%d" % i] = [S, R, C, K]
        shapes["b%d" % i] = [K]
    shapes.update({"w5": [4096, 9216], "w6": [4096, 4096], "w7": [classes, 4096],
                   "b5": [4096, 1], "b6": [4096, 1], "b7": [classes, 1]})
    return shapes


def seed_sequence(base, count):
    """The seeds the host layer hands to successive Randn / RandBernoulli calls after
    SetRandomSeed(base): splitmix64 of base + k * golden ratio, k = 1, 2, ..."""
    M = (1 << 64) - 1
    out = []
    for k in range(1, count + 1):
        z = (base + 0x9E3779B97F4A7C15 * k) & M
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        out.append(z ^ (z >> 31))
    return out


def alexnet_forward(p, data, batch, classes=1000, masks=None):
    """Forward pass only: (acts[0..11], probabilities).  masks = (mask6, mask7) for dropout."""
    N = batch
    cv = [(N,) + c for c in ALEX_CONVS]
    pool = lambda C, H: (N, C, H, H, 2, 2, 3, 3, 0, 0)
    acts = [None] * 12
    acts[0] = data
    acts[1] = _relu(ora.conv_fwd(acts[0], p["w0"], p["b0"], *cv[0]))     # 96 x 55 x 55
    acts[2] = ora.pool_fwd(ora.POOL_MAX, acts[1], *pool(96, 55))         # 27
    acts[3] = _relu(ora.conv_fwd(acts[2], p["w1"], p["b1"], *cv[1]))     # 256 x 27 x 27
    acts[4] = ora.pool_fwd(ora.POOL_MAX, acts[3], *pool(256, 27))        # 13
    acts[5] = _relu(ora.conv_fwd(acts[4], p["w2"], p["b2"], *cv[2]))
    acts[6] = _relu(ora.conv_fwd(acts[5], p["w3"], p["b3"], *cv[3]))
    acts[7] = _relu(ora.conv_fwd(acts[6], p["w4"], p["b4"], *cv[4]))     # 256 x 13 x 13
    acts[8] = ora.pool_fwd(ora.POOL_MAX, acts[7], *pool(256, 13))        # 6 -> 9216
    acts[9] = _relu(_fc(p["w5"], acts[8], p["b5"], 4096, 9216, N))
    if masks:
        acts[9] = ora.arithmetic(ora.MUL, acts[9], masks[0])
    acts[10] = _relu(_fc(p["w6"], acts[9], p["b6"], 4096, 4096, N))
    if masks:
        acts[10] = ora.arithmetic(ora.MUL, acts[10], masks[1])
    acts[11] = _fc(p["w7"], acts[10], p["b7"], classes, 4096, N)
    out = ora.softmax_instance_fwd(acts[11], N, classes, 1, 1)
    return acts, out


def alexnet_backward(p, acts, out, label, batch, classes=1000, masks=None):
    """Backward pass from given forward results: (gradients, sensitivities, L1 mass behind
    every bias gradient).  `acts` / `out` need not come from alexnet_forward: evaluated at
    another implementation's activations it opens the gates and routes the pooling
    gradients the way that implementation did."""
    N = batch
    cv = [(N,) + c for c in ALEX_CONVS]
    pool = lambda C, H: (N, C, H, H, 2, 2, 3, 3, 0, 0)
    sens = [None] * 12
    sens[11] = ora.arithmetic(ora.SUB, out, label)
    mm = lambda a, b, m, n, k: ora.matmult(a, b, m, n, k, fast=True)
    sens[10] = mm(ora.transpose(p["w7"], 4096, classes), sens[11], 4096, N, classes)
    if masks:
        sens[10] = ora.arithmetic(ora.MUL, sens[10], masks[1])
    sens[10] = _relu_bwd(sens[10], acts[10])
    sens[9] = mm(ora.transpose(p["w6"], 4096, 4096), sens[10], 4096, N, 4096)
    if masks:
        sens[9] = ora.arithmetic(ora.MUL, sens[9], masks[0])
    sens[9] = _relu_bwd(sens[9], acts[9])
    sens[8] = mm(ora.transpose(p["w5"], 9216, 4096), sens[9], 9216, N, 4096)
    sens[7] = _relu_bwd(ora.pool_bwd(ora.POOL_MAX, sens[8], acts[8], acts[7], *pool(256, 13)), acts[7])
    sens[6] = _relu_bwd(ora.conv_bwd_data(sens[7], p["w4"], *cv[4]), acts[6])
    sens[5] = _relu_bwd(ora.conv_bwd_data(sens[6], p["w3"], *cv[3]), acts[5])
    sens[4] = ora.conv_bwd_data(sens[5], p["w2"], *cv[2])
    sens[3] = _relu_bwd(ora.pool_bwd(ora.POOL_MAX, sens[4], acts[4], acts[3], *pool(256, 27)), acts[3])
    sens[2] = ora.conv_bwd_data(sens[3], p["w1"], *cv[1])
    sens[1] = _relu_bwd(ora.pool_bwd(ora.POOL_MAX, sens[2], acts[2], acts[1], *pool(96, 55)), acts[1])
    g = {
        "w7": mm(sens[11], ora.transpose(acts[10], N, 4096), classes, 4096, N),
        "w6": mm(sens[10], ora.transpose(acts[9], N, 4096), 4096, 4096, N),
        "w5": mm(sens[9], ora.transpose(acts[8], N, 9216), 4096, 9216, N),
        "w4": ora.conv_bwd_filter(sens[7], acts[6], *cv[4]),
        "w3": ora.conv_bwd_filter(sens[6], acts[5], *cv[3]),
        "w2": ora.conv_bwd_filter(sens[5], acts[4], *cv[2]),
        "w1": ora.conv_bwd_filter(sens[3], acts[2], *cv[1]),
        "w0": ora.conv_bwd_filter(sens[1], acts[0], *cv[0]),
        "b7": ora.reduction(ora.SUM, sens[11], [classes, N], [1]),
        "b6": ora.reduction(ora.SUM, sens[10], [4096, N], [1]),
        "b5": ora.reduction(ora.SUM, sens[9], [4096, N], [1]),
        "b4": ora.conv_bwd_bias(sens[7], N, 256, 13, 13),
        "b3": ora.conv_bwd_bias(sens[6], N, 384, 13, 13),
        "b2": ora.conv_bwd_bias(sens[5], N, 384, 13, 13),
        "b1": ora.conv_bwd_bias(sens[3], N, 256, 27, 27),
        "b0": ora.conv_bwd_bias(sens[1], N, 96, 55, 55),
    }
    # L1 mass behind every bias gradient: the scale its rounding error is measured against
    l1 = {
        "b7": ora.reduction(ora.SUM, np.abs(sens[11]), [classes, N], [1]),
        "b6": ora.reduction(ora.SUM, np.abs(sens[10]), [4096, N], [1]),
        "b5": ora.reduction(ora.SUM, np.abs(sens[9]), [4096, N], [1]),
        "b4": ora.conv_bwd_bias(np.abs(sens[7]), N, 256, 13, 13),
        "b3": ora.conv_bwd_bias(np.abs(sens[6]), N, 384, 13, 13),
        "b2": ora.conv_bwd_bias(np.abs(sens[5]), N, 384, 13, 13),
        "b1": ora.conv_bwd_bias(np.abs(sens[3]), N, 256, 27, 27),
        "b0": ora.conv_bwd_bias(np.abs(sens[1]), N, 96, 55, 55),
    }
    return g, sens, l1


def dropout_masks(batch, dropout_rate, seed_base):
    """drop6 / drop7 masks: the library's first two RandBernoulli draws after
    SetRandomSeed(seed_base)."""
    s6, s7 = seed_sequence(seed_base, 2)
    return (ora.rand_bernoulli(4096 * batch, s6, dropout_rate),
            ora.rand_bernoulli(4096 * batch, s7, dropout_rate))


def alexnet_step(p, data, label, lr, batch, classes=1000, dropout_rate=0.0, seed_base=None,
                 keep=False):
    """dropout_rate > 0 adds the reference application's drop6 / drop7
    (owl/apps/imagenet_alexnet/alexnet.py:86-89,97-101) with the masks the library draws for
    the first two RandBernoulli calls after SetRandomSeed(seed_base).  keep=True also returns
    the activations ("acts") and sensitivities ("sens") of every layer in the results."""
    masks = dropout_masks(batch, dropout_rate, seed_base) if dropout_rate > 0.0 else None
    acts, out = alexnet_forward(p, data, batch, classes, masks)
    g, sens, l1 = alexnet_backward(p, acts, out, label, batch, classes, masks)
    newp = {k: _sgd(p[k], g[k], lr, batch) for k in p}
    res = {"prob": out}
    res.update({"g_" + k: v for k, v in g.items()})
    res.update({"l1_" + k: v for k, v in l1.items()})
    if keep:
        res["acts"], res["sens"] = acts, sens
    return newp, res


def make_inputs(kind, batch, seed=1000, classes=None):
    """Seeded host inputs of the benchmark configurations: weights ~ N(0, 0.01), biases 0,
    MNIST-like data uniform[0,1], AlexNet data ~ N(0,1), labels uniform one-hot."""
    rng = np.random.default_rng(seed)
    if kind == "mlp":
        shapes = {"w0": [256, 784], "b0": [256, 1], "w1": [10, 256], "b1": [10, 1]}
        data = rng.random(784 * batch, dtype=np.float32)
        classes = 10
    elif kind == "cnn":
        shapes = {"w0": [5, 5, 1, 16], "b0": [16], "w1": [5, 5, 16, 32], "b1": [32],
                  "w2": [10, 512], "b2": [10, 1]}
        data = rng.random(28 * 28 * batch, dtype=np.float32)
        classes = 10
    elif kind == "alexnet":
        classes = classes or 1000
        shapes = alexnet_param_shapes(classes)
        data = rng.standard_normal(227 * 227 * 3 * batch, dtype=np.float32)
    else:
        raise ValueError(kind)
    params = {}
    for name in sorted(shapes):
        n = int(np.prod(shapes[name]))
        params[name] = (np.zeros(n, np.float32) if name.startswith("b")
                        else (rng.standard_normal(n, dtype=np.float32) * np.float32(0.01)))
    lab = rng.integers(0, classes, size=batch)
    label = np.zeros((batch, classes), np.float32)
    label[np.arange(batch), lab] = 1.0
    return params, data, label.ravel()


# ---------------------------------------------------------------------------------------
# Caffe-style networks as the reference's owl.net package runs them (owl/owl/net/net.py):
# a chain of units, each a tuple; `acts[i]` is the output of unit i (acts[-1] of the data).
#   ("conv", name, C, K, H, W, pad, stride, kernel)   ConvConnection  net.py:639-731
#   ("relu",)                                          ReluUnit: gradient gated by the INPUT
#   ("lrn", C, H, W, local_size, alpha, beta)          LRNUnit
#   ("pool", C, H, W, kernel, stride, pad)             PoolingUnit (max)
#   ("fc", name, n_in, n_out)                          FullyConnection
#   ("dropout", n, ratio)                              DropoutUnit: x * mask * 1/(1-ratio)
# followed by the softmax loss unit: sens = prob - onehot.
def caffe_alexnet_units(classes=1000):
    return [("conv", "conv1", 3, 96, 227, 227, 0, 4, 11), ("relu",), ("lrn", 96, 55, 55, 5, 1e-4, 0.75),
            ("pool", 96, 55, 55, 3, 2, 0),
            ("conv", "conv2", 96, 256, 27, 27, 2, 1, 5), ("relu",), ("lrn", 256, 27, 27, 5, 1e-4, 0.75),
            ("pool", 256, 27, 27, 3, 2, 0),
            ("conv", "conv3", 256, 384, 13, 13, 1, 1, 3), ("relu",),
            ("conv", "conv4", 384, 384, 13, 13, 1, 1, 3), ("relu",),
            ("conv", "conv5", 384, 256, 13, 13, 1, 1, 3), ("relu",), ("pool", 256, 13, 13, 3, 2, 0),
            ("fc", "fc6", 9216, 4096), ("relu",), ("dropout", 4096, 0.5),
            ("fc", "fc7", 4096, 4096), ("relu",), ("dropout", 4096, 0.5),
            ("fc", "fc8", 4096, classes)]


def caffe_param_shapes(units):
    shapes = {}
    for u in units:
        if u[0] == "conv":
            _, name, C, K, _, _, _, _, k = u
            shapes[name] = ([k, k, C, K], [K])
        elif u[0] == "fc":
            shapes[u[1]] = ([u[3], u[2]], [u[3], 1])
    return shapes


def caffe_forward(units, params, data, batch, masks=()):
    """params: name -> (weight, bias).  masks: one Bernoulli mask per dropout unit, in order
    (empty: the TEST phase, dropout passes through).  Returns (acts, probabilities)."""
    N = batch
    acts, x, masks = [], data, list(masks)
    for u in units:
        if u[0] == "conv":
            _, name, C, K, H, W, pad, stride, k = u
            x = ora.conv_fwd(x, params[name][0], params[name][1], N, C, K, H, W, pad, pad, stride, stride, k, k)
        elif u[0] == "relu":
            x = _relu(x)
        elif u[0] == "lrn":
            _, C, H, W, size, alpha, beta = u
            x = ora.lrn_fwd(x, size, alpha, beta, N, C, H, W)[0]
        elif u[0] == "pool":
            _, C, H, W, k, s, p = u
            x = ora.pool_fwd(ora.POOL_MAX, x, N, C, H, W, s, s, k, k, p, p)
        elif u[0] == "fc":
            _, name, nin, nout = u
            x = _fc(params[name][0], x, params[name][1], nout, nin, N)
        elif u[0] == "dropout":
            if masks:
                scale = np.float32(1.0 / (1.0 - u[2]))
                x = ora.arithmetic_const(ora.MUL, 1, scale, ora.arithmetic(ora.MUL, x, masks.pop(0)))
        else:
            raise ValueError(u[0])
        acts.append(x)
    classes = units[-1][3]
    return acts, ora.softmax_instance_fwd(x, N, classes, 1, 1)


def caffe_backward(units, params, data, acts, prob, labels, batch, masks=()):
    """Gradients name -> (weight gradient, bias gradient) from given forward results (the
    oracle's own or another implementation's: see alexnet_backward)."""
    N = batch
    classes = units[-1][3]
    onehot = np.zeros((N, classes), np.float32)
    onehot[np.arange(N), np.asarray(labels).astype(np.int64)] = 1
    sen = ora.arithmetic(ora.SUB, prob, onehot.ravel())
    masks = list(masks)
    grads = {}
    mm = lambda a, b, m, n, k: ora.matmult(a, b, m, n, k, fast=True)
    for i in range(len(units) - 1, -1, -1):
        u = units[i]
        bottom = acts[i - 1] if i > 0 else data
        if u[0] == "conv":
            _, name, C, K, H, W, pad, stride, k = u
            geo = (N, C, K, H, W, pad, pad, stride, stride, k, k)
            Ho = (H + 2 * pad - k) // stride + 1
            grads[name] = (ora.conv_bwd_filter(sen, bottom, *geo), ora.conv_bwd_bias(sen, N, K, Ho, Ho))
            sen = ora.conv_bwd_data(sen, params[name][0], *geo) if i > 0 else None
        elif u[0] == "relu":
            sen = ora.activation_bwd(ora.RELU, sen, acts[i], bottom)
        elif u[0] == "lrn":
            _, C, H, W, size, alpha, beta = u
            top, scale = ora.lrn_fwd(bottom, size, alpha, beta, N, C, H, W)
            sen = ora.lrn_bwd(bottom, top, scale, sen, size, alpha, beta, N, C, H, W)
        elif u[0] == "pool":
            _, C, H, W, k, s, p = u
            sen = ora.pool_bwd(ora.POOL_MAX, sen, acts[i], bottom, N, C, H, W, s, s, k, k, p, p)
        elif u[0] == "fc":
            _, name, nin, nout = u
            grads[name] = (mm(sen, ora.transpose(bottom, N, nin), nout, nin, N),
                           ora.reduction(ora.SUM, sen, [nout, N], [1]))
            sen = mm(ora.transpose(params[name][0], nin, nout), sen, nin, N, nout)
        elif u[0] == "dropout":
            if masks:
                scale = np.float32(1.0 / (1.0 - u[2]))
                sen = ora.arithmetic_const(ora.MUL, 1, scale, ora.arithmetic(ora.MUL, sen, masks.pop()))
    return grads


def caffe_update(value, delta, grad, base_lr, lr_mult, weight_decay, decay_mult, momentum, batch):
    """WeightedComputeUnit.weight_update (net.py:241-262), operation by operation in fp32:
    delta' = momentum*delta - (lr*lr_mult/batch)*grad - (lr*lr_mult*wd*decay_mult)*value;
    value' = value + delta'.  Returns (value', delta')."""
    f = np.float32
    t = ora.arithmetic_const(ora.MUL, 0, f(momentum), delta)
    t = ora.arithmetic(ora.SUB, t, ora.arithmetic_const(ora.MUL, 0, f(base_lr * lr_mult / batch), grad))
    t = ora.arithmetic(ora.SUB, t, ora.arithmetic_const(ora.MUL, 0, f(base_lr * lr_mult * weight_decay * decay_mult), value))
    return ora.arithmetic(ora.ADD, value, t), t
