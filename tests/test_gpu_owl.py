"""The NArray front end (minerva_amd.owl) on the GPU: shape conventions, operators and the
training steps of the reference's Python applications (owl/apps/mnist/mnist_mlp.py:41-60,
owl/apps/mnist/mnist_cnn.py:55-83), written against the front end exactly as those
programs are written against the reference's binding, and checked against numpy
(bit-exact where one IEEE operation is involved) and the CPU oracle (1e-4 normwise)."""
import numpy as np
import pytest

from gpu_util import ALEX_ACT_ELEMS, TOL, assert_bits_equal, compare_alexnet_step, normwise, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def owl():
    from minerva_amd import owl as front
    dev = front.create_gpu_device(0)
    front.set_device(dev)
    yield front
    front.close_devices()


@pytest.fixture(scope="module")
def ora():
    from oracle import mnv_oracle
    return mnv_oracle


def _rand(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def _nd(owl, flat, shape):
    """NArray of Minerva shape `shape` over a flat buffer in Minerva's element order."""
    return owl.from_numpy(np.asarray(flat, np.float32).reshape(list(reversed(shape))))


def test_shapes_follow_minerva(owl):
    a = _rand((3, 4, 5), 1)
    n = owl.from_numpy(a)
    assert n.shape == [5, 4, 3]                       # dimensions reversed, same bytes
    assert_bits_equal(n.to_numpy(), a, "round trip")
    assert n.to_numpy().shape == (3, 4, 5)
    r = n.reshape([20, 3])
    assert r.shape == [20, 3]
    assert_bits_equal(r.to_numpy().ravel(), a.ravel(), "reshape keeps the element order")
    z, o = owl.zeros([7, 2]), owl.ones([7, 2])
    assert z.shape == [7, 2] and z.count_zero() == 14 and o.count_zero() == 0
    assert_bits_equal(o.to_numpy(), np.ones((2, 7), np.float32), "ones")
    assert owl.has_cuda() == 1 and owl.get_gpu_device_count() >= 1
    with pytest.raises(NotImplementedError):
        owl.create_cpu_device()


def test_operators_are_single_ieee_operations(owl):
    from minerva_amd.owl import elewise as ele
    x, y = _rand((33, 17), 2), _rand((33, 17), 3) + np.float32(3)
    a, b = owl.from_numpy(x), owl.from_numpy(y)
    say("owl arithmetic")
    f = np.float32
    cases = {
        "a+b": (a + b, x + y), "a-b": (a - b, x - y), "a/b": (a / b, x / y),
        "mult": (ele.mult(a, b), x * y),
        "a+c": (a + 2.5, x + f(2.5)), "c+a": (2.5 + a, f(2.5) + x),
        "a-c": (a - 2.5, x - f(2.5)), "c-a": (2.5 - a, f(2.5) - x),
        "a*c": (a * 3.0, x * f(3)), "c*a": (3.0 * a, f(3) * x),
        "a/c": (a / 3.0, x / f(3)), "c/b": (3.0 / b, f(3) / y),
        "-a": (-a, -x),
    }
    for name, (got, want) in cases.items():
        assert_bits_equal(got.to_numpy(), want, name)
    c = owl.from_numpy(x)
    c += b
    c -= 1.5
    c *= 2.0
    c /= b
    assert_bits_equal(c.to_numpy(), ((x + y) - f(1.5)) * f(2) / y, "in-place chain")
    assert_bits_equal(a.to_numpy(), x, "operands are not modified")


def test_matrix_product_transpose_and_broadcast(owl):
    m, k, n = 37, 29, 11
    A, B = _rand((m, k), 4), _rand((k, n), 5)      # mathematical matrices
    a, b = owl.from_numpy(A.T.copy()), owl.from_numpy(B.T.copy())
    assert a.shape == [m, k] and b.shape == [k, n]
    say("owl matmult")
    c = a * b
    assert c.shape == [m, n]
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert normwise(c.to_numpy().T, want) <= TOL
    assert_bits_equal(a.trans().to_numpy(), A, "trans")
    col, row = _rand((m, 1), 6), _rand((1, n), 7)
    cn = c.to_numpy().T
    assert_bits_equal((c + owl.from_numpy(col.T.copy())).to_numpy().T, cn + col, "{m,n} + {m,1}")
    assert_bits_equal((c - owl.from_numpy(row.T.copy())).to_numpy().T, cn - row, "{m,n} - {1,n}")
    d = owl.from_numpy(A.T.copy())
    d *= b                                              # `*=` of two arrays is the product too
    assert_bits_equal(d.to_numpy(), c.to_numpy(), "a *= b")


def test_reductions_and_argmax(owl):
    m, n = 23, 14
    X = _rand((m, n), 8)
    X[3, 5] = X[7, 5] = 9.0                            # a tie: the lower index wins
    x = owl.from_numpy(X.T.copy())
    say("owl reductions")
    assert x.sum(0).shape == [1, n] and x.sum(1).shape == [m, 1]
    assert normwise(x.sum(0).to_numpy().ravel(), X.astype(np.float64).sum(axis=0)) <= TOL
    assert normwise(x.sum(1).to_numpy().ravel(), X.astype(np.float64).sum(axis=1)) <= TOL
    assert_bits_equal(x.max(0).to_numpy().ravel(), X.max(axis=0), "max over dim 0")
    assert_bits_equal(x.max(1).to_numpy().ravel(), X.max(axis=1), "max over dim 1")
    assert_bits_equal(x.max_index(0).to_numpy().ravel(), X.argmax(axis=0).astype(np.float32), "max_index")
    assert x.max_index(0).to_numpy().ravel()[5] == 3.0
    assert normwise(x.sum([0, 1]).to_numpy().ravel(), [X.astype(np.float64).sum()]) <= TOL
    rel = owl.from_numpy(np.maximum(X, 0))
    assert rel.count_zero() == int((X <= 0).sum())


def test_elementwise_functions(owl, ora):
    from minerva_amd.owl import elewise as ele
    X, DY = _rand((19, 21), 9), _rand((19, 21), 10)
    x, dy = owl.from_numpy(X), owl.from_numpy(DY)
    say("owl elewise")
    assert normwise(ele.exp(x).to_numpy(), np.exp(X.astype(np.float64))) <= TOL
    assert normwise(ele.ln(ele.exp(x)).to_numpy(), X) <= TOL
    assert normwise(ele.sigm(x).to_numpy(), 1 / (1 + np.exp(-X.astype(np.float64)))) <= TOL
    assert normwise(ele.tanh(x).to_numpy(), np.tanh(X.astype(np.float64))) <= TOL
    assert_bits_equal(ele.relu(x).to_numpy(), np.maximum(X, 0) + np.float32(0), "relu")
    y = ele.relu(x)
    assert_bits_equal(ele.relu_back(dy, y).to_numpy(), np.where(X > 0, DY, np.float32(0)), "relu_back")
    s = ele.sigm(x)
    sn = s.to_numpy().astype(np.float64)
    assert normwise(ele.sigm_back(dy, s).to_numpy(), DY * sn * (1 - sn)) <= TOL
    t = ele.tanh(x)
    tn = t.to_numpy().astype(np.float64)
    assert normwise(ele.tanh_back(dy, t).to_numpy(), DY * (1 - tn * tn)) <= TOL


def test_concat_slice_and_random(owl):
    A, B = _rand((6, 5), 11), _rand((4, 5), 12)       # Minerva shapes [5,6] and [5,4]
    a, b = owl.from_numpy(A), owl.from_numpy(B)
    c = owl.concat([a, b], 1)
    assert c.shape == [5, 10]
    assert_bits_equal(c.to_numpy(), np.concatenate([A, B], axis=0), "concat along dim 1")
    s = owl.slice(c, 1, 2, 5)
    assert_bits_equal(s.to_numpy(), np.concatenate([A, B], axis=0)[2:7], "slice along dim 1")
    owl.set_random_seed(77)
    r = owl.randn([512, 256], 1.0, 0.5).to_numpy()
    assert abs(r.mean() - 1.0) < 0.01 and abs(r.std() - 0.5) < 0.01
    p = owl.randb([512, 256], 0.3).to_numpy()
    assert set(np.unique(p)) <= {0.0, 1.0} and abs(p.mean() - 0.3) < 0.01
    owl.set_random_seed(77)
    assert_bits_equal(owl.randn([512, 256], 1.0, 0.5).to_numpy(), r, "same seed, same numbers")


def _step_size(lr, batch):
    return float(np.float32(lr) / np.float32(batch))


def test_mlp_training_step_like_the_reference_app(owl, ora):
    """owl/apps/mnist/mnist_mlp.py:41-60 line by line, on the seeded benchmark inputs."""
    from minerva_amd.owl import conv as co, elewise as ele
    from oracle import nets
    batch, lr = 256, 0.01
    params, data, label = nets.make_inputs("mlp", batch)
    want_p, res = nets.mlp_step(dict(params), data, label, lr, batch)
    say("owl mlp step")
    w1, b1 = _nd(owl, params["w0"], [256, 784]), _nd(owl, params["b0"], [256, 1])
    w2, b2 = _nd(owl, params["w1"], [10, 256]), _nd(owl, params["b1"], [10, 1])
    a1, target = _nd(owl, data, [784, batch]), _nd(owl, label, [10, batch])
    a2 = ele.relu(w1 * a1 + b1)
    a3 = w2 * a2 + b2
    out = co.softmax(a3)
    s3 = out - target
    s2 = ele.relu_back(w2.trans() * s3, a2)
    gw1, gb1 = s2 * a1.trans(), s2.sum(1)
    gw2, gb2 = s3 * a2.trans(), s3.sum(1)
    eps = _step_size(lr, batch)
    w1 -= eps * gw1
    w2 -= eps * gw2
    b1 -= eps * gb1
    b2 -= eps * gb2
    owl.wait_for_all()
    assert out.shape == [10, batch]
    assert normwise(out.to_numpy().ravel(), res["prob"]) <= TOL
    for got, key in ((gw1, "w0"), (gb1, "b0"), (gw2, "w1"), (gb2, "b1")):
        ref = res["g_" + key].astype(np.float64)
        bound = TOL * float(np.max(np.abs(ref)))
        assert float(np.max(np.abs(got.to_numpy().ravel() - ref))) <= bound, "gradient " + key
    for got, key in ((w1, "w0"), (b1, "b0"), (w2, "w1"), (b2, "b1")):
        assert normwise(got.to_numpy().ravel(), want_p[key]) <= TOL, "updated " + key
    # the accuracy check of the application: arg-max of the output against the labels
    wrong = np.count_nonzero((out.max_index(0) - target.max_index(0)).to_numpy())
    ref_wrong = np.count_nonzero(res["prob"].reshape(batch, 10).argmax(axis=1) !=
                                 label.reshape(batch, 10).argmax(axis=1))
    assert wrong == ref_wrong


def test_cnn_training_step_like_the_reference_app(owl, ora):
    """owl/apps/mnist/mnist_cnn.py:55-83 (second stage padded by 2 and pooled 3x3/3 as the
    application does), on the seeded benchmark inputs."""
    from minerva_amd.owl import conv, elewise as ele
    from oracle import nets
    batch, lr = 16, 0.01
    params, data, label = nets.make_inputs("cnn", batch)
    want_p, res = nets.cnn_step(dict(params), data, label, lr, batch, pad2=2, pool2=3)
    say("owl cnn step")
    convs = [conv.Convolver(0, 0, 1, 1), conv.Convolver(2, 2, 1, 1)]
    pools = [conv.Pooler(2, 2, 2, 2, 0, 0, conv.pool_op.max), conv.Pooler(3, 3, 3, 3, 0, 0, conv.pool_op.max)]
    weights = [_nd(owl, params["w0"], [5, 5, 1, 16]), _nd(owl, params["w1"], [5, 5, 16, 32]),
               _nd(owl, params["w2"], [10, 512])]
    bias = [_nd(owl, params["b0"], [16]), _nd(owl, params["b1"], [32]), _nd(owl, params["b2"], [10, 1])]
    samples = _nd(owl, data, [28, 28, 1, batch])
    target = _nd(owl, label, [10, batch])
    fc_shape = [512, batch]
    acts = [None] * 6
    acts[0] = samples
    acts[1] = ele.relu(convs[0].ff(acts[0], weights[0], bias[0]))
    acts[2] = pools[0].ff(acts[1])
    acts[3] = ele.relu(convs[1].ff(acts[2], weights[1], bias[1]))
    acts[4] = pools[1].ff(acts[3])
    acts[5] = weights[2] * acts[4].reshape(fc_shape) + bias[2]
    out = conv.softmax(acts[5], conv.soft_op.instance)
    errs = [None] * 6
    errs[5] = out - target
    errs[4] = (weights[2].trans() * errs[5]).reshape(acts[4].shape)
    errs[3] = ele.relu_back(pools[1].bp(errs[4], acts[4], acts[3]), acts[3])
    errs[2] = convs[1].bp(errs[3], acts[2], weights[1])
    errs[1] = ele.relu_back(pools[0].bp(errs[2], acts[2], acts[1]), acts[1])
    wgrad = [convs[0].weight_grad(errs[1], acts[0], weights[0]),
             convs[1].weight_grad(errs[3], acts[2], weights[1]),
             errs[5] * acts[4].reshape(fc_shape).trans()]
    bgrad = [convs[0].bias_grad(errs[1]), convs[1].bias_grad(errs[3]), errs[5].sum(1)]
    eps = _step_size(lr, batch)
    for k in range(3):
        weights[k] -= eps * wgrad[k]
        bias[k] -= eps * bgrad[k]
    owl.wait_for_all()
    assert acts[1].shape == [24, 24, 16, batch] and acts[4].shape == [4, 4, 32, batch]
    assert normwise(out.to_numpy().ravel(), res["prob"]) <= TOL
    for k in range(3):
        ref = res["g_w%d" % k].astype(np.float64)
        assert float(np.max(np.abs(wgrad[k].to_numpy().ravel() - ref))) <= TOL * float(np.max(np.abs(ref))), k
        assert normwise(bgrad[k].to_numpy().ravel(), res["g_b%d" % k]) <= TOL, k
        assert normwise(weights[k].to_numpy().ravel(), want_p["w%d" % k]) <= TOL
        assert normwise(bias[k].to_numpy().ravel(), want_p["b%d" % k]) <= TOL


def test_lrn_and_average_pooling_wrappers(owl, ora):
    from minerva_amd.owl import conv
    N, C, H, W = 2, 7, 5, 6
    X, DY = _rand((N, C, H, W), 13), _rand((N, C, H, W), 14)
    x = owl.from_numpy(X)
    say("owl lrn / avg pool")
    lrn = conv.Lrner(5, 1e-4, 0.75)
    scale = owl.zeros(x.shape)
    top = lrn.ff(x, scale)
    want_top, want_scale = ora.lrn_fwd(X.ravel(), 5, 1e-4, 0.75, N, C, H, W)
    assert normwise(top.to_numpy().ravel(), want_top) <= TOL
    assert normwise(scale.to_numpy().ravel(), want_scale) <= TOL
    dx = lrn.bp(x, top, scale, owl.from_numpy(DY))
    want_dx = ora.lrn_bwd(X.ravel(), want_top, want_scale, DY.ravel(), 5, 1e-4, 0.75, N, C, H, W)
    assert normwise(dx.to_numpy().ravel(), want_dx) <= TOL
    pool = conv.Pooler(3, 3, 2, 2, 1, 1, conv.pool_op.avg)
    y = pool.ff(x)
    want_y = ora.pool_fwd(ora.POOL_AVG, X.ravel(), N, C, H, W, 2, 2, 3, 3, 1, 1)
    assert normwise(y.to_numpy().ravel(), want_y) <= TOL
    sm = conv.softmax(owl.from_numpy(_rand((4, 3, 2, 5), 15)), conv.soft_op.channel)
    assert sm.shape == [5, 2, 3, 4]


def test_alexnet_application_step_with_dropout(owl, ora):
    """The AlexNet application (owl/apps/imagenet_alexnet/alexnet.py:64-126) on the front end,
    drop6 / drop7 included: the masks are the library's first two Bernoulli draws after
    seeding, which the oracle reproduces from the seed."""
    from minerva_amd.owl import models
    from oracle import nets
    batch, lr, seed, keep = 2, 0.01, 424242, 0.5
    params, data, label = nets.make_inputs("alexnet", batch)
    masks = nets.dropout_masks(batch, keep, seed)
    say("alexnet + dropout oracle forward b=2 (CPU)")
    ora_acts, ora_prob = nets.alexnet_forward(params, data, batch, masks=masks)
    say("owl alexnet step b=2")
    net = models.AlexNet()
    net.keep_activations = True
    net.load([params["w%d" % k] for k in range(8)], [params["b%d" % k] for k in range(8)])
    owl.set_random_seed(seed)
    out, wgrad, bgrad = net.train_one_mb(_nd(owl, data, [227, 227, 3, batch]),
                                         _nd(owl, label, [1000, batch]), keep)
    net.sgd(wgrad, bgrad, batch, lr)
    owl.wait_for_all()
    got = {"prob": out.to_numpy().ravel()}
    for k in range(8):
        got["g_w%d" % k] = wgrad[k].to_numpy().ravel()
        got["g_b%d" % k] = bgrad[k].to_numpy().ravel()
        got["w%d" % k] = net.weights[k].to_numpy().ravel()
        got["b%d" % k] = net.bias[k].to_numpy().ravel()
    gpu_acts = {i: net.last_acts[i].to_numpy().ravel() for i in ALEX_ACT_ELEMS}
    net.last_acts = None
    compare_alexnet_step(got, gpu_acts, params, data, label, batch, lr, ora_acts, ora_prob, masks=masks)
    # the momentum / weight-decay update of the application, one step from zero deltas
    before = [w.to_numpy().copy() for w in net.weights]
    net.update(wgrad, bgrad, batch, 0.9, lr, 0.0005)
    f = np.float32
    for k in (0, 7):
        delta = (f(0.9) * f(0)) - f(lr / batch) * wgrad[k].to_numpy() - f(lr * 0.0005) * before[k]
        assert normwise(net.weights[k].to_numpy(), before[k] + delta) <= 1e-6


def test_errors_surface_as_exceptions(owl):
    """The reference aborts the process on a failed CHECK; the front end raises instead."""
    from minerva_amd import hostapi
    a, b = owl.zeros([4, 3]), owl.zeros([5, 3])
    with pytest.raises(hostapi.HostError):
        a + b                      # neither equal shapes nor a dimension of size 1
    with pytest.raises(hostapi.HostError):
        a * b                      # inner dimensions differ
    with pytest.raises(hostapi.HostError):
        a.sum(2)                   # no such dimension
    with pytest.raises(ValueError):
        owl.zeros([4, 0])
    with pytest.raises(ValueError):
        owl.set_device(12345)
    # the device keeps working after a refused operator
    assert (a + 1.0).count_zero() == 0
