"""The opt-in fused epilogues through the C ABI: each fused entry point must return, bit for
bit, what the chain of separate entry points returns (same IEEE operations in the same
order), on shapes that reach every convolution policy, tile shape and split path, the SGEMM
tiles with and without k ranges, and every pooling-gradient kernel; and, like the separate
operators, agree with the CPU oracle normwise to 1e-4 (selections bit for bit)."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, TOL, assert_bits_equal, net_batches, normwise, run_steps, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


def _rand(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def _ws(gpu, query, args, workspace):
    nbytes = getattr(gpu.L, query)(*args) if workspace else 0
    buf = gpu.empty(nbytes // 4 + 1) if nbytes else None
    return (buf.p if buf else None), ctypes.c_size_t(nbytes), buf


CONV = [
    # N, C, K, H, W, ph, pw, sv, sh, R, S
    (2, 3, 4, 7, 9, 0, 0, 1, 1, 3, 5),        # generic / no-padding policies, 128x32 tile
    (2, 2, 3, 8, 7, 2, 1, 2, 3, 3, 2),        # strided, padded, ragged fit
    (3, 32, 48, 10, 11, 1, 2, 1, 1, 3, 5),    # (tap, channel) fast policies
    (5, 130, 70, 9, 9, 1, 1, 1, 1, 3, 3),     # several tiles in both GEMM dimensions
    (8, 16, 96, 48, 48, 1, 1, 1, 1, 3, 3),    # 96-column tiles forward
    (8, 96, 16, 48, 48, 1, 1, 1, 1, 3, 3),    # 96-column tiles in the data gradient
    (2, 24, 33, 15, 14, 0, 0, 1, 1, 4, 4),    # reduction cut into k ranges on small tiles
    (2, 16, 32, 12, 12, 2, 2, 1, 1, 5, 5),    # MNIST CNN layer 2
    (4, 3, 96, 227, 227, 0, 0, 4, 4, 11, 11),  # AlexNet conv1
    (4, 384, 256, 13, 13, 1, 1, 1, 1, 3, 3),   # AlexNet conv5
]


@pytest.mark.parametrize("p", CONV, ids=lambda p: "x".join(map(str, p)))
@pytest.mark.parametrize("workspace", [True, False])
def test_conv_fused_epilogues_equal_the_operator_chain(gpu, ora, p, workspace):
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    Ho, Wo = (H + 2 * ph - R) // sv + 1, (W + 2 * pw - S) // sh + 1
    x, w, b = _rand(N * C * H * W, 140), _rand(K * C * R * S, 141, 0.1), _rand(K, 142, 0.5)
    nt, nb = N * K * Ho * Wo, N * C * H * W
    dx, dw, db = gpu.up(x), gpu.up(w), gpu.up(b)
    conv, chain, fused = gpu.empty(nt), gpu.empty(nt), gpu.up(np.full(nt, np.nan, np.float32))
    wp, wb, keep = _ws(gpu, "mnv_conv_fwd_workspace_bytes", p, workspace)
    say("conv fwd + relu", p, workspace)
    gpu.call("mnv_conv_fwd", dx.p, dw.p, db.p, conv.p, *p, wp, wb)
    gpu.call("mnv_relu_fwd", conv.p, chain.p, ctypes.c_size_t(nt))
    gpu.call("mnv_conv_fwd_relu", dx.p, dw.p, db.p, fused.p, *p, wp, wb)
    got = gpu.down(fused)
    assert_bits_equal(got, gpu.down(chain), "conv_fwd_relu vs conv_fwd + relu_fwd")
    if N * K * Ho * Wo * C * R * S < 3e8:
        ref = ora.activation_fwd(ora.RELU, ora.conv_fwd(x, w, b, *p))
        assert normwise(got, ref) <= TOL
    # data gradient gated by the activations of the convolution's input
    dy = _rand(nt, 143)
    act = np.maximum(_rand(nb, 144), 0).astype(np.float32)   # post-ReLU values: many zeros
    ddy, dact = gpu.up(dy), gpu.up(act)
    plain, chain, fused = gpu.empty(nb), gpu.empty(nb), gpu.up(np.full(nb, np.nan, np.float32))
    wp, wb, keep = _ws(gpu, "mnv_conv_bwd_data_workspace_bytes", p, workspace)
    say("conv bwd data + relu bwd", p, workspace)
    gpu.call("mnv_conv_bwd_data", ddy.p, dw.p, plain.p, *p, wp, wb)
    gpu.call("mnv_relu_bwd", dact.p, dact.p, plain.p, chain.p, ctypes.c_size_t(nb))
    gpu.call("mnv_conv_bwd_data_relu", ddy.p, dw.p, dact.p, fused.p, *p, wp, wb)
    got = gpu.down(fused)
    assert_bits_equal(got, gpu.down(chain), "conv_bwd_data_relu vs conv_bwd_data + relu_bwd")
    if N * K * Ho * Wo * C * R * S < 3e8:
        ref = ora.activation_bwd(ora.RELU, ora.conv_bwd_data(dy, w, *p), act, act)
        assert normwise(got, ref) <= TOL
    assert gpu.L.mnv_conv_bwd_data_relu(ddy.p, dw.p, None, fused.p, *p, wp, wb, gpu.dev.stream) == -1


@pytest.mark.parametrize("p", CONV, ids=lambda p: "x".join(map(str, p)))
@pytest.mark.parametrize("workspace", [True, False])
def test_filter_gradient_with_the_update_in_its_store(gpu, ora, p, workspace):
    """mnv_conv_bwd_filter_sgd against mnv_conv_bwd_filter followed by mnv_sgd_update, bit for
    bit, into a fresh filter and in place; against the oracle's three operators at 1e-4."""
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    Ho, Wo = (H + 2 * ph - R) // sv + 1, (W + 2 * pw - S) // sh + 1
    x, dy = _rand(N * C * H * W, 145), _rand(N * K * Ho * Wo, 146)
    w = _rand(K * C * R * S, 147, 0.1)
    scale = float(np.float32(0.01) / np.float32(N))
    dx, ddy, dw = gpu.up(x), gpu.up(dy), gpu.up(w)
    nf = w.size
    grad, chain = gpu.empty(nf), gpu.empty(nf)
    fused = gpu.up(np.full(nf, np.nan, np.float32))
    wp, wb, keep = _ws(gpu, "mnv_conv_bwd_filter_workspace_bytes", p, workspace)
    say("conv bwd filter + sgd update", p, workspace)
    gpu.call("mnv_conv_bwd_filter", dx.p, ddy.p, grad.p, *p, wp, wb)
    gpu.call("mnv_sgd_update", dw.p, grad.p, ctypes.c_float(scale), chain.p, ctypes.c_size_t(nf))
    gpu.call("mnv_conv_bwd_filter_sgd", dx.p, ddy.p, dw.p, ctypes.c_float(scale), fused.p, *p, wp, wb)
    want = gpu.down(chain)
    assert_bits_equal(gpu.down(fused), want, "conv_bwd_filter_sgd vs conv_bwd_filter + sgd_update")
    gpu.call("mnv_conv_bwd_filter_sgd", dx.p, ddy.p, dw.p, ctypes.c_float(scale), dw.p, *p, wp, wb)
    assert_bits_equal(gpu.down(dw), want, "conv_bwd_filter_sgd in place")
    if N * K * Ho * Wo * C * R * S < 3e8:
        g = ora.conv_bwd_filter(dy, x, *p)
        ref = ora.arithmetic(ora.SUB, w, ora.arithmetic_const(ora.MUL, 0, scale, g))
        # the update is small against the weights: compare the step taken, not the sum
        assert normwise(want - w, ref - w) <= 1e-3
        assert normwise(want, ref) <= TOL
    assert gpu.L.mnv_conv_bwd_filter_sgd(dx.p, ddy.p, None, ctypes.c_float(scale), fused.p, *p, wp, wb,
                                         gpu.dev.stream) == -1


GEMM = [(3, 5, 2), (37, 29, 53), (130, 70, 19), (256, 256, 784), (10, 256, 256), (1000, 256, 512),
        (4096, 256, 4096), (4096, 2, 9216), (1000, 2, 4096), (512, 384, 100)]


@pytest.mark.parametrize("m,n,k", GEMM)
@pytest.mark.parametrize("workspace", [True, False])
def test_sgemm_fused_epilogues_equal_the_operator_chain(gpu, m, n, k, workspace):
    a, b = _rand(m * k, 150, 0.1), _rand(k * n, 151)
    bias = _rand(m, 152)
    gate = np.maximum(_rand(m * n, 153), 0).astype(np.float32)
    da, db, dbias, dgate = gpu.up(a), gpu.up(b), gpu.up(bias), gpu.up(gate)
    prod, t1, t2 = gpu.empty(m * n), gpu.empty(m * n), gpu.empty(m * n)
    fused = gpu.up(np.full(m * n, np.nan, np.float32))
    wp, wb, keep = _ws(gpu, "mnv_sgemm_nn_workspace_bytes", (m, n, k), workspace)
    say("sgemm epilogues", m, n, k, workspace)
    gpu.call("mnv_sgemm_nn", da.p, db.p, prod.p, m, n, k, wp, wb)
    gpu.call("mnv_norm_add_row", prod.p, dbias.p, t1.p, m, n)
    gpu.call("mnv_sgemm_nn_bias", da.p, db.p, dbias.p, fused.p, m, n, k, 0, wp, wb)
    assert_bits_equal(gpu.down(fused), gpu.down(t1), "sgemm + bias")
    gpu.call("mnv_relu_fwd", t1.p, t2.p, ctypes.c_size_t(m * n))
    gpu.call("mnv_sgemm_nn_bias", da.p, db.p, dbias.p, fused.p, m, n, k, 1, wp, wb)
    got = gpu.down(fused)
    assert_bits_equal(got, gpu.down(t2), "sgemm + bias + relu")
    A = a.reshape(k, m).T.astype(np.float64)
    B = b.reshape(n, k).T.astype(np.float64)
    ref = np.maximum(A @ B + bias[:, None].astype(np.float64), 0)
    assert normwise(got.reshape(n, m).T, ref) <= TOL
    gpu.call("mnv_relu_bwd", dgate.p, dgate.p, prod.p, t1.p, ctypes.c_size_t(m * n))
    gpu.call("mnv_sgemm_nn_relu_bwd", da.p, db.p, dgate.p, fused.p, m, n, k, wp, wb)
    assert_bits_equal(gpu.down(fused), gpu.down(t1), "sgemm + relu gradient")


@pytest.mark.parametrize("m,n,k", [(7, 5, 3), (64, 64, 64), (130, 70, 33), (256, 784, 256), (784, 256, 10),
                                   (4096, 256, 1000), (1000, 256, 4096), (4096, 9216, 256),
                                   (9216, 256, 4096), (100, 36, 5000), (132, 260, 68),
                                   (2100, 2052, 260)])
@pytest.mark.parametrize("workspace", [True, False])
def test_sgemm_with_a_transposed_operand_equals_transpose_then_sgemm(gpu, m, n, k, workspace):
    """mnv_sgemm_tn / mnv_sgemm_nt against mnv_transpose followed by mnv_sgemm_nn (and
    mnv_relu_bwd for the gated form), bit for bit, and against the fp64 product."""
    a, b = _rand(m * k, 154, 0.1), _rand(k * n, 155)
    gate = np.maximum(_rand(m * n, 156), 0).astype(np.float32)
    da, db, dgate = gpu.up(a), gpu.up(b), gpu.up(gate)      # a{m,k}, b{k,n}
    at, bt = gpu.empty(m * k), gpu.empty(k * n)
    gpu.call("mnv_transpose", da.p, at.p, m, k)              # at{k,m}
    gpu.call("mnv_transpose", db.p, bt.p, k, n)              # bt{n,k}
    prod, gated = gpu.empty(m * n), gpu.empty(m * n)
    fused = gpu.up(np.full(m * n, np.nan, np.float32))
    wp, wb, keep = _ws(gpu, "mnv_sgemm_nn_workspace_bytes", (m, n, k), workspace)
    say("sgemm with transposed operands", m, n, k, workspace)
    gpu.call("mnv_sgemm_nn", da.p, db.p, prod.p, m, n, k, wp, wb)
    want = gpu.down(prod)
    gpu.call("mnv_sgemm_tn", at.p, db.p, None, fused.p, m, n, k, wp, wb)
    assert_bits_equal(gpu.down(fused), want, "A given transposed")
    gpu.call("mnv_sgemm_nt", da.p, bt.p, fused.p, m, n, k, wp, wb)
    assert_bits_equal(gpu.down(fused), want, "B given transposed")
    gpu.call("mnv_relu_bwd", dgate.p, dgate.p, prod.p, gated.p, ctypes.c_size_t(m * n))
    gpu.call("mnv_sgemm_tn", at.p, db.p, dgate.p, fused.p, m, n, k, wp, wb)
    assert_bits_equal(gpu.down(fused), gpu.down(gated), "A given transposed + relu gradient")
    A = a.reshape(k, m).T.astype(np.float64)
    B = b.reshape(n, k).T.astype(np.float64)
    assert normwise(want.reshape(n, m).T, A @ B) <= TOL
    # the weight gradient with the update in its store: w - scale * (a * bt^T)
    w = _rand(m * n, 157, 0.05)
    scale = float(np.float32(0.01) / np.float32(256))
    dw, chain = gpu.up(w), gpu.empty(m * n)
    gpu.call("mnv_sgd_update", dw.p, prod.p, ctypes.c_float(scale), chain.p, ctypes.c_size_t(m * n))
    gpu.call("mnv_sgemm_nt_sgd", da.p, bt.p, dw.p, ctypes.c_float(scale), fused.p, m, n, k, wp, wb)
    stepped = gpu.down(chain)
    assert_bits_equal(gpu.down(fused), stepped, "B given transposed + sgd update")
    gpu.call("mnv_sgemm_nt_sgd", da.p, bt.p, dw.p, ctypes.c_float(scale), dw.p, m, n, k, wp, wb)
    assert_bits_equal(gpu.down(dw), stepped, "B given transposed + sgd update, in place")


POOL = [
    # N, C, H, W, sv, sh, kh, kw, ph, pw
    (2, 96, 55, 55, 2, 2, 3, 3, 0, 0),    # AlexNet pool1: ordered scatter, large planes
    (3, 256, 13, 13, 2, 2, 3, 3, 0, 0),   # pool5: small configuration
    (4, 16, 24, 24, 2, 2, 2, 2, 0, 0),    # MNIST CNN: 2x2/2
    (4, 32, 12, 12, 3, 3, 3, 3, 0, 0),    # 3x3/3: the gather kernel
    (3, 5, 9, 11, 2, 2, 3, 3, 1, 1),      # padded: windows that start outside the plane
    (1, 2, 6, 5, 2, 3, 3, 2, 1, 1),       # rectangular window and strides
    (1, 3, 100, 95, 2, 2, 3, 3, 1, 1),    # planes too large for LDS: direct kernel
    (5000, 1, 6, 6, 2, 2, 3, 3, 0, 0),
]


def test_sgemm_transposed_operands_at_4096_cubed(gpu):
    """The benchmark's square product with either operand given transposed: the bits of
    transposing first (mnv_sgemm_nn at this size is checked against fp64 samples elsewhere)."""
    n = 4096
    a, b = _rand(n * n, 160, 0.1), _rand(n * n, 161)
    da, db = gpu.up(a), gpu.up(b)
    at, bt, prod = gpu.empty(n * n), gpu.empty(n * n), gpu.empty(n * n)
    fused = gpu.up(np.full(n * n, np.nan, np.float32))
    say("sgemm 4096^3 with transposed operands")
    gpu.call("mnv_transpose", da.p, at.p, n, n)
    gpu.call("mnv_transpose", db.p, bt.p, n, n)
    gpu.call("mnv_sgemm_nn", da.p, db.p, prod.p, n, n, n, None, ctypes.c_size_t(0))
    want = gpu.down(prod)
    gpu.call("mnv_sgemm_tn", at.p, db.p, None, fused.p, n, n, n, None, ctypes.c_size_t(0))
    assert_bits_equal(gpu.down(fused), want, "A given transposed, 4096^3")
    gpu.call("mnv_sgemm_nt", da.p, bt.p, fused.p, n, n, n, None, ctypes.c_size_t(0))
    assert_bits_equal(gpu.down(fused), want, "B given transposed, 4096^3")


@pytest.mark.parametrize("p", POOL)
def test_maxpool_bwd_relu_equals_the_operator_chain(gpu, ora, p):
    N, C, H, W, sv, sh, kh, kw, ph, pw = p
    rng = np.random.default_rng(160)
    # post-ReLU activations with heavy ties: whole windows of zeros, equal positive values
    x = np.maximum(rng.integers(-3, 4, size=N * C * H * W), 0).astype(np.float32)
    Ho, Wo = gpu.L.mnv_pooled_size(H, kh, sv, ph), gpu.L.mnv_pooled_size(W, kw, sh, pw)
    dy = _rand(N * C * Ho * Wo, 161)
    dx, ddy, top = gpu.up(x), gpu.up(dy), gpu.empty(N * C * Ho * Wo)
    routed, chain = gpu.empty(x.size), gpu.empty(x.size)
    fused = gpu.up(np.full(x.size, np.nan, np.float32))
    say("maxpool bwd + relu bwd", p)
    gpu.call("mnv_maxpool_fwd", dx.p, top.p, *p)
    gpu.call("mnv_maxpool_bwd", dx.p, top.p, ddy.p, routed.p, *p)
    gpu.call("mnv_relu_bwd", dx.p, dx.p, routed.p, chain.p, ctypes.c_size_t(x.size))
    gpu.call("mnv_maxpool_bwd_relu", dx.p, top.p, ddy.p, fused.p, *p)
    got = gpu.down(fused)
    assert_bits_equal(got, gpu.down(chain), "maxpool_bwd_relu vs maxpool_bwd + relu_bwd")
    topo = ora.pool_fwd(ora.POOL_MAX, x, *p)
    ref = ora.activation_bwd(ora.RELU, ora.pool_bwd(ora.POOL_MAX, dy, topo, x, *p), x, x)
    assert_bits_equal(got, ref, "maxpool_bwd_relu vs the oracle's two operators")
    # activations that are not post-ReLU (negative maxima, NaN): the gate still equals the chain
    x2 = _rand(x.size, 162)
    x2[::97] = np.nan
    dx2 = gpu.up(x2)
    gpu.call("mnv_maxpool_bwd", dx2.p, top.p, ddy.p, routed.p, *p)
    gpu.call("mnv_relu_bwd", dx2.p, dx2.p, routed.p, chain.p, ctypes.c_size_t(x.size))
    gpu.call("mnv_maxpool_bwd_relu", dx2.p, top.p, ddy.p, fused.p, *p)
    assert_bits_equal(gpu.down(fused), gpu.down(chain), "gate on arbitrary activations")


@pytest.mark.parametrize("n", [1, 5, 4099, 1 << 20, 37748736])
def test_sgd_update_equals_scale_then_subtract(gpu, ora, n):
    w, g = _rand(n, 170, 0.01), _rand(n, 171)
    scale = float(np.float32(0.01) / np.float32(256))
    dw, dg, step, chain = gpu.up(w), gpu.up(g), gpu.empty(n), gpu.empty(n)
    fused = gpu.up(np.full(n, np.nan, np.float32))
    say("sgd update", n)
    gpu.call("mnv_const_mul", dg.p, step.p, ctypes.c_float(scale), ctypes.c_size_t(n))
    gpu.call("mnv_sub", dw.p, step.p, chain.p, ctypes.c_size_t(n))
    gpu.call("mnv_sgd_update", dw.p, dg.p, ctypes.c_float(scale), fused.p, ctypes.c_size_t(n))
    got = gpu.down(fused)
    assert_bits_equal(got, gpu.down(chain), "sgd_update vs const_mul + sub")
    ref = ora.arithmetic(ora.SUB, w, ora.arithmetic_const(ora.MUL, 0, scale, g))
    assert_bits_equal(got, ref, "sgd_update vs the oracle's two operators")


@pytest.mark.parametrize("kind,batch,variant", [("mlp", 256, 0), ("cnn", 256, 0), ("cnn", 16, 1),
                                                ("alexnet", 2, 0), ("alexnet", 256, 0)])
def test_fused_training_steps_bit_identical_to_operator_by_operator(kind, batch, variant):
    """The training graphs with the fused operators switched on: every parameter, gradient
    and probability after each of two steps has the bits of the operator-by-operator step
    (which the other tests compare with the oracle), with fewer operators issued."""
    params, batches = net_batches(kind, batch, 2 if batch < 256 or kind != "alexnet" else 1)
    say("fused vs separate operators:", kind, batch, variant)
    plain = run_steps(kind, batch, variant, 0.01, params, batches)
    ops_plain = run_steps.ops_issued
    fused = run_steps(kind, batch, variant, 0.01, params, batches, fused=True)
    ops_fused = run_steps.ops_issued
    updates = run_steps(kind, batch, variant, 0.01, params, batches, fused_updates=True)
    ops_updates = run_steps.ops_issued
    for step, (a, b, c) in enumerate(zip(plain, fused, updates)):
        for k in a:
            assert_bits_equal(b[k], a[k], "%s after step %d" % (k, step))
        # with the weight updates folded into the gradient kernels there are no weight
        # gradients to read; everything else, the updated weights first of all, keeps its bits
        assert sorted(set(a) - set(c)) == sorted("g_" + k for k in params if k.startswith("w"))
        for k in c:
            assert_bits_equal(c[k], a[k], "%s after step %d, updates in the gradient kernels" % (k, step))
    assert ops_updates < ops_fused < ops_plain
    say("  operators issued: %d with fused updates, %d fused, %d separate" % (ops_updates, ops_fused, ops_plain))


def test_fused_host_operators_by_name():
    """The fused operators through the named-operator entry of the host layer, each against
    the pair of separate operators."""
    from minerva_amd import hostapi
    r = hostapi.Runtime(0, sync_each_op=True)
    x = r.tensor(_rand(2 * 3 * 9 * 8, 180), [8, 9, 3, 2])
    w = r.tensor(_rand(5 * 3 * 3 * 3, 181), [3, 3, 3, 5])
    b = r.tensor(_rand(5, 182), [5])
    conv = [1, 1, 1, 1]
    y = r.top("relu_forward", [r.top("conv_forward", [x, w, b], conv)])
    assert_bits_equal(r.top("conv_forward_relu", [x, w, b], conv).read(), y.read(), "conv+relu")
    dy = r.tensor(_rand(int(np.prod(y.dims)), 183), y.dims)
    act = r.top("relu_forward", [x])
    want = r.top("relu_backward", [r.top("conv_backward_data", [dy, act, w], conv), act, act])
    got = r.top("conv_backward_data_relu", [dy, act, w], conv)
    assert_bits_equal(got.read(), want.read(), "conv bwd data + relu bwd")
    pool = [0, 3, 3, 2, 2, 0, 0]
    top = r.top("pooling_forward", [act], pool)
    dt = r.tensor(_rand(int(np.prod(top.dims)), 184), top.dims)
    want = r.top("relu_backward", [r.top("pooling_backward", [dt, top, act], pool), act, act])
    got = r.top("pooling_backward_relu", [dt, top, act], pool[1:])
    assert_bits_equal(got.read(), want.read(), "pool bwd + relu bwd")
    a = r.tensor(_rand(37 * 21, 185), [37, 21])
    bm = r.tensor(_rand(21 * 13, 186), [21, 13])
    bias = r.tensor(_rand(37, 187), [37, 1])
    prod = r.top("matmult", [a, bm])
    plus = r.top("norm_arithmetic", [prod, bias], [0])
    assert_bits_equal(r.top("matmult_bias", [a, bm, bias], [0]).read(), plus.read(), "fc")
    assert_bits_equal(r.top("matmult_bias", [a, bm, bias], [1]).read(),
                      r.top("relu_forward", [plus]).read(), "fc + relu")
    gate = r.top("relu_forward", [r.tensor(_rand(37 * 13, 188), [37, 13])])
    assert_bits_equal(r.top("matmult_relu_backward", [a, bm, gate]).read(),
                      r.top("relu_backward", [prod, gate, gate]).read(), "matmult + relu bwd")
    g = r.tensor(_rand(37 * 21, 189), [37, 21])
    step = r.top("arithmetic_const", [g], [2, 0.125, 0])
    assert_bits_equal(r.top("sgd_update", [a, g], [0.125]).read(),
                      r.top("arithmetic", [a, step], [1]).read(), "sgd update")
    with pytest.raises(hostapi.HostError):
        r.top("matmult_bias", [a, bm, b], [0])          # bias of the wrong extent
    with pytest.raises(hostapi.HostError):
        r.top("sgd_update", [a, bm], [0.1])                # gradient of another size
    r.close()
