"""The C++ host layer on the GPU: every Minerva operator through closure -> Task ->
HipDevice -> FnBundle -> hip::<Op> -> C ABI, checked against the CPU oracle in the style
of the reference's own unit tests (tests/unittest_*.cpp), plus the device's allocator,
its four-stream thread pool, its error convention, and the three training graphs."""
import json
import os

import numpy as np
import pytest

from gpu_util import (ALEX_ACT_ELEMS, TOL, assert_bits_equal, compare_alexnet_step, compare_step,
                      normwise, say)

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def rt():
    from minerva_amd import hostapi
    r = hostapi.Runtime(0, sync_each_op=True)
    yield r
    r.close()


def _rand(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def test_arithmetic_like_reference_unit_tests(rt, ora):
    dims = [2, 3, 4, 5, 6]   # tests/unittest_arithmetic.cpp
    a, b = _rand(720, 60), _rand(720, 61)
    for typ in (ora.ADD, ora.SUB, ora.MUL, ora.DIV):
        got, od = rt.op("arithmetic", [(a, dims), (b, dims)], [typ])
        assert od == dims
        assert_bits_equal(got, ora.arithmetic(typ, a, b), "arithmetic %d" % typ)
        for side in (0, 1):
            got, _ = rt.op("arithmetic_const", [(a, dims)], [typ, 3.291, side])
            assert_bits_equal(got, ora.arithmetic_const(typ, side, 3.291, a), "const")
    for typ in (ora.EXP, ora.NEG):
        got, _ = rt.op("elewise", [(a, dims)], [typ])
        assert normwise(got, ora.elewise(typ, a)) <= TOL
    got, _ = rt.op("elewise", [(np.abs(a) + 500, dims)], [ora.LN])
    assert normwise(got, ora.elewise(ora.LN, np.abs(a) + np.float32(500))) <= TOL


def test_norm_arithmetic_and_reductions(rt, ora):
    x = _rand(63, 62)
    row, col = _rand(7, 63), _rand(9, 64)
    got, _ = rt.op("norm_arithmetic", [(x, [9, 7]), (row, [1, 7])], [ora.ADD])
    assert_bits_equal(got, ora.norm_arithmetic(ora.ADD, x, [9, 7], row, [0]), "{9,7}+{1,7}")
    got, _ = rt.op("norm_arithmetic", [(x, [9, 7]), (col, [9, 1])], [ora.MUL])
    assert_bits_equal(got, ora.norm_arithmetic(ora.MUL, x, [9, 7], col, [1]), "{9,7}*{9,1}")
    iota = np.arange(15, dtype=np.float32)
    for typ, dim, want in ((ora.MAX, 0, [4, 9, 14]), (ora.MAX, 1, [10, 11, 12, 13, 14]),
                           (ora.SUM, 0, [10, 35, 60]), (ora.SUM, 1, [15, 18, 21, 24, 27])):
        got, od = rt.op("reduction", [(iota, [5, 3])], [typ, dim])
        np.testing.assert_array_equal(got, want)
        assert od == ([1, 3] if dim == 0 else [5, 1])
    got, od = rt.op("maxindex", [(iota, [5, 3])], [0])
    np.testing.assert_array_equal(got, [4, 4, 4])
    # higher rank, first and last dimension (the CPU implementation is N-d)
    y = _rand(4 * 3 * 5, 65)
    for dim in (0, 2):
        got, _ = rt.op("reduction", [(y, [4, 3, 5])], [ora.MAX, dim])
        assert_bits_equal(got, ora.reduction(ora.MAX, y, [4, 3, 5], [dim]), "3-d max")
        got, _ = rt.op("maxindex", [(y, [4, 3, 5])], [dim])
        assert_bits_equal(got, ora.maxindex(y, [4, 3, 5], dim), "3-d maxindex")
    v = _rand(15, 66)
    got, _ = rt.op("norm_arithmetic", [(y, [4, 3, 5]), (v, [1, 3, 5])], [ora.SUB])
    assert_bits_equal(got, ora.norm_arithmetic(ora.SUB, y, [4, 3, 5], v, [0]), "3-d norm")


def test_matmult_transpose_reshape(rt, ora):
    a, b = _rand(6, 67), _rand(10, 68)   # tests/unittest_sgemm.cpp: {3,2} x {2,5}
    got, od = rt.op("matmult", [(a, [3, 2]), (b, [2, 5])])
    assert od == [3, 5]
    assert normwise(got, ora.matmult(a, b, 3, 5, 2)) <= TOL
    x = _rand(35, 69)
    got, od = rt.op("trans", [(x, [5, 7])])
    assert od == [7, 5]
    assert_bits_equal(got, ora.transpose(x, 7, 5), "trans")
    got, od = rt.op("reshape", [(x, [5, 7])], [7, 5, 1])
    assert od == [7, 5, 1]
    assert_bits_equal(got, x, "reshape")


def test_activations_and_softmax(rt, ora):
    dims = [7, 6, 3, 2]  # tests/unittest_activation.cpp
    x, dy = _rand(252, 70), _rand(252, 71)
    names = {ora.SIGMOID: "sigmoid", ora.RELU: "relu", ora.TANH: "tanh"}
    for alg, nm in names.items():
        y_ref = ora.activation_fwd(alg, x)
        got, _ = rt.op(nm + "_forward", [(x, dims)])
        got2, _ = rt.op("activation_forward", [(x, dims)], [alg])
        assert_bits_equal(got, got2, "Elewise:: and Convolution:: entry points agree")
        assert normwise(got, y_ref) <= TOL
        back, _ = rt.op(nm + "_backward", [(dy, dims), (y_ref, dims), (x, dims)])
        back2, _ = rt.op("activation_backward", [(dy, dims), (y_ref, dims), (x, dims)], [alg])
        assert_bits_equal(back, back2, "backward entry points agree")
        assert normwise(back, ora.activation_bwd(alg, dy, y_ref, x)) <= TOL
    z = _rand(10 * 256, 72) * 3
    y, od = rt.op("softmax_forward", [(z, [10, 1, 1, 256])], [0])
    ref = ora.softmax_instance_fwd(z, 256, 10, 1, 1)
    assert normwise(y, ref) <= TOL
    d, _ = rt.op("softmax_backward", [(_rand(2560, 73), [10, 1, 1, 256]), (ref, [10, 1, 1, 256])], [0])
    assert normwise(d, ora.softmax_instance_bwd(_rand(2560, 73), ref, 256, 10, 1, 1)) <= TOL
    c, _ = rt.op("softmax_forward", [(z[:120], [4, 3, 5, 2])], [1])
    assert normwise(c, ora.softmax_channel_fwd(z[:120], 2, 5, 3, 4)) <= TOL


def test_convolution_golden_and_gradients(rt, ora):
    for case in json.load(open(os.path.join(GOLD, "conv_forward.json"))):
        W, H, C, N = case["input_size"]
        S, R, _, K = case["weight_size"]
        x = np.array(case["input"], np.float32)
        w = np.array(case["weight"], np.float32)
        b = np.array(case["bias"] or [0] * K, np.float32)
        info = [case["pad_height"], case["pad_width"], case["stride_vertical"],
                case["stride_horizontal"]]
        got, od = rt.op("conv_forward", [(x, case["input_size"]), (w, case["weight_size"]), (b, [K])],
                        info)
        assert od == case["correct_size"]
        idx = np.arange(got.size)
        want = np.array(case["correct_without_bias"], np.float32) + b[(idx // 16) % K]
        assert np.max(np.abs(got - want)) < 1e-3
        p = (N, C, K, H, W, *info, R, S)
        dy = _rand(got.size, 74)
        gd, od = rt.op("conv_backward_data", [(dy, od), (x, case["input_size"]), (w, case["weight_size"])], info)
        assert od == case["input_size"]
        assert normwise(gd, ora.conv_bwd_data(dy, w, *p)) <= TOL
        gf, od = rt.op("conv_backward_filter", [(dy, case["correct_size"]), (x, case["input_size"]),
                                                (w, case["weight_size"])], info)
        assert od == case["weight_size"]
        assert normwise(gf, ora.conv_bwd_filter(dy, x, *p)) <= TOL
        gb, od = rt.op("conv_backward_bias", [(dy, case["correct_size"])])
        assert od == [K]
        assert normwise(gb, ora.conv_bwd_bias(dy, N, K, case["correct_size"][1], case["correct_size"][0])) <= TOL


def test_pooling_golden_and_gradient(rt, ora):
    for case in json.load(open(os.path.join(GOLD, "pooling_forward.json"))):
        x = np.array(case["input"], np.float32)
        prm = [0, case["height"], case["width"], case["stride_vertical"], case["stride_horizontal"],
               case["pad_height"], case["pad_width"]]
        got, od = rt.op("pooling_forward", [(x, case["input_size"])], prm)
        assert od == case["correct_size"]          # EXPECT_EQ(output.Size(), correct_size)
        np.testing.assert_array_equal(got, np.array(case["correct"], np.float32))
        dy = _rand(got.size, 75)
        back, od = rt.op("pooling_backward", [(dy, od), (got, od), (x, case["input_size"])], prm)
        assert od == case["input_size"]
        W, H, C, N = case["input_size"]
        ref = ora.pool_bwd(ora.POOL_MAX, dy, got, x, N, C, H, W, *prm[3:5], *prm[1:3], *prm[5:7])
        assert_bits_equal(back, ref, "pool bwd")


def test_lrn_forward_and_backward(rt, ora):
    W, H, C, N = 6, 5, 12, 3
    size = [W, H, C, N]
    x = _rand(W * H * C * N, 76) * 3
    prm = [5, 1e-2, 0.75]
    top, scale = ora.lrn_fwd(x, 5, 1e-2, 0.75, N, C, H, W)
    got, od = rt.op("lrn_forward", [(x, size), (np.zeros_like(x), size)], prm)
    assert od == size
    assert normwise(got, top) <= TOL
    dy = _rand(x.size, 77)
    back, od = rt.op("lrn_backward", [(x, size), (top, size), (scale, size), (dy, size)], prm)
    assert od == size
    assert normwise(back, ora.lrn_bwd(x, top, scale, dy, 5, 1e-2, 0.75, N, C, H, W)) <= TOL


def test_concat_slice_select(rt, ora):
    # channel concat of image batches {W,H,C,N}, the reference's main use (cuda.cpp:97-118)
    a, b, c = _rand(5 * 4 * 3 * 2, 80), _rand(5 * 4 * 6 * 2, 81), _rand(5 * 4 * 1 * 2, 82)
    da, db, dc = [5, 4, 3, 2], [5, 4, 6, 2], [5, 4, 1, 2]
    got, od = rt.op("concat", [(a, da), (b, db), (c, dc)], [2])
    assert od == [5, 4, 10, 2]
    assert_bits_equal(got, ora.concat([a, b, c], [da, db, dc], 2), "concat channels")
    # along the last dimension (plain append) and along dimension 0 (not in the reference)
    got, od = rt.op("concat", [(a, da), (a, da)], [3])
    assert od == [5, 4, 3, 4]
    assert_bits_equal(got, ora.concat([a, a], [da, da], 3), "concat images")
    m1, m2 = _rand(6, 83), _rand(9, 84)
    got, od = rt.op("concat", [(m1, [2, 3]), (m2, [3, 3])], [0])
    assert od == [5, 3]
    assert_bits_equal(got, ora.concat([m1, m2], [[2, 3], [3, 3]], 0), "concat rows")
    # slices undo the concat
    cat = ora.concat([a, b, c], [da, db, dc], 2)
    got, od = rt.op("slice", [(cat, [5, 4, 10, 2])], [2, 3, 6])
    assert od == db
    assert_bits_equal(got, b, "slice channels")
    got, od = rt.op("slice", [(cat, [5, 4, 10, 2])], [3, 1, 1])
    assert od == [5, 4, 10, 1]
    assert_bits_equal(got, ora.slice_(cat, [5, 4, 10, 2], 3, 1, 1), "slice images")
    got, od = rt.op("select", [(m2, [3, 3])], [2, 0, 2])
    assert od == [3, 3]
    assert_bits_equal(got, ora.select(m2, 3, 3, [2, 0, 2]), "select")
    from minerva_amd import hostapi
    with pytest.raises(hostapi.HostError, match="extent mismatch"):
        rt.op("concat", [(a, da), (_rand(4 * 4 * 3 * 2, 85), [4, 4, 3, 2])], [2])
    with pytest.raises(hostapi.HostError, match="range outside"):
        rt.op("slice", [(a, da)], [2, 2, 2])
    with pytest.raises(hostapi.HostError, match="out of range"):
        rt.op("select", [(m2, [3, 3])], [3])


def test_threshold_norm_and_index(rt, ora):
    x = _rand(24, 86) * 2
    got, od = rt.op("threshold_norm", [(x, [4, 6])], [0.5])
    assert od == [4, 6]
    assert_bits_equal(got, ora.threshold_norm(x, 0.5), "threshold norm")
    got, od = rt.op("index", [(x, [4, 6])], [2, 4, 2])      # third {4,2} block
    assert od == [4, 2]
    assert_bits_equal(got, x[16:24], "index")
    from minerva_amd import hostapi
    with pytest.raises(hostapi.HostError, match="outside the input"):
        rt.op("index", [(x, [4, 6])], [3, 4, 2])


def test_random_operators(rt, ora):
    from minerva_amd import hostapi
    hostapi.Runtime.set_random_seed(5)
    a, od = rt.op("randn", [], [0.0, 0.01, 64, 33], out_capacity=64 * 33)
    b, _ = rt.op("randn", [], [0.0, 0.01, 64, 33], out_capacity=64 * 33)
    assert od == [64, 33]
    assert abs(a.mean()) < 1e-3 and abs(a.std() - 0.01) < 1e-3      # the "var" field is the deviation
    assert not np.array_equal(a, b)                                  # successive calls differ
    hostapi.Runtime.set_random_seed(5)
    a2, _ = rt.op("randn", [], [0.0, 0.01, 64, 33], out_capacity=64 * 33)
    assert_bits_equal(a2, a, "same seed sequence, same tensor")
    m, _ = rt.op("rand_bernoulli", [], [0.25, 100, 100], out_capacity=10000)
    assert set(np.unique(m)) <= {0.0, 1.0} and abs(m.mean() - 0.25) < 0.02
    with pytest.raises(hostapi.HostError, match="probability out of range"):
        rt.op("rand_bernoulli", [], [1.5, 4], out_capacity=4)


def test_error_convention(rt):
    from minerva_amd import hostapi
    a = _rand(6, 76)
    with pytest.raises(hostapi.HostError, match="size must match"):
        rt.op("arithmetic", [(a, [2, 3]), (a, [3, 2])], [0])
    with pytest.raises(hostapi.HostError, match="size must match"):
        rt.op("matmult", [(a, [2, 3]), (a, [2, 3])])
    with pytest.raises(hostapi.HostError, match="cannot replicate"):
        rt.op("norm_arithmetic", [(a, [2, 3]), (a[:4], [2, 2])], [0])
    with pytest.raises(hostapi.HostError, match="first or the last"):
        rt.op("reduction", [(_rand(24, 77), [2, 3, 4])], [0, 1])
    with pytest.raises(hostapi.HostError, match="channels mismatch"):
        rt.op("conv_forward", [(_rand(36, 78), [3, 3, 2, 2]), (a[:4], [2, 2, 1, 1]), (a[:1], [1])],
              [0, 0, 1, 1])
    with pytest.raises(hostapi.HostError, match="unknown operator"):
        rt.op("no_such_operator", [(a, [6])])
    # the runtime is still usable after a failed check
    got, _ = rt.op("arithmetic", [(a, [6]), (a, [6])], [0])
    assert_bits_equal(got, a + a, "after error")


def test_device_manager_creates_the_device_and_refuses_a_missing_gpu():
    # device_manager.cpp:33-47: devices are made by GPU index and live in the manager; the
    # runtime's device comes from there
    from minerva_amd import hostapi
    with pytest.raises(hostapi.HostError, match="no GPU #99"):
        hostapi.Runtime(99)
    r = hostapi.Runtime(0)
    a = _rand(12, 79)
    got, _ = r.op("arithmetic", [(a, [3, 4]), (a, [3, 4])], [2])
    assert_bits_equal(got, a * a, "product on the managed device")
    r.close()


def test_pooled_allocator_reuses_exact_sizes(rt):
    a = _rand(5000, 79)
    rt.op("arithmetic", [(a, [5000]), (a, [5000])], [0])
    total0, cached0 = rt.pool_stats()
    for _ in range(5):
        rt.op("arithmetic", [(a, [5000]), (a, [5000])], [0])
    total1, cached1 = rt.pool_stats()
    assert total1 == total0, "same-size requests must be served from the free lists"
    assert cached1 >= 3  # two inputs and one output went back to the pool


def test_four_stream_thread_pool(rt):
    a, b = _rand(100003, 80), _rand(100003, 81)
    out = rt.concurrent_adds(a, b, 24)
    for i in range(24):
        assert_bits_equal(out[i], a + b, "concurrent add %d" % i)


@pytest.mark.parametrize("mode", ["stream_order", "dataflow"])
def test_thread_pool_tasks_without_per_operator_sync(mode):
    """Tasks of the thread pool run on whichever worker stream takes them.  With the
    per-operator synchronisation switched off they must still be complete (stream order:
    each worker drains its stream; dataflow: the reader waits for all streams) before the
    results are copied back on stream 0."""
    from minerva_amd import hostapi
    r = hostapi.Runtime(0, sync_each_op=False, dataflow=(mode == "dataflow"))
    a, b = _rand(3000003, 82), _rand(3000003, 83)
    for _ in range(3):
        out = r.concurrent_adds(a, b, 16)
        for i in range(16):
            assert_bits_equal(out[i], a + b, "concurrent add %d (%s)" % (i, mode))
    r.close()


def _run_net(kind, batch, steps, sync_each_op, variant=0, lr=0.01, keep_acts=False):
    from minerva_amd import hostapi
    from oracle import nets
    params, data, label = nets.make_inputs(kind, batch)
    r = hostapi.Runtime(0, sync_each_op=sync_each_op)
    net = hostapi.Net(r, kind, batch, variant)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(data, label)
    if keep_acts:
        net.keep_activations()
    for _ in range(steps):
        net.step(lr)
    r.sync()
    out = {k: net.read(k, n) for k, n in net.params.items()}
    if keep_acts:
        out["acts"] = {i: net.read("act%d" % i, n * batch) for i, n in ALEX_ACT_ELEMS.items()}
    out.update({"g_" + k: net.read("g_" + k, n) for k, n in net.params.items()})
    out["prob"] = net.read("prob", label.size)
    ops = r.ops_issued()
    net.close()
    r.close()
    return out, ops


def test_mlp_step_matches_oracle(ora):
    from oracle import nets
    params, data, label = nets.make_inputs("mlp", 256)
    p = dict(params)
    for _ in range(2):
        p, res = nets.mlp_step(p, data, label, 0.01, 256)
    say("mlp 2 steps, per-op sync")
    got, ops = _run_net("mlp", 256, 2, True)
    compare_step(got, p, res)
    say("mlp 2 steps, one sync per step")
    got2, _ = _run_net("mlp", 256, 2, False)
    for k in got:
        assert_bits_equal(got[k], got2[k], "sync mode must not change " + k)
    assert ops >= 2 * 25


@pytest.mark.parametrize("variant", [0, 1])
def test_cnn_step_matches_oracle(ora, variant):
    from oracle import nets
    batch = 16
    params, data, label = nets.make_inputs("cnn", batch)
    kw = dict(pad2=2, pool2=3) if variant else {}
    p, res = nets.cnn_step(dict(params), data, label, 0.01, batch, **kw)
    say("cnn step variant", variant)
    got, _ = _run_net("cnn", batch, 1, True, variant)
    compare_step(got, p, res)


@pytest.mark.parametrize("variant", [0, 1])
def test_cnn_step_batch_256_matches_oracle(ora, variant):
    """The kernel plans of the benchmark's batch: 128x32 tiles and filter gradients cut into
    hundreds of k ranges are chosen from the batch, so the step is compared at 256 too."""
    from oracle import nets
    batch = 256
    params, data, label = nets.make_inputs("cnn", batch)
    kw = dict(pad2=2, pool2=3) if variant else {}
    p, res = nets.cnn_step(dict(params), data, label, 0.01, batch, **kw)
    say("cnn step b=256 variant", variant)
    got, _ = _run_net("cnn", batch, 1, False, variant)
    compare_step(got, p, res)


_ALEX2 = {}


def _alexnet_oracle_b2():
    """One oracle step at batch 2 with every activation and sensitivity kept (CPU, ~5 s),
    shared by the tests below."""
    if not _ALEX2:
        from oracle import nets
        params, data, label = nets.make_inputs("alexnet", 2)
        say("alexnet oracle step b=2 (CPU)")
        p, res = nets.alexnet_step(dict(params), data, label, 0.01, 2, keep=True)
        _ALEX2.update(params=params, data=data, label=label, newp=p, res=res)
    return _ALEX2


def test_alexnet_step_matches_oracle_small_batch(ora):
    batch = 2
    o = _alexnet_oracle_b2()
    params, data, label, res = o["params"], o["data"], o["label"], o["res"]
    say("alexnet GPU step b=2")
    got, ops = _run_net("alexnet", batch, 1, False, keep_acts=True)
    compare_alexnet_step(got, got["acts"], params, data, label, batch, 0.01, res["acts"], res["prob"])
    # the loss itself (cross entropy of the probabilities) agrees to 1e-5
    lab = label.reshape(batch, -1).argmax(axis=1)
    ce = lambda pr: -np.log(pr.reshape(batch, -1)[np.arange(batch), lab].astype(np.float64)).mean()
    assert abs(ce(got["prob"]) - ce(res["prob"])) <= 1e-5 * abs(ce(res["prob"]))
    assert ops > 80


def test_alexnet_backward_on_oracle_activations(ora):
    """Why the whole-step comparison above needs its looser gradient bounds: the only
    discontinuous operators of the step are the ReLU gates and the arg-max routing of the
    pooling gradients.  Here the backward pass runs on the GPU from the ORACLE's forward
    activations, so both sides open the same gates and route to the same maxima, and every
    sensitivity and every gradient then agrees with the oracle normwise to 1e-4."""
    from minerva_amd import hostapi
    from oracle import nets
    N = 2
    o = _alexnet_oracle_b2()
    params, label, res = o["params"], o["label"], o["res"]
    acts, sens = res["acts"], res["sens"]
    shapes = nets.alexnet_param_shapes()
    act_dims = {0: [227, 227, 3, N], 1: [55, 55, 96, N], 2: [27, 27, 96, N], 3: [27, 27, 256, N],
                4: [13, 13, 256, N], 5: [13, 13, 384, N], 6: [13, 13, 384, N], 7: [13, 13, 256, N],
                8: [6, 6, 256, N], 9: [4096, N], 10: [4096, N]}
    r = hostapi.Runtime(0, sync_each_op=False)
    A = {i: r.tensor(acts[i], d) for i, d in act_dims.items()}
    W = {k: r.tensor(v, shapes[k]) for k, v in params.items() if k.startswith("w")}
    conv = {i: list(nets.ALEX_CONVS[i][4:8]) for i in range(5)}   # ph, pw, sv, sh
    pool = [0, 3, 3, 2, 2, 0, 0]
    say("alexnet backward chain on oracle activations (GPU)")
    S = {11: r.tensor(sens[11], [1000, N])}
    relu_bwd = lambda d, a: r.top("relu_backward", [d, a, a])
    S[10] = relu_bwd(r.top("matmult", [r.top("trans", [W["w7"]]), S[11]]), A[10])
    S[9] = relu_bwd(r.top("matmult", [r.top("trans", [W["w6"]]), S[10]]), A[9])
    S[8] = r.top("reshape", [r.top("matmult", [r.top("trans", [W["w5"]]), S[9]])], act_dims[8])
    S[7] = relu_bwd(r.top("pooling_backward", [S[8], A[8], A[7]], pool), A[7])
    S[6] = relu_bwd(r.top("conv_backward_data", [S[7], A[6], W["w4"]], conv[4]), A[6])
    S[5] = relu_bwd(r.top("conv_backward_data", [S[6], A[5], W["w3"]], conv[3]), A[5])
    S[4] = r.top("conv_backward_data", [S[5], A[4], W["w2"]], conv[2])
    S[3] = relu_bwd(r.top("pooling_backward", [S[4], A[4], A[3]], pool), A[3])
    S[2] = r.top("conv_backward_data", [S[3], A[2], W["w1"]], conv[1])
    S[1] = relu_bwd(r.top("pooling_backward", [S[2], A[2], A[1]], pool), A[1])
    A8 = r.top("reshape", [A[8]], [9216, N])
    G = {"w7": r.top("matmult", [S[11], r.top("trans", [A[10]])]),
         "w6": r.top("matmult", [S[10], r.top("trans", [A[9]])]),
         "w5": r.top("matmult", [S[9], r.top("trans", [A8])]),
         "b7": r.top("reduction", [S[11]], [0, 1]), "b6": r.top("reduction", [S[10]], [0, 1]),
         "b5": r.top("reduction", [S[9]], [0, 1])}
    for i, s_idx, a_idx in ((4, 7, 6), (3, 6, 5), (2, 5, 4), (1, 3, 2), (0, 1, 0)):
        G["w%d" % i] = r.top("conv_backward_filter", [S[s_idx], A[a_idx], W["w%d" % i]], conv[i])
        G["b%d" % i] = r.top("conv_backward_bias", [S[s_idx]])
    r.sync()
    worst = {}
    for i in range(1, 11):
        worst["sens%d" % i] = normwise(S[i].read(), sens[i])
    for k, t in G.items():
        worst["g_" + k] = normwise(t.read(), res["g_" + k])
    r.close()
    say("same-gates backward: worst normwise error %.2e (%s)"
        % (max(worst.values()), max(worst, key=worst.get)))
    bad = {k: v for k, v in worst.items() if not v <= TOL}
    assert not bad, bad


def test_alexnet_forward_batch_256_prefix_matches_oracle(ora):
    """The benchmark's own shape: one step at batch 256, and the probabilities of its first
    four images against the oracle's forward pass at batch 4 on the same parameters and
    images (the forward pass treats images independently, so the prefix is an exact check
    of the batch-256 kernel plans: conv1..conv5 tiles, pooling groups, FC split counts)."""
    from minerva_amd import hostapi
    from oracle import nets
    B, nb = 256, 4
    params, data, label = nets.make_inputs("alexnet", B)
    per = 3 * 227 * 227
    say("alexnet oracle forward b=4 (CPU)")
    _, want = nets.alexnet_forward(params, np.ascontiguousarray(data[:nb * per]), nb)
    say("alexnet GPU step b=256")
    r = hostapi.Runtime(0, sync_each_op=False)
    net = hostapi.Net(r, "alexnet", B)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(data, label)
    net.step(0.01)
    r.sync()
    prob = net.read("prob", 1000 * B)
    gb7 = net.read("g_b7", 1000)
    gw7 = net.read("g_w7", 1000 * 4096)
    w7 = net.read("w7", 1000 * 4096)
    net.close()
    r.close()
    assert normwise(prob[:nb * 1000], want) <= TOL
    P = prob.reshape(B, 1000).astype(np.float64)
    assert np.max(np.abs(P.sum(axis=1) - 1.0)) <= 1e-5
    # what the rest of the step lets the host check exactly: the last layer's bias gradient is
    # the column sum of (prob - label), and the update is w - lr/B * g in fp32
    s11 = prob.reshape(B, 1000) - label.reshape(B, 1000)
    assert normwise(gb7, s11.astype(np.float64).sum(axis=0)) <= TOL
    step = (np.float32(0.01) / np.float32(B)) * gw7
    assert_bits_equal(w7, params["w7"] - step, "SGD update of w7 at b=256")


def test_alexnet_gradients_batch_256_against_oracle_on_a_replicated_batch(ora):
    """The backward pass at the benchmark's batch size, which the oracle cannot walk in
    reasonable time: a batch of 64 copies of four images.  Weight and bias gradients are sums
    over the images, so they must be 64 times the oracle's gradients for the four images
    (the oracle's backward pass evaluated at the GPU's activations of the first copy: same
    ReLU gates and pooling routes).  This runs every batch-256 kernel plan of the backward
    pass (k ranges of the filter gradients, cut tails of the data gradients, grouped
    workgroups of the inner products) against the oracle."""
    from minerva_amd import hostapi
    from oracle import nets
    B, nb = 256, 4
    params, data4, label4 = nets.make_inputs("alexnet", nb)
    data = np.tile(data4, B // nb)
    label = np.tile(label4, B // nb)
    say("alexnet GPU step b=256 on 64 copies of 4 images")
    r = hostapi.Runtime(0, sync_each_op=False)
    net = hostapi.Net(r, "alexnet", B)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(data, label)
    net.keep_activations()
    net.step(0.01)
    r.sync()
    prob = net.read("prob", 1000 * B)
    acts = {i: net.read("act%d" % i, n * B) for i, n in ALEX_ACT_ELEMS.items()}
    got = {k: net.read("g_" + k, n) for k, n in net.params.items()}
    net.close()
    r.close()
    # every copy of an image must give the same probabilities (to rounding: copies that fall
    # into differently cut tiles are summed in a different order)
    P = prob.reshape(B // nb, nb * 1000)
    assert normwise(P, np.broadcast_to(P[0], P.shape)) <= 1e-5
    acts4 = [data4] + [acts[i][:n * nb] for i, n in sorted(ALEX_ACT_ELEMS.items())] + [None]
    say("alexnet oracle backward b=4 at the GPU's activations (CPU)")
    g4, _, _ = nets.alexnet_backward(params, acts4, np.ascontiguousarray(prob[:nb * 1000]), label4, nb)
    worst = {k: normwise(got[k], np.float32(B // nb) * g4[k].astype(np.float64)) for k in sorted(params)}
    say("  worst normwise error %.2e (%s)" % (max(worst.values()), max(worst, key=worst.get)))
    bad = {k: v for k, v in worst.items() if not v <= TOL}
    assert not bad, bad


def test_alexnet_step_with_dropout_matches_oracle(ora):
    """The reference application's graph including drop6 / drop7: the masks come from the
    library's generator, which the oracle reproduces bit for bit from the seed sequence."""
    from minerva_amd import hostapi
    from oracle import nets
    batch, seed = 2, 20240607
    o = _alexnet_oracle_b2()
    params, data, label = o["params"], o["data"], o["label"]
    masks = nets.dropout_masks(batch, 0.5, seed)
    say("alexnet + dropout oracle forward b=2 (CPU)")
    acts, prob = nets.alexnet_forward(params, data, batch, masks=masks)
    say("alexnet + dropout GPU step b=2")
    hostapi.Runtime.set_random_seed(seed)
    got, ops = _run_net("alexnet", batch, 1, False, variant=1, keep_acts=True)
    compare_alexnet_step(got, got["acts"], params, data, label, batch, 0.01, acts, prob, masks=masks)
    plain = o["res"]
    # dropout changed the result: the plain graph's probabilities differ
    assert normwise(got["prob"], plain["prob"]) > 1e-3 or np.max(np.abs(got["g_w7"] - plain["g_w7"])) > 0
