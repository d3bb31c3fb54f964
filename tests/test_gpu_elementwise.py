"""GPU parity of the HBM-streaming ops against the CPU oracle, through the C ABI.
Bit-exact: add/sub/mul/div, scalar ops, neg, relu forward/backward, fill, copy,
broadcast add/sub/mul/div.  Normwise <= 1e-4: exp, ln, sigmoid, tanh and the sigmoid /
tanh gradients."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, TOL, assert_bits_equal, normwise, say

pytestmark = pytest.mark.gpu

SIZES = [1, 3, 4, 255, 1024, 4097, 1 << 20, (1 << 20) + 3]


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


def _rand(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


@pytest.mark.parametrize("n", SIZES)
def test_binary_ops_bit_exact(gpu, ora, n):
    a, b = _rand(n, 1), _rand(n, 2)
    b[b == 0] = 1
    da, db, dc = gpu.up(a), gpu.up(b), gpu.empty(n)
    for name, typ in (("mnv_add", ora.ADD), ("mnv_sub", ora.SUB), ("mnv_mul", ora.MUL),
                      ("mnv_div", ora.DIV)):
        say(name, n)
        gpu.call(name, da.p, db.p, dc.p, n)
        assert_bits_equal(gpu.down(dc), ora.arithmetic(typ, a, b), name)


def test_binary_ops_unaligned_pointers(gpu, ora):
    n = 10001
    a, b = _rand(n + 1, 3), _rand(n + 1, 4)
    da, db, dc = gpu.up(a), gpu.up(b), gpu.empty(n + 1)
    gpu.call("mnv_add", da.offset(1), db.offset(1), dc.offset(1), n)
    assert_bits_equal(gpu.down(dc)[1:], ora.arithmetic(ora.ADD, a[1:], b[1:]), "add+1")


def test_binary_ops_special_values(gpu, ora):
    sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, 1.17e-38, 1, -1],
                  np.float32)
    a = np.repeat(sp, sp.size)
    b = np.tile(sp, sp.size)
    da, db, dc = gpu.up(a), gpu.up(b), gpu.empty(a.size)
    for name, typ in (("mnv_add", ora.ADD), ("mnv_sub", ora.SUB), ("mnv_mul", ora.MUL),
                      ("mnv_div", ora.DIV)):
        gpu.call(name, da.p, db.p, dc.p, a.size)
        assert_bits_equal(gpu.down(dc), ora.arithmetic(typ, a, b), name + " specials")


def test_binary_full_size_8192x8192(gpu, ora):
    n = 8192 * 8192
    a, b = _rand(n, 5), _rand(n, 6)
    da, db, dc = gpu.up(a), gpu.up(b), gpu.empty(n)
    for name, typ in (("mnv_add", ora.ADD), ("mnv_mul", ora.MUL), ("mnv_sub", ora.SUB)):
        say(name, "8192x8192")
        gpu.call(name, da.p, db.p, dc.p, n)
        assert_bits_equal(gpu.down(dc), ora.arithmetic(typ, a, b), name)


@pytest.mark.parametrize("n", [1, 5, 4099, 1 << 18])
def test_scalar_ops_bit_exact(gpu, ora, n):
    x = _rand(n, 7)
    x[x == 0] = 2
    v = 3.291  # tests/unittest_arithmetic_const.cpp:75
    dx, dy = gpu.up(x), gpu.empty(n)
    table = [("mnv_const_add", ora.ADD, 1), ("mnv_const_sub", ora.SUB, 1),
             ("mnv_const_rsub", ora.SUB, 0), ("mnv_const_mul", ora.MUL, 1),
             ("mnv_const_div", ora.DIV, 1), ("mnv_const_rdiv", ora.DIV, 0)]
    for name, typ, side in table:
        say(name, n)
        gpu.call(name, dx.p, dy.p, ctypes.c_float(v), n)
        assert_bits_equal(gpu.down(dy), ora.arithmetic_const(typ, side, v, x), name)


def test_left_const_chain(gpu, ora):
    # tests/unittest_leftconst.cpp:7-49: chained (c - x)
    x = _rand(720, 8)
    dx, d1, d2 = gpu.up(x), gpu.empty(720), gpu.empty(720)
    gpu.call("mnv_const_rsub", dx.p, d1.p, ctypes.c_float(2.5), 720)
    gpu.call("mnv_const_rsub", d1.p, d2.p, ctypes.c_float(-1.25), 720)
    want = ora.arithmetic_const(ora.SUB, 0, -1.25, ora.arithmetic_const(ora.SUB, 0, 2.5, x))
    assert_bits_equal(gpu.down(d2), want, "left const chain")


@pytest.mark.parametrize("n", [1, 7, 4098, 1 << 20])
def test_unary_ops(gpu, ora, n):
    x = _rand(n, 9, 3.0)
    dx, dy = gpu.up(x), gpu.empty(n)
    gpu.call("mnv_neg", dx.p, dy.p, n)
    assert_bits_equal(gpu.down(dy), ora.elewise(ora.NEG, x), "neg")
    gpu.call("mnv_exp", dx.p, dy.p, n)
    got, ref = gpu.down(dy), ora.elewise(ora.EXP, x)
    assert np.max(np.abs(got / ref - 1)) <= TOL  # elementwise relative, stricter than normwise
    pos = np.abs(x) + np.float32(500)  # tests/unittest_elewise.cpp: ln on N(500,1)
    dp = gpu.up(pos)
    gpu.call("mnv_ln", dp.p, dy.p, n)
    assert normwise(gpu.down(dy), ora.elewise(ora.LN, pos)) <= TOL
    gpu.call("mnv_copy", dx.p, dy.p, n)
    assert_bits_equal(gpu.down(dy), x, "copy")
    gpu.call("mnv_fill", dy.p, n, ctypes.c_float(-1.5))
    assert_bits_equal(gpu.down(dy), np.full(n, -1.5, np.float32), "fill")


@pytest.mark.parametrize("n", [1, 6, 7 * 6 * 3 * 2, 4099, 1 << 20])
def test_activation_forward(gpu, ora, n):
    x = _rand(n, 10, 2.0)
    if n >= 6:
        x[:6] = [0.0, -0.0, np.nan, -1.0, 1.0, 1e-30]
    dx, dy = gpu.up(x), gpu.empty(n)
    gpu.call("mnv_relu_fwd", dx.p, dy.p, n)
    assert_bits_equal(gpu.down(dy), ora.activation_fwd(ora.RELU, x), "relu")
    x = np.nan_to_num(x)
    dx = gpu.up(x)
    gpu.call("mnv_sigmoid_fwd", dx.p, dy.p, n)
    assert normwise(gpu.down(dy), ora.activation_fwd(ora.SIGMOID, x)) <= TOL
    gpu.call("mnv_tanh_fwd", dx.p, dy.p, n)
    assert normwise(gpu.down(dy), ora.activation_fwd(ora.TANH, x)) <= TOL


@pytest.mark.parametrize("n", [1, 5, 4099, 1 << 20])
def test_activation_backward(gpu, ora, n):
    x = _rand(n, 11, 2.0)
    if n >= 5:
        x[:5] = [0.0, -0.0, -2.0, 2.0, 1e-30]
    dy = _rand(n, 12)
    dxb, ddy, dout = gpu.up(x), gpu.up(dy), gpu.empty(n)
    for name, alg in (("mnv_relu_bwd", ora.RELU), ("mnv_sigmoid_bwd", ora.SIGMOID),
                      ("mnv_tanh_bwd", ora.TANH)):
        y = ora.activation_fwd(alg, x)
        dyt = gpu.up(y)
        say(name, n)
        gpu.call(name, dxb.p, dyt.p, ddy.p, dout.p, n)
        ref = ora.activation_bwd(alg, dy, y, x)
        if alg == ora.RELU:
            assert_bits_equal(gpu.down(dout), ref, name)
        else:
            assert normwise(gpu.down(dout), ref) <= TOL


def test_non_temporal_instantiations_8192x8192(gpu, ora):
    """Calls whose traffic reaches 512 MB run the non-temporal instantiations of the streaming
    kernels: at 8192 x 8192 that is every one-input operator and every activation gradient of
    the bandwidth benchmark, and the cached softmax gradient on lines of 8192.  Each is
    compared with the oracle at that size (selections and single IEEE operations bit for bit)."""
    m = n_lines = 8192
    n = m * n_lines
    x = _rand(n, 16, 2.0)
    x[:6] = [0.0, -0.0, -2.0, 2.0, 1e-30, -1e-30]
    dy = _rand(n, 17)
    dx, ddy, dout = gpu.up(x), gpu.up(dy), gpu.empty(n)
    v = 3.291
    for name, args, ref in (
            ("mnv_const_mul", (ctypes.c_float(v),), lambda: ora.arithmetic_const(ora.MUL, 1, v, x)),
            ("mnv_const_div", (ctypes.c_float(v),), lambda: ora.arithmetic_const(ora.DIV, 1, v, x)),
            ("mnv_copy", (), lambda: x),
            ("mnv_neg", (), lambda: ora.elewise(ora.NEG, x)),
            ("mnv_relu_fwd", (), lambda: ora.activation_fwd(ora.RELU, x))):
        say(name, "8192x8192")
        gpu.call(name, dx.p, dout.p, *args, n)
        assert_bits_equal(gpu.down(dout), ref(), name + " 8192^2")
    say("mnv_div 8192x8192")
    den = dy.copy()
    den[den == 0] = 1
    dden = gpu.up(den)
    gpu.call("mnv_div", dx.p, dden.p, dout.p, n)
    assert_bits_equal(gpu.down(dout), ora.arithmetic(ora.DIV, x, den), "div 8192^2")
    del dden
    say("mnv_exp 8192x8192")
    gpu.call("mnv_exp", dx.p, dout.p, n)
    assert np.max(np.abs(gpu.down(dout) / ora.elewise(ora.EXP, x) - 1)) <= TOL
    tops = {}
    for name, alg in (("mnv_sigmoid_fwd", ora.SIGMOID), ("mnv_tanh_fwd", ora.TANH)):
        say(name, "8192x8192")
        gpu.call(name, dx.p, dout.p, n)
        tops[alg] = ora.activation_fwd(alg, x)
        assert normwise(gpu.down(dout), tops[alg]) <= TOL
    tops[ora.RELU] = ora.activation_fwd(ora.RELU, x)
    for name, alg in (("mnv_relu_bwd", ora.RELU), ("mnv_sigmoid_bwd", ora.SIGMOID),
                      ("mnv_tanh_bwd", ora.TANH)):
        say(name, "8192x8192")
        dtop = gpu.up(tops[alg])
        gpu.call(name, dx.p, dtop.p, ddy.p, dout.p, n)
        ref = ora.activation_bwd(alg, dy, tops[alg], x)
        if alg == ora.RELU:
            assert_bits_equal(gpu.down(dout), ref, name + " 8192^2")
        else:
            assert normwise(gpu.down(dout), ref) <= TOL
        del dtop
    say("softmax_instance_bwd 8192 lines of 8192")
    top = ora.softmax_instance_fwd(x, n_lines, m, 1, 1)
    dtop = gpu.up(top)
    gpu.call("mnv_softmax_instance_bwd", ddy.p, dtop.p, dout.p, n_lines, m, 1, 1)
    got = gpu.down(dout).reshape(n_lines, m)
    ref = ora.softmax_instance_bwd(dy, top, n_lines, m, 1, 1).reshape(n_lines, m)
    err = np.max(np.abs(got.astype(np.float64) - ref), axis=1) / np.max(np.abs(ref), axis=1)
    assert err.max() <= TOL, "softmax bwd: worst line %d, %.3e" % (int(err.argmax()), err.max())


NORM_SHAPES = [(9, 7), (1, 5), (5, 1), (1000, 33), (4096, 256), (8192, 64), (10, 256)]


@pytest.mark.parametrize("m,n", NORM_SHAPES)
def test_norm_arithmetic_bit_exact(gpu, ora, m, n):
    x = _rand(m * n, 13)
    row = _rand(n, 14)  # shape {1,n}: replicated along dim 0
    col = _rand(m, 15)  # shape {m,1}: replicated along dim 1
    row[row == 0] = 1
    col[col == 0] = 1
    dx, dr, dc, do = gpu.up(x), gpu.up(row), gpu.up(col), gpu.empty(m * n)
    for op, typ in (("add", ora.ADD), ("sub", ora.SUB), ("mul", ora.MUL), ("div", ora.DIV)):
        say("norm", op, m, n)
        gpu.call("mnv_norm_%s_col" % op, dx.p, dr.p, do.p, m, n)
        assert_bits_equal(gpu.down(do), ora.norm_arithmetic(typ, x, [m, n], row, [0]), op + "_col")
        gpu.call("mnv_norm_%s_row" % op, dx.p, dc.p, do.p, m, n)
        assert_bits_equal(gpu.down(do), ora.norm_arithmetic(typ, x, [m, n], col, [1]), op + "_row")


def test_invalid_arguments_are_rejected(gpu):
    L = gpu.L
    d = gpu.empty(16)
    assert L.mnv_add(None, d.p, d.p, 16, gpu.dev.stream) == -1
    assert L.mnv_add(None, None, None, 0, gpu.dev.stream) == 0  # empty input is a no-op
    assert L.mnv_norm_add_col(d.p, d.p, d.p, -1, 4, gpu.dev.stream) == -1
    assert L.mnv_reduce_sum_col(d.p, d.p, 0, 4, gpu.dev.stream) == -1
    assert L.mnv_sgemm_nn(d.p, d.p, d.p, 4, 4, 0, None, 0, gpu.dev.stream) == -1
    assert L.mnv_conv_fwd(d.p, d.p, d.p, d.p, 1, 1, 1, 2, 2, 0, 0, 1, 1, 3, 3, None, 0, gpu.dev.stream) == -1
    assert L.mnv_maxpool_fwd(d.p, d.p, 1, 1, 4, 4, 0, 1, 2, 2, 0, 0, gpu.dev.stream) == -1


# ------------------------------------------------- Concat / Slice / Select movement
@pytest.mark.parametrize("row_elems,rows,sp,dp,shift", [
    (64, 5, 64, 200, 0),        # 16-byte path
    (64, 5, 128, 64, 0),
    (63, 7, 70, 91, 0),         # scalar path: odd run length
    (64, 3, 64, 64, 1),         # scalar path: unaligned pointers
    (1, 1000, 3, 2, 0),         # many one-float rows
    (70000, 3, 70000, 140000, 0),
])
def test_copy_2d(gpu, row_elems, rows, sp, dp, shift):
    src = _rand(rows * sp + shift, 90)
    dst0 = _rand(rows * dp + shift, 91)
    dsrc, ddst = gpu.up(src), gpu.up(dst0)
    gpu.call("mnv_copy_2d", ctypes.c_void_p(dsrc.ptr + 4 * shift), ctypes.c_void_p(ddst.ptr + 4 * shift),
             ctypes.c_size_t(row_elems), ctypes.c_size_t(rows), ctypes.c_size_t(sp), ctypes.c_size_t(dp))
    want = dst0.copy()
    for r in range(rows):
        want[shift + r * dp: shift + r * dp + row_elems] = src[shift + r * sp: shift + r * sp + row_elems]
    assert_bits_equal(gpu.down(ddst), want, "copy_2d (elements between rows untouched)")


def test_select_columns(gpu, ora):
    rows, cols = 37, 11
    x = _rand(rows * cols, 92)
    idx = [3, 0, 10, 3, 7]
    dx, dd = gpu.up(x), gpu.up(np.full(rows * len(idx), np.nan, np.float32))
    arr = (ctypes.c_int * len(idx))(*idx)
    nbytes = gpu.L.mnv_select_workspace_bytes(len(idx))
    ws = gpu.empty(nbytes // 4 + 1)
    gpu.call("mnv_select", dx.p, dd.p, arr, len(idx), rows, cols, ws.p, ctypes.c_size_t(nbytes))
    assert_bits_equal(gpu.down(dd), ora.select(x, rows, cols, idx), "select")
    # out-of-range index and missing workspace are refused
    bad = (ctypes.c_int * 1)(cols)
    assert gpu.L.mnv_select(dx.p, dd.p, bad, 1, rows, cols, ws.p, ctypes.c_size_t(nbytes), gpu.dev.stream) == -1
    assert gpu.L.mnv_select(dx.p, dd.p, arr, len(idx), rows, cols, None, ctypes.c_size_t(0), gpu.dev.stream) == -2


# ----------------------------------------------------------------------- random
@pytest.mark.parametrize("n", [1, 3, 4, 1001, 1 << 20])
def test_random_generators_match_oracle(gpu, ora, n):
    seed = 0x0123456789abcdef
    d = gpu.up(np.full(n + 1, np.nan, np.float32))
    gpu.call("mnv_rand_bernoulli", d.p, ctypes.c_size_t(n), ctypes.c_uint64(seed), ctypes.c_float(0.3))
    out = gpu.down(d)
    assert_bits_equal(out[:n], ora.rand_bernoulli(n, seed, 0.3), "bernoulli: same bits as the oracle")
    assert np.isnan(out[n])
    gpu.call("mnv_randn", d.p, ctypes.c_size_t(n), ctypes.c_uint64(seed), ctypes.c_float(-1.0),
             ctypes.c_float(0.5))
    out = gpu.down(d)
    # same uniforms, device log / sin / cos instead of libm: absolute agreement of the normals
    assert np.max(np.abs(out[:n] - ora.randn(n, seed, -1.0, 0.5))) <= 2e-5
    assert np.isnan(out[n])
    # an unaligned destination takes the scalar stores
    gpu.call("mnv_rand_bernoulli", ctypes.c_void_p(d.ptr + 4), ctypes.c_size_t(n), ctypes.c_uint64(seed),
             ctypes.c_float(0.3))
    assert_bits_equal(gpu.down(d)[1:n + 1], ora.rand_bernoulli(n, seed, 0.3), "bernoulli, unaligned")
    assert gpu.L.mnv_rand_bernoulli(d.p, ctypes.c_size_t(n), ctypes.c_uint64(1), ctypes.c_float(1.5),
                                    gpu.dev.stream) == -1


def test_randn_distribution_at_full_size(gpu):
    n = 8192 * 8192
    d = gpu.empty(n)
    gpu.call("mnv_randn", d.p, ctypes.c_size_t(n), ctypes.c_uint64(99), ctypes.c_float(0.0), ctypes.c_float(1.0))
    z = gpu.down(d)
    assert np.isfinite(z).all()
    assert abs(float(z.mean(dtype=np.float64))) < 1e-3 and abs(float(z.std(dtype=np.float64)) - 1.0) < 1e-3
    # tails: P(|z| > 4) = 6.33e-5
    assert abs(np.count_nonzero(np.abs(z) > 4) / n - 6.334e-5) < 5e-6


def test_threshold_norm_bit_exact(gpu, ora):
    n = 100003
    x = _rand(n, 95) * 2
    x[:4] = [0.0, -0.0, 0.7, -0.7]
    dx, dy = gpu.up(x), gpu.empty(n)
    gpu.call("mnv_threshold_norm", dx.p, dy.p, ctypes.c_float(0.7), ctypes.c_size_t(n))
    assert_bits_equal(gpu.down(dy), ora.threshold_norm(x, 0.7), "threshold norm")
