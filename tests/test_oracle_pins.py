"""Pins the CPU oracle before anything is compared against it.

Sources of truth, in order: the golden vectors held by the reference's own tests
(tests/golden/*.json, extracted from tests/unittest_conv_forward.cpp:7-68 and
tests/unittest_pooling_forward.cpp:7-81), the closed forms of the reference's
other unit tests, and what the mathematics fixes (fp64 closed forms, adjoint
identities, finite differences, brute force).  None of these retypes the oracle's
own formula.
"""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    with open(os.path.join(GOLD, name)) as f:
        return json.load(f)


# ---------------------------------------------------------------- golden vectors

@pytest.mark.parametrize("case", _load("conv_forward.json"), ids=lambda c: c["name"])
def test_conv_forward_golden(ora, case):
    W, H, C, N = case["input_size"]
    S, R, C2, K = case["weight_size"]
    assert C == C2
    x = np.array(case["input"], dtype=np.float32)
    w = np.array(case["weight"], dtype=np.float32)
    bias = np.array(case["bias"], dtype=np.float32) if case["bias"] else np.zeros(K, np.float32)
    out = ora.conv_fwd(x, w, bias, N, C, K, H, W, case["pad_height"], case["pad_width"],
                       case["stride_vertical"], case["stride_horizontal"], R, S)
    Wo, Ho, K2, N2 = case["correct_size"]
    assert (K2, N2) == (K, N) and out.size == Wo * Ho * K * N
    # unittest_conv_forward.cpp:66: expected = correct_raw[i] + bias[(i / 16) % 5]
    idx = np.arange(out.size)
    want = np.array(case["correct_without_bias"], np.float32) + bias[(idx // (Wo * Ho)) % K]
    assert np.max(np.abs(out - want)) < 1e-5  # reference tolerance is 1e-3; we are far inside


def test_conv_forward_golden_rejects_unflipped_kernel(ora):
    """A cross-correlation (un-flipped filter) must NOT reproduce the golden vector."""
    case = _load("conv_forward.json")[0]
    W, H, C, N = case["input_size"]
    S, R, _, K = case["weight_size"]
    x = np.array(case["input"], np.float32)
    w = np.array(case["weight"], np.float32).reshape(K, C, R, S)[:, :, ::-1, ::-1].copy()
    out = ora.conv_fwd(x, w, None, N, C, K, H, W, 0, 0, 1, 1, R, S)
    assert np.max(np.abs(out - np.array(case["correct_without_bias"], np.float32))) > 1.0


@pytest.mark.parametrize("case", _load("pooling_forward.json"), ids=lambda c: c["name"])
def test_pooling_forward_golden(ora, case):
    W, H, C, N = case["input_size"]
    x = np.array(case["input"], np.float32)
    Wo, Ho, _, _ = case["correct_size"]
    assert ora.pooled_size(H, case["height"], case["stride_vertical"], case["pad_height"]) == Ho
    assert ora.pooled_size(W, case["width"], case["stride_horizontal"], case["pad_width"]) == Wo
    out = ora.pool_fwd(ora.POOL_MAX, x, N, C, H, W, case["stride_vertical"],
                       case["stride_horizontal"], case["height"], case["width"],
                       case["pad_height"], case["pad_width"])
    np.testing.assert_array_equal(out, np.array(case["correct"], np.float32))


# ------------------------------------------------- closed forms of reference tests

def test_reduction_closed_forms(ora):
    # tests/unittest_reduction.cpp:6-149: {5,3} iota
    x = np.arange(15, dtype=np.float32)
    np.testing.assert_array_equal(ora.reduction(ora.MAX, x, [5, 3], [0]), [4, 9, 14])
    np.testing.assert_array_equal(ora.reduction(ora.MAX, x, [5, 3], [1]), [10, 11, 12, 13, 14])
    np.testing.assert_array_equal(ora.reduction(ora.SUM, x, [5, 3], [0]), [10, 35, 60])
    np.testing.assert_array_equal(ora.reduction(ora.SUM, x, [5, 3], [1]), [15, 18, 21, 24, 27])
    np.testing.assert_array_equal(ora.maxindex(x, [5, 3], 0), [4, 4, 4])
    np.testing.assert_array_equal(ora.maxindex(x, [5, 3], 1), [2, 2, 2, 2, 2])


def test_reduction_sequential_order_is_observable(ora):
    # sequential fp32 left fold: (1e8 + 1) + -1e8 = 0 in fp32, but 1e8 + -1e8 + 1 = 1
    x = np.array([1e8, 1.0, -1e8, 1e8, -1e8, 1.0], np.float32)
    np.testing.assert_array_equal(ora.reduction(ora.SUM, x, [3, 2], [0]), [0.0, 1.0])


def test_reduction_nd_against_numpy(ora):
    rng = np.random.default_rng(3)
    dims = [4, 3, 5]
    x = rng.integers(-8, 8, size=60).astype(np.float32)  # small ints: sums exact in fp32
    a = x.reshape(dims[::-1])  # numpy axis k <-> minerva dim (2-k)
    for rd in ([0], [1], [2], [0, 2], [1, 2]):
        axes = tuple(2 - d for d in rd)
        np.testing.assert_array_equal(ora.reduction(ora.SUM, x, dims, rd),
                                      a.sum(axis=axes, keepdims=True).ravel())
        np.testing.assert_array_equal(ora.reduction(ora.MAX, x, dims, rd),
                                      a.max(axis=axes, keepdims=True).ravel())
    for d in range(3):
        np.testing.assert_array_equal(ora.maxindex(x, dims, d),
                                      a.argmax(axis=2 - d).ravel().astype(np.float32))


def test_maxindex_ties_and_nan(ora):
    x = np.array([1, 3, 3, 2, 5, 5, 5, 0], np.float32)
    np.testing.assert_array_equal(ora.maxindex(x, [4, 2], 0), [1, 0])
    # NaN never wins unless first (strict '<' is false for NaN)
    y = np.array([1, np.nan, 2, 0, np.nan, 1, 2, 3], np.float32)
    np.testing.assert_array_equal(ora.maxindex(y, [4, 2], 0), [2, 0])


def test_arithmetic_closed_forms(ora):
    rng = np.random.default_rng(0)
    a = rng.standard_normal(720).astype(np.float32)
    b = rng.standard_normal(720).astype(np.float32)
    np.testing.assert_array_equal(ora.arithmetic(ora.ADD, a, b), a + b)
    np.testing.assert_array_equal(ora.arithmetic(ora.SUB, a, b), a - b)
    np.testing.assert_array_equal(ora.arithmetic(ora.MUL, a, b), a * b)
    np.testing.assert_array_equal(ora.arithmetic(ora.DIV, a, b), a / b)
    v = np.float32(3.291)  # tests/unittest_arithmetic_const.cpp:75
    np.testing.assert_array_equal(ora.arithmetic_const(ora.SUB, 0, v, a), v - a)
    np.testing.assert_array_equal(ora.arithmetic_const(ora.SUB, 1, v, a), a - v)
    np.testing.assert_array_equal(ora.arithmetic_const(ora.DIV, 0, v, a), v / a)
    np.testing.assert_array_equal(ora.arithmetic_const(ora.DIV, 1, v, a), a / v)
    np.testing.assert_array_equal(ora.arithmetic_const(ora.MUL, 1, v, a), a * v)
    np.testing.assert_array_equal(ora.arithmetic_const(ora.ADD, 0, v, a), v + a)
    np.testing.assert_array_equal(ora.elewise(ora.NEG, a), -a)


def test_transcendentals_against_fp64(ora):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(5000) * 3).astype(np.float32)
    x64 = x.astype(np.float64)
    assert np.max(np.abs(ora.elewise(ora.EXP, x) / np.exp(x64) - 1)) < 3e-7
    pos = np.abs(x) + np.float32(0.5)
    assert np.max(np.abs(ora.elewise(ora.LN, pos) - np.log(pos.astype(np.float64)))) < 3e-7
    assert np.max(np.abs(ora.activation_fwd(ora.SIGMOID, x) - 1 / (1 + np.exp(-x64)))) < 2e-7
    assert np.max(np.abs(ora.activation_fwd(ora.TANH, x) - np.tanh(x64))) < 2e-7
    r = ora.activation_fwd(ora.RELU, np.array([-1, -0.0, 0.0, 2, np.nan], np.float32))
    np.testing.assert_array_equal(r, np.array([0, 0, 0, 2, 0], np.float32))
    assert not np.signbit(r[1])


def test_norm_arithmetic_closed_forms(ora):
    # tests/unittest_norm_arithmetic.cpp:6-36: {9,7}+{1,7} and {9,7}*{9,1}
    rng = np.random.default_rng(2)
    x = rng.standard_normal(63).astype(np.float32)
    a = x.reshape(7, 9)  # a[col, row]
    row = rng.standard_normal(7).astype(np.float32)
    col = rng.standard_normal(9).astype(np.float32)
    np.testing.assert_array_equal(ora.norm_arithmetic(ora.ADD, x, [9, 7], row, [0]),
                                  (a + row[:, None]).ravel())
    np.testing.assert_array_equal(ora.norm_arithmetic(ora.MUL, x, [9, 7], col, [1]),
                                  (a * col[None, :]).ravel())
    np.testing.assert_array_equal(ora.norm_arithmetic(ora.SUB, x, [9, 7], col, [1]),
                                  (a - col[None, :]).ravel())
    np.testing.assert_array_equal(ora.norm_arithmetic(ora.DIV, x, [9, 7], row, [0]),
                                  (a / row[:, None]).ravel())
    # N-d: replicate dims 0 and 2 of {3,4,5}
    y = rng.standard_normal(60).astype(np.float32)
    v = rng.standard_normal(4).astype(np.float32)
    want = y.reshape(5, 4, 3) + v[None, :, None]
    np.testing.assert_array_equal(ora.norm_arithmetic(ora.ADD, y, [3, 4, 5], v, [0, 2]),
                                  want.ravel())


def test_matmult_textbook_and_fp64(ora):
    # tests/unittest_sgemm.cpp:7-28: {3,2} x {2,5}; then a larger case vs fp64
    rng = np.random.default_rng(4)
    for (m, k, n) in [(3, 2, 5), (37, 53, 29)]:
        a = rng.standard_normal(m * k).astype(np.float32)
        b = rng.standard_normal(k * n).astype(np.float32)
        A = a.reshape(k, m).T.astype(np.float64)  # col-major {m,k}
        B = b.reshape(n, k).T.astype(np.float64)
        want = (A @ B)
        got = ora.matmult(a, b, m, n, k).reshape(n, m).T
        assert np.max(np.abs(got - want)) < 1e-5 * max(1.0, np.max(np.abs(want)))
        np.testing.assert_array_equal(ora.matmult(a, b, m, n, k, fast=True).reshape(n, m).T, got)
    # an asymmetric, integer-valued case catches a transposed operand or index slip exactly
    a = np.arange(6, dtype=np.float32)       # A{3,2}: A[i,l] = i + 3l
    b = np.arange(10, dtype=np.float32) - 4  # B{2,5}: B[l,j] = l + 2j - 4
    want = np.array([[sum((i + 3 * l) * (l + 2 * j - 4) for l in range(2)) for j in range(5)]
                     for i in range(3)], np.float32)
    np.testing.assert_array_equal(ora.matmult(a, b, 3, 5, 2).reshape(5, 3).T, want)


def test_transpose(ora):
    x = np.arange(12, dtype=np.float32)  # in{n=4,m=3}: in[j + i*4]
    out = ora.transpose(x, 3, 4)         # out{3,4}: out[i + j*3]
    np.testing.assert_array_equal(out.reshape(4, 3), x.reshape(3, 4).T)


def test_softmax_forward(ora):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(10 * 17) * 4).astype(np.float32)
    y = ora.softmax_dim0(x, 10).reshape(17, 10)
    x64 = x.reshape(17, 10).astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(y - want)) < 3e-7
    assert np.max(np.abs(y.sum(axis=1) - 1)) < 1e-6
    # instance == dim-0 softmax on {K,1,1,N}; channel == instance when H = W = 1
    np.testing.assert_array_equal(ora.softmax_channel_fwd(x, 17, 10, 1, 1), y.ravel())
    # channel mode on a real {W,H,C,N} tensor against fp64
    n, c, h, w = 2, 5, 3, 4
    z = rng.standard_normal(n * c * h * w).astype(np.float32)
    z64 = z.reshape(n, c, h, w).astype(np.float64)
    e = np.exp(z64 - z64.max(axis=1, keepdims=True))
    assert np.max(np.abs(ora.softmax_channel_fwd(z, n, c, h, w).reshape(n, c, h, w)
                         - e / e.sum(axis=1, keepdims=True))) < 3e-7


def _fd(f, x, dy, eps=1e-3):
    """Central finite difference of <f(x), dy> in fp64."""
    g = np.zeros(x.size)
    for i in range(x.size):
        xp, xm = x.copy(), x.copy()
        xp[i] += eps
        xm[i] -= eps
        g[i] = np.dot(f(xp) - f(xm), dy) / (2 * eps)
    return g


def test_softmax_backward_finite_difference(ora):
    rng = np.random.default_rng(6)
    n, c, h, w = 2, 4, 2, 3
    x = rng.standard_normal(n * c * h * w)
    dy = rng.standard_normal(x.size)

    def inst(v):
        v = v.reshape(n, -1)
        e = np.exp(v - v.max(axis=1, keepdims=True))
        return (e / e.sum(axis=1, keepdims=True)).ravel()

    def chan(v):
        v = v.reshape(n, c, h, w)
        e = np.exp(v - v.max(axis=1, keepdims=True))
        return (e / e.sum(axis=1, keepdims=True)).ravel()

    got = ora.softmax_instance_bwd(dy, inst(x), n, c, h, w)
    assert np.max(np.abs(got - _fd(inst, x, dy))) < 1e-5
    got = ora.softmax_channel_bwd(dy, chan(x), n, c, h, w)
    assert np.max(np.abs(got - _fd(chan, x, dy))) < 1e-5


def test_activation_backward_finite_difference(ora):
    rng = np.random.default_rng(7)
    x = rng.standard_normal(40)
    x[np.abs(x) < 0.05] = 0.3  # keep relu away from its kink
    dy = rng.standard_normal(40)
    fwd = {ora.SIGMOID: lambda v: 1 / (1 + np.exp(-v)), ora.RELU: lambda v: np.maximum(v, 0),
           ora.TANH: np.tanh}
    for alg, f in fwd.items():
        got = ora.activation_bwd(alg, dy, f(x), x)
        assert np.max(np.abs(got - _fd(f, x, dy, 1e-4))) < 2e-5


# --------------------------------------------------- convolution: adjoint + brute

CONV_CASES = [
    # N, C, K, H, W, ph, pw, sv, sh, R, S
    (2, 3, 4, 7, 9, 0, 0, 1, 1, 3, 5),
    (2, 2, 3, 8, 7, 2, 1, 2, 3, 3, 2),   # strided, padded, non-square, ragged fit
    (1, 4, 2, 6, 6, 1, 1, 1, 1, 3, 3),
]


def _conv64(x, w, N, C, K, H, W, ph, pw, sv, sh, R, S):
    """fp64 brute force written from the cuDNN CONVOLUTION definition with numpy slicing
    (a different loop structure from the oracle: it scatters taps instead of gathering)."""
    Ho, Wo = (H + 2 * ph - R) // sv + 1, (W + 2 * pw - S) // sh + 1
    xp = np.zeros((N, C, H + 2 * ph, W + 2 * pw))
    xp[:, :, ph:ph + H, pw:pw + W] = x.reshape(N, C, H, W)
    wf = w.reshape(K, C, R, S)[:, :, ::-1, ::-1]
    out = np.zeros((N, K, Ho, Wo))
    for r in range(R):
        for s in range(S):
            patch = xp[:, :, r:r + sv * Ho:sv, s:s + sh * Wo:sh][:, :, :Ho, :Wo]
            out += np.einsum("nchw,kc->nkhw", patch, wf[:, :, r, s])
    return out.ravel()


@pytest.mark.parametrize("p", CONV_CASES)
def test_conv_forward_bruteforce(ora, p):
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    rng = np.random.default_rng(8)
    x = rng.standard_normal(N * C * H * W).astype(np.float32)
    w = rng.standard_normal(K * C * R * S).astype(np.float32)
    b = rng.standard_normal(K).astype(np.float32)
    got = ora.conv_fwd(x, w, b, *p)
    Ho, Wo = ora.conv_out_size(H, R, sv, ph), ora.conv_out_size(W, S, sh, pw)
    want = _conv64(x.astype(np.float64), w.astype(np.float64), *p).reshape(N, K, Ho * Wo) \
        + b[None, :, None]
    assert np.max(np.abs(got - want.ravel())) < 2e-5


@pytest.mark.parametrize("p", CONV_CASES)
def test_conv_backward_adjoint_identities(ora, p):
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    rng = np.random.default_rng(9)
    x = rng.standard_normal(N * C * H * W).astype(np.float32)
    w = rng.standard_normal(K * C * R * S).astype(np.float32)
    Ho, Wo = ora.conv_out_size(H, R, sv, ph), ora.conv_out_size(W, S, sh, pw)
    dy = rng.standard_normal(N * K * Ho * Wo).astype(np.float32)
    y = _conv64(x.astype(np.float64), w.astype(np.float64), *p)
    lhs = np.dot(y, dy.astype(np.float64))
    dx = ora.conv_bwd_data(dy, w, *p).astype(np.float64)
    dw = ora.conv_bwd_filter(dy, x, *p).astype(np.float64)
    assert abs(np.dot(dx, x) - lhs) < 1e-4 * max(1, abs(lhs))
    assert abs(np.dot(dw, w) - lhs) < 1e-4 * max(1, abs(lhs))
    # the adjoint identity holds for ANY x / w only if dX, dW are the true adjoints:
    for _ in range(3):
        x2 = rng.standard_normal(x.size)
        w2 = rng.standard_normal(w.size)
        assert abs(np.dot(dx, x2) - np.dot(_conv64(x2, w.astype(np.float64), *p), dy)) < 2e-4 * max(1, abs(lhs))
        assert abs(np.dot(dw, w2) - np.dot(_conv64(x.astype(np.float64), w2, *p), dy)) < 2e-4 * max(1, abs(lhs))
    db = ora.conv_bwd_bias(dy, N, K, Ho, Wo)
    assert np.max(np.abs(db - dy.reshape(N, K, -1).astype(np.float64).sum(axis=(0, 2)))) < 1e-4


# --------------------------------------------------------------- pooling beyond golden

POOL_CASES = [
    # N, C, H, W, sv, sh, kh, kw, ph, pw
    (2, 3, 7, 9, 2, 2, 3, 3, 0, 0),
    (1, 2, 6, 5, 2, 3, 3, 2, 1, 1),
    (2, 2, 8, 8, 2, 2, 2, 2, 0, 0),
    (1, 1, 5, 5, 1, 1, 3, 3, 1, 1),
]


def _windows(H, W, sv, sh, kh, kw, ph, pw, Ho, Wo):
    for i in range(Ho):
        for j in range(Wo):
            ys, xs = max(i * sv - ph, 0), max(j * sh - pw, 0)
            ye, xe = min(i * sv - ph + kh, H), min(j * sh - pw + kw, W)
            yield i, j, ys, ye, xs, xe


@pytest.mark.parametrize("p", POOL_CASES)
def test_pool_bruteforce(ora, p):
    N, C, H, W, sv, sh, kh, kw, ph, pw = p
    rng = np.random.default_rng(10)
    # few distinct values => many ties, which is what the tie policy is about
    x = rng.integers(0, 4, size=N * C * H * W).astype(np.float32)
    Ho, Wo = ora.pooled_size(H, kh, sv, ph), ora.pooled_size(W, kw, sh, pw)
    dy = rng.standard_normal(N * C * Ho * Wo).astype(np.float32)
    X = x.reshape(N * C, H, W)
    top = ora.pool_fwd(ora.POOL_MAX, x, *p).reshape(N * C, Ho, Wo)
    avg = ora.pool_fwd(ora.POOL_AVG, x, *p).reshape(N * C, Ho, Wo)
    dx, mask = ora.pool_bwd(ora.POOL_MAX, dy, top, x, *p, want_mask=True)
    dxa = ora.pool_bwd(ora.POOL_AVG, dy, avg, x, *p)
    want_dx = np.zeros((N * C, H, W))
    want_dxa = np.zeros((N * C, H, W))
    DY = dy.reshape(N * C, Ho, Wo)
    for q in range(N * C):
        for i, j, ys, ye, xs, xe in _windows(H, W, sv, sh, kh, kw, ph, pw, Ho, Wo):
            win = X[q, ys:ye, xs:xe]
            assert top[q, i, j] == win.max()
            assert abs(avg[q, i, j] - win.sum() / (kh * kw)) < 1e-6
            a = int(np.argmax(win))  # numpy argmax = first max in row-major scan
            yy, xx = ys + a // (xe - xs), xs + a % (xe - xs)
            assert mask.reshape(N * C, Ho, Wo)[q, i, j] == yy * W + xx
            want_dx[q, yy, xx] += DY[q, i, j]
            want_dxa[q, ys:ye, xs:xe] += DY[q, i, j] / (kh * kw)
    assert np.max(np.abs(dx.reshape(N * C, H, W) - want_dx)) < 1e-5
    assert np.max(np.abs(dxa.reshape(N * C, H, W) - want_dxa)) < 1e-5
    assert abs(dx.astype(np.float64).sum() - dy.astype(np.float64).sum()) < 1e-4


def test_pooled_size_matches_ceil_mode_formula(ora):
    # closed form of ceil-mode pooling with the "last window must start inside" clip
    import math
    for H in range(1, 14):
        for k in range(1, 6):
            for s in range(1, 5):
                for p in range(0, k // 2 + 1):
                    if H + 2 * p < k:
                        continue
                    want = math.ceil((H + 2 * p - k) / s) + 1
                    if (want - 1) * s >= H + p:
                        want -= 1
                    assert ora.pooled_size(H, k, s, p) == want


# ------------------------------------------------------------------------ LRN
def _lrn64(x, size, alpha, beta, n, c, h, w, backward_window=False):
    """fp64 closed form: (top, scale) with the window written out as a direct sum."""
    X = x.reshape(n, c, h * w).astype(np.float64)
    pre = size - (size + 1) // 2 if backward_window else (size - 1) // 2
    post = size - pre - 1
    scale = np.empty_like(X)
    for k in range(c):
        lo, hi = max(k - pre, 0), min(k + post, c - 1)
        scale[:, k] = 1.0 + alpha / size * (X[:, lo:hi + 1] ** 2).sum(axis=1)
    return (X * scale ** (-beta)).ravel(), scale.ravel()


@pytest.mark.parametrize("size,c", [(5, 8), (3, 7), (1, 4), (5, 96), (4, 9), (5, 3)])
def test_lrn_forward_closed_form(ora, size, c):
    rng = np.random.default_rng(70 + size + c)
    n, h, w = 2, 3, 4
    alpha, beta = 1e-1, 0.75   # a large alpha makes the normalisation visible
    x = (rng.standard_normal(n * c * h * w) * 3).astype(np.float32)
    top, scale = ora.lrn_fwd(x, size, alpha, beta, n, c, h, w)
    want_top, want_scale = _lrn64(x, size, alpha, beta, n, c, h, w)
    assert np.max(np.abs(scale - want_scale) / want_scale) < 2e-6
    assert np.max(np.abs(top - want_top)) <= 2e-6 * np.max(np.abs(want_top))
    # a window shifted by one channel (the plausible off-by-one) must not pass
    if size > 1 and c >= size:
        X = x.reshape(n, c, h * w).astype(np.float64)
        wrong = np.empty_like(X)
        pre, post = (size - 1) // 2 + 1, size - (size - 1) // 2 - 2
        for k in range(c):
            lo, hi = max(k - pre, 0), min(k + post, c - 1)
            wrong[:, k] = 1.0 + alpha / size * (X[:, lo:hi + 1] ** 2).sum(axis=1)
        assert np.max(np.abs(scale - wrong.ravel()) / wrong.ravel()) > 1e-3


@pytest.mark.parametrize("size,c", [(5, 8), (3, 5), (4, 7), (5, 3)])
def test_lrn_backward_finite_difference(ora, size, c):
    rng = np.random.default_rng(80 + size + c)
    n, h, w = 1, 2, 2
    alpha, beta = 2e-1, 0.75
    x = rng.standard_normal(n * c * h * w).astype(np.float32)
    dy = rng.standard_normal(x.size).astype(np.float32)
    top, scale = ora.lrn_fwd(x, size, alpha, beta, n, c, h, w)
    got = ora.lrn_bwd(x, top, scale, dy, size, alpha, beta, n, c, h, w)

    def fwd(v):
        return _lrn64(v, size, alpha, beta, n, c, h, w)[0]

    # the backward window (cuda_kernel.h:291-292: pre_pad = size - (size+1)/2) is the adjoint
    # of the forward one (cuda_kernel.h:234-235) for even sizes too, so the finite difference
    # of the forward pass pins it
    want = _fd(fwd, x.astype(np.float64), dy.astype(np.float64), eps=1e-4)
    assert np.max(np.abs(got - want)) < 2e-5 * max(1.0, np.max(np.abs(want)))


# ------------------------------------------------------------------------ RNG
def test_philox_known_answer_vectors(ora):
    # philox4x32_10 known-answer vectors of the Random123 distribution (kat_vectors)
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
         (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in kat:
        assert tuple(ora.philox4x32_10(ctr, key)) == want


def test_random_tensors_mapping_and_distribution(ora):
    from scipy import stats
    n, seed = 400003, 0x1234567890abcdef
    z = ora.randn(n, seed, 1.5, 2.0)
    # element 4b+t comes from counter (b, 0, 0, 0) and the two halves of the seed as key
    x = ora.philox4x32_10((7, 0, 0, 0), (seed & 0xffffffff, seed >> 32))
    u1 = np.float32((x[0] >> 8) + 1) * np.float32(2.0 ** -24)
    u2 = np.float32(x[1] >> 8) * np.float32(2.0 ** -24)
    r = np.sqrt(-2.0 * np.log(np.float64(u1)))
    assert abs(z[28] - (1.5 + 2.0 * r * np.cos(2 * np.pi * np.float64(u2)))) < 1e-5
    assert abs(z[29] - (1.5 + 2.0 * r * np.sin(2 * np.pi * np.float64(u2)))) < 1e-5
    # distribution: mean, deviation, and a Kolmogorov-Smirnov test against N(1.5, 2)
    assert abs(z.mean() - 1.5) < 0.02 and abs(z.std() - 2.0) < 0.02
    assert stats.kstest((z[:100000] - 1.5) / 2.0, "norm").pvalue > 1e-3
    assert np.array_equal(ora.randn(n, seed, 1.5, 2.0), z)          # a function of the seed
    assert not np.array_equal(ora.randn(n, seed + 1, 1.5, 2.0), z)
    assert np.array_equal(ora.randn(1001, seed, 1.5, 2.0), z[:1001])  # and not of the length
    b = ora.rand_bernoulli(n, seed, 0.3)
    assert set(np.unique(b)) == {0.0, 1.0}
    assert abs(b.mean() - 0.3) < 0.005
    assert b[28] == (1.0 if np.float32(x[0] >> 8) * np.float32(2.0 ** -24) < np.float32(0.3) else 0.0)
    assert ora.rand_bernoulli(1000, 3, 0.0).sum() == 0 and ora.rand_bernoulli(1000, 3, 1.0).sum() == 1000


def test_threshold_norm_is_a_clip(ora):
    x = np.array([-3.0, -1.0, -0.5, 0.0, 0.25, 1.0, 2.5, np.inf, -np.inf], np.float32)
    got = ora.threshold_norm(x, 1.0)
    # |x| / x * t is exactly sign(x) * t, so the operator is a clip to [-t, t] (inf/inf = nan)
    want = np.clip(x, -1.0, 1.0)
    assert np.array_equal(got[:7], want[:7])
    assert np.isnan(got[7]) and np.isnan(got[8])


def test_benchmark_inputs_of_package_and_oracle_agree():
    """The package's generator of the benchmark inputs (what bench.py feeds the GPU) and
    the oracle's (what the parity tests feed both sides) are the same seeded data."""
    from minerva_amd import configs
    from oracle import nets
    for kind, batch in (("mlp", 5), ("cnn", 3), ("alexnet", 1)):
        pa, da, la = configs.make_inputs(kind, batch)
        pb, db, lb = nets.make_inputs(kind, batch)
        assert sorted(pa) == sorted(pb)
        for k in pa:
            assert np.array_equal(pa[k], pb[k]), (kind, k)
        assert np.array_equal(da, db) and np.array_equal(la, lb), kind
