"""Operands of 2^29 elements and more (2 GiB; the reference's own limit is int element
counts, 2^31 - 1): SGEMM cuts the product into panels and the convolutions run chunk by chunk
over the images, instead of refusing the call.  The tensors are generated on the device (the
library's counter-based generator, itself checked against the oracle) so that nothing of
that size crosses the host; results are compared with the same product assembled from
calls below the limit (the oracle-checked path) and with fp64 dot products on sampled
outputs."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, TOL, normwise, say
from minerva_amd import capi

pytestmark = pytest.mark.gpu
SZ = ctypes.c_size_t


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


def _device_normal(gpu, n, seed, stddev=1.0):
    buf = gpu.empty(n)
    gpu.call("mnv_randn", buf.p, SZ(n), ctypes.c_uint64(seed), ctypes.c_float(0.0), ctypes.c_float(stddev))
    return buf


def _down(gpu, buf, first, count):
    """`count` floats of a device buffer starting at element `first`."""
    out = np.empty(count, np.float32)
    capi.check(gpu.L.mnv_memcpy_d2h(out.ctypes.data_as(ctypes.c_void_p), buf.offset(first), SZ(4 * count),
                                    gpu.dev.stream), "d2h")
    gpu.dev.sync()
    return out


@pytest.mark.parametrize("m,n,k", [(32768, 48, 16384),      # A is 2^29 elements: two k ranges
                                   (64, 32768, 16384)])     # B is 2^29 elements: two column panels
def test_sgemm_operand_of_two_gib(gpu, m, n, k):
    assert max(m * k, k * n) >= 1 << 29
    da, db = _device_normal(gpu, m * k, 300), _device_normal(gpu, k * n, 301)
    dc = gpu.up(np.full(m * n, np.nan, np.float32))
    say("sgemm with a 2 GiB operand", m, n, k)
    gpu.call("mnv_sgemm_nn", da.p, db.p, dc.p, m, n, k, None, SZ(0))
    c = gpu.down(dc)
    assert np.isfinite(c).all()
    # the same product from two halves of the k range, each below the limit: the columns of A
    # are contiguous; the matching rows of B are gathered with the library's 2-D copy
    k1 = k // 2
    want = np.zeros(m * n, np.float64)
    for first, count in ((0, k1), (k1, k - k1)):
        bh, ch = gpu.empty(count * n), gpu.empty(m * n)
        gpu.call("mnv_copy_2d", db.offset(first), bh.p, SZ(count), SZ(n), SZ(k), SZ(count))
        gpu.call("mnv_sgemm_nn", da.offset(first * m), bh.p, ch.p, m, n, count, None, SZ(0))
        want += gpu.down(ch)
    assert normwise(c, want) <= 1e-5
    # fp64 check of one output column (one row where A's rows are cheap to fetch)
    rng = np.random.default_rng(302)
    j = int(rng.integers(0, n))
    bcol = _down(gpu, db, j * k, k).astype(np.float64)
    scale = float(np.max(np.abs(c)))
    if m <= 64:   # A^T rows are cheap to fetch in full: all of column j of C in fp64
        a = _down(gpu, da, 0, m * k).reshape(k, m).astype(np.float64)
        assert normwise(c.reshape(n, m)[j], a.T @ bcol) <= TOL
    else:         # one entry of column j: row i of A is strided by m, so A comes back in blocks
        i = int(rng.integers(0, m))
        arow = np.empty(k, np.float64)
        for l0 in range(0, k, 2048):   # 2048 columns of A at a time: m * 2048 floats
            blk = _down(gpu, da, l0 * m, m * min(2048, k - l0)).reshape(-1, m)
            arow[l0:l0 + blk.shape[0]] = blk[:, i]
        assert abs(c.reshape(n, m)[j, i] - float(np.dot(arow, bcol))) <= TOL * scale


def test_convolution_over_a_two_gib_batch(gpu):
    N, C, K, H, W, ph, pw, sv, sh, R, S = 2100, 64, 8, 64, 64, 1, 1, 1, 1, 3, 3
    geo = (C, K, H, W, ph, pw, sv, sh, R, S)
    per_b, per_t, nw = C * H * W, K * H * W, K * C * R * S
    assert N * per_b >= 1 << 29
    dx = _device_normal(gpu, N * per_b, 310)
    ddy = _device_normal(gpu, N * per_t, 311)
    w = (np.random.default_rng(312).standard_normal(nw) * 0.05).astype(np.float32)
    b = np.random.default_rng(313).standard_normal(K).astype(np.float32)
    dw, db = gpu.up(w), gpu.up(b)
    wsb = 64 << 20
    ws = gpu.empty(wsb // 4)
    top = gpu.up(np.full(N * per_t, np.nan, np.float32))
    say("conv fwd over 2100 images (two launches)")
    gpu.call("mnv_conv_fwd", dx.p, dw.p, db.p, top.p, N, *geo, ws.p, SZ(wsb))
    # image ranges at both ends and across the boundary between the launches (2047 images
    # fit one), recomputed by calls below the limit, and one of them against fp64
    Wt = w.reshape(K, C, R, S)[:, :, ::-1, ::-1].astype(np.float64)
    for first, count in ((0, 6), (2040, 14), (N - 5, 5)):
        sub = gpu.empty(count * per_t)
        gpu.call("mnv_conv_fwd", dx.offset(first * per_b), dw.p, db.p, sub.p, count, *geo, ws.p, SZ(wsb))
        got = _down(gpu, top, first * per_t, count * per_t)
        ref = gpu.down(sub)
        assert np.isfinite(got).all() and normwise(got, ref) <= 1e-5, (first, count)
    X = _down(gpu, dx, 2047 * per_b, per_b).reshape(C, H, W).astype(np.float64)   # first image of launch 2
    Y = _down(gpu, top, 2047 * per_t, per_t).reshape(K, H, W)
    rng = np.random.default_rng(314)
    for _ in range(16):
        k, i, j = rng.integers(K), rng.integers(1, H - 1), rng.integers(1, W - 1)
        ref = float(np.sum(X[:, i - 1:i + 2, j - 1:j + 2] * Wt[k])) + float(b[k])
        assert abs(Y[k, i, j] - ref) <= TOL * float(np.max(np.abs(Y)))
    del top
    say("conv bwd data over 2100 images")
    dbd = gpu.empty(N * per_b)
    gpu.call("mnv_conv_bwd_data", ddy.p, dw.p, dbd.p, N, *geo, ws.p, SZ(wsb))
    for first, count in ((0, 4), (2044, 8), (N - 3, 3)):
        sub = gpu.empty(count * per_b)
        gpu.call("mnv_conv_bwd_data", ddy.offset(first * per_t), dw.p, sub.p, count, *geo, ws.p, SZ(wsb))
        got = _down(gpu, dbd, first * per_b, count * per_b)
        assert np.isfinite(got).all() and normwise(got, gpu.down(sub)) <= 1e-5, (first, count)
    del dbd
    say("conv bwd filter over 2100 images (accumulated launch by launch)")
    dfd = gpu.up(np.full(nw, np.nan, np.float32))
    gpu.call("mnv_conv_bwd_filter", dx.p, ddy.p, dfd.p, N, *geo, ws.p, SZ(wsb))
    want = np.zeros(nw, np.float64)
    part = gpu.empty(nw)
    for first in range(0, N, 300):
        count = min(300, N - first)
        gpu.call("mnv_conv_bwd_filter", dx.offset(first * per_b), ddy.offset(first * per_t), part.p, count,
                 *geo, ws.p, SZ(wsb))
        want += gpu.down(part)
    assert normwise(gpu.down(dfd), want) <= 1e-5
    # a single image beyond the limit is still refused
    assert gpu.L.mnv_conv_fwd(dx.p, dw.p, db.p, part.p, 1, 1 << 16, 1, 128, 128, 0, 0, 1, 1, 1, 1, None,
                              SZ(0), gpu.dev.stream) == -1
