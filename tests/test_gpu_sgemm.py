"""GPU parity of the MFMA SGEMM against the CPU oracle (normwise <= 1e-4) and, at
sizes the oracle cannot reach, against properties: an fp64 reference on sampled
entries, exact reproduction of a permuted operand, and linearity."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, TOL, assert_bits_equal, normwise, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


def _rand(n, seed):
    return np.random.default_rng(seed).standard_normal(n).astype(np.float32)


def _gemm(gpu, a, b, m, n, k, workspace=True):
    da, db, dc = gpu.up(a), gpu.up(b), gpu.empty(m * n)
    ws_bytes = gpu.L.mnv_sgemm_nn_workspace_bytes(m, n, k) if workspace else 0
    ws = gpu.empty(ws_bytes // 4 + 1) if ws_bytes else None
    gpu.call("mnv_sgemm_nn", da.p, db.p, dc.p, m, n, k, ws.p if ws else None,
             ctypes.c_size_t(ws_bytes))
    return gpu.down(dc)


SMALL = [(3, 5, 2), (1, 1, 1), (37, 29, 53), (64, 64, 16), (128, 128, 128), (130, 70, 19),
         (256, 256, 784), (10, 256, 256), (256, 10, 256), (257, 129, 65), (1000, 256, 512),
         (4, 4, 4096), (512, 384, 100)]


@pytest.mark.parametrize("m,n,k", SMALL)
@pytest.mark.parametrize("workspace", [True, False])
def test_sgemm_against_oracle(gpu, ora, m, n, k, workspace):
    a, b = _rand(m * k, 30), _rand(k * n, 31)
    say("sgemm", m, n, k, "workspace" if workspace else "no workspace")
    got = _gemm(gpu, a, b, m, n, k, workspace)
    ref = ora.matmult(a, b, m, n, k, fast=True)
    assert normwise(got, ref) <= TOL
    A = a.reshape(k, m).T.astype(np.float64)
    B = b.reshape(n, k).T.astype(np.float64)
    assert normwise(got.reshape(n, m).T, A @ B) <= TOL


def _random_shapes(count, seed):
    """Seeded extents around what the plans branch on: tile edges (63 / 64 / 65, 127 / 128 / 129),
    multiples of four and not, a k of one slab and of many."""
    rng = np.random.default_rng(seed)
    edge = [1, 2, 3, 4, 15, 16, 17, 63, 64, 65, 96, 127, 128, 129, 191, 192, 255, 256, 257]
    out = []
    while len(out) < count:
        pick = lambda hi: int(rng.choice(edge)) if rng.random() < 0.5 else int(rng.integers(1, hi))
        m, n, k = pick(700), pick(700), pick(3000)
        if m * n * k <= 80e6:
            out.append((m, n, k))
    return out


@pytest.mark.parametrize("m,n,k", _random_shapes(60, 7))
def test_sgemm_random_shapes_against_fp64(gpu, m, n, k):
    """mnv_sgemm_nn with and without a workspace, and the same product with either operand
    given transposed (mnv_sgemm_tn / mnv_sgemm_nt), against the fp64 product."""
    a, b = _rand(m * k, 60), _rand(k * n, 61)
    A = a.reshape(k, m).T.astype(np.float64)   # column-major m x k
    B = b.reshape(n, k).T.astype(np.float64)   # column-major k x n
    want = (A @ B).T.reshape(-1)               # column-major m x n, flattened
    say("sgemm, random shape", m, n, k)
    for workspace in (True, False):
        assert normwise(_gemm(gpu, a, b, m, n, k, workspace), want) <= TOL
    ws_bytes = gpu.L.mnv_sgemm_nn_workspace_bytes(m, n, k)
    ws = gpu.empty(ws_bytes // 4 + 1)
    dc = gpu.empty(m * n)
    at = gpu.up(np.ascontiguousarray(a.reshape(k, m).T).reshape(-1))   # A^T: column-major k x m
    gpu.call("mnv_sgemm_tn", at.p, gpu.up(b).p, None, dc.p, m, n, k, ws.p, ctypes.c_size_t(ws_bytes))
    assert normwise(gpu.down(dc), want) <= TOL
    bt = gpu.up(np.ascontiguousarray(b.reshape(n, k).T).reshape(-1))   # B^T: column-major n x k
    gpu.call("mnv_sgemm_nt", gpu.up(a).p, bt.p, dc.p, m, n, k, ws.p, ctypes.c_size_t(ws_bytes))
    assert normwise(gpu.down(dc), want) <= TOL


def _plan(gpu, m, n, k, ws_bytes):
    tile, ranges, groups = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert gpu.L.mnv_sgemm_nn_plan(m, n, k, ctypes.c_size_t(ws_bytes), ctypes.byref(tile),
                                   ctypes.byref(ranges), ctypes.byref(groups)) == 0
    return tile.value, ranges.value, groups.value


GROUPED = [  # m, n, k, workspace: plans with four wavefront groups per workgroup
    (1000, 1000, 2049, False),  # ragged in every extent, the last slab holds one k
    (777, 1030, 777, False),    # 49 slabs: the last group multiplies one slab, a partial one
    (500, 500, 3000, True),     # with k ranges in memory as well
    (200, 1000, 4099, True),
    (36, 4096, 5000, True),     # a single partial tile in m
    (1000, 130, 8200, True),    # five ranges of four quarters, 513 slabs
    (1024, 1024, 1024, True),   # no k ranges at all: one workgroup per tile and CU
    (4096, 256, 9216, True),   # 128x128 tiles, four ranges
]


@pytest.mark.parametrize("m,n,k,workspace", GROUPED)
def test_sgemm_with_grouped_workgroups(gpu, m, n, k, workspace):
    """Products whose plan runs four wavefront groups per workgroup (each group a quarter of
    the workgroup's k range, added through LDS) against the fp64 product."""
    ws_bytes = gpu.L.mnv_sgemm_nn_workspace_bytes(m, n, k) if workspace else 0
    tile, ranges, groups = _plan(gpu, m, n, k, ws_bytes)
    assert groups == 4, "the case is meant to take the grouped kernel"
    a, b = _rand(m * k, 40), _rand(k * n, 41)
    say("sgemm, grouped workgroups", m, n, k, "tile", tile, "k ranges", ranges)
    got = _gemm(gpu, a, b, m, n, k, workspace).reshape(n, m)
    A = a.reshape(k, m).astype(np.float64)   # A[l, i]
    B = b.reshape(n, k).astype(np.float64)   # B[j, l]
    if m * n * k <= 2e9:
        assert normwise(got, B @ A) <= TOL
    else:
        rng = np.random.default_rng(42)
        rows, cols = rng.integers(0, m, 64), rng.integers(0, n, 64)
        assert normwise(got[np.ix_(cols, rows)], B[cols] @ A[:, rows]) <= TOL
    # identical calls give identical bits (the groups are added in a fixed order)
    assert_bits_equal(_gemm(gpu, a, b, m, n, k, workspace).reshape(n, m), got, "second call")


@pytest.mark.parametrize("m,n,k", [(2100, 2100, 700), (2052, 2300, 261), (4224, 4100, 300)])
def test_sgemm_with_a_cut_tail(gpu, m, n, k):
    """Tile counts a little over a multiple of 256 (1089 and 1188 small tiles, 1089 large ones): with a
    workspace the tiles past the multiple are cut into k ranges and added by a second
    kernel; against the fp64 product, and against the same call without a workspace
    (no cut) to the tolerance of two fp32 summation orders."""
    assert gpu.L.mnv_sgemm_nn_workspace_bytes(m, n, k) > 0
    assert _plan(gpu, m, n, k, gpu.L.mnv_sgemm_nn_workspace_bytes(m, n, k))[1:] == (1, 1)
    a, b = _rand(m * k, 44), _rand(k * n, 45)
    say("sgemm, cut tail", m, n, k)
    got = _gemm(gpu, a, b, m, n, k, True).reshape(n, m)
    plain = _gemm(gpu, a, b, m, n, k, False).reshape(n, m)
    A = a.reshape(k, m).astype(np.float64)
    B = b.reshape(n, k).astype(np.float64)
    want = B @ A
    assert normwise(got, want) <= TOL
    assert normwise(plain, want) <= TOL
    assert normwise(got, plain) <= 1e-5
    assert_bits_equal(_gemm(gpu, a, b, m, n, k, True).reshape(n, m), got, "second call")


@pytest.mark.parametrize("m,n,k", [(4092, 4092, 520), (4095, 4093, 515), (8192, 2048, 512)])
def test_sgemm_on_256_row_tiles(gpu, m, n, k):
    """Large products whose 256 x 128 tiles fill the chip in whole rounds take that tile (eight
    wavefronts per workgroup): ragged edges in both extents, vector and scalar fetches, against
    the fp64 product element by element, and the same bits with either operand transposed."""
    ws_bytes = gpu.L.mnv_sgemm_nn_workspace_bytes(m, n, k)
    assert _plan(gpu, m, n, k, ws_bytes) == (256, 1, 1), "the case is meant to take the 256-row tile"
    a, b = _rand(m * k, 46), _rand(k * n, 47)
    say("sgemm, 256 x 128 tiles", m, n, k)
    got = _gemm(gpu, a, b, m, n, k)
    A = a.reshape(k, m).astype(np.float64)
    B = b.reshape(n, k).astype(np.float64)
    want = B @ A
    err = np.abs(got.reshape(n, m) - want)
    worst = np.unravel_index(int(np.argmax(err)), err.shape)
    assert err[worst] <= TOL * float(np.max(np.abs(want))), "largest error at column %d, row %d" % worst
    ws = gpu.empty(ws_bytes // 4 + 1)
    dc = gpu.empty(m * n)
    at = gpu.up(np.ascontiguousarray(a.reshape(k, m).T).reshape(-1))
    gpu.call("mnv_sgemm_tn", at.p, gpu.up(b).p, None, dc.p, m, n, k, ws.p, ctypes.c_size_t(ws_bytes))
    assert_bits_equal(gpu.down(dc), got, "A given transposed")
    bt = gpu.up(np.ascontiguousarray(b.reshape(n, k).T).reshape(-1))
    gpu.call("mnv_sgemm_nt", gpu.up(a).p, bt.p, dc.p, m, n, k, ws.p, ctypes.c_size_t(ws_bytes))
    assert_bits_equal(gpu.down(dc), got, "B given transposed")


def test_sgemm_reference_unit_test_shape(gpu):
    # tests/unittest_sgemm.cpp:7-28: {3,2} x {2,5} against the triple loop
    a = np.arange(6, dtype=np.float32)
    b = np.arange(10, dtype=np.float32) - 4
    want = np.array([[sum((i + 3 * l) * (l + 2 * j - 4) for l in range(2)) for j in range(5)]
                     for i in range(3)], np.float32)
    np.testing.assert_array_equal(_gemm(gpu, a, b, 3, 5, 2).reshape(5, 3).T, want)


BIG = [(4096, 4096, 4096), (4096, 256, 9216), (4096, 256, 4096), (1000, 256, 4096),
       (9216, 256, 4096), (4096, 9216, 256)]


@pytest.mark.parametrize("m,n,k", BIG)
def test_sgemm_config_shapes_full_fp64(gpu, m, n, k):
    """The products of the benchmark configuration against the fp64 product, every element
    (tests/unittest_sgemm.cpp:19-27 compares every element of its small product the same
    way).  A sampled sub-product and the four corners go first: they fail fast and name a
    place; the full comparison then reaches every output tile, so an error confined to one
    tile (tile order, a partial tile at an edge, one k range) cannot pass."""
    a, b = _rand(m * k, 32), _rand(k * n, 33)
    say("sgemm big", m, n, k)
    got = _gemm(gpu, a, b, m, n, k).reshape(n, m)
    A = a.reshape(k, m).astype(np.float64)   # A[l, i]
    B = b.reshape(n, k).astype(np.float64)   # B[j, l]
    rng = np.random.default_rng(34)
    rows = rng.integers(0, m, 48)
    cols = rng.integers(0, n, 48)
    assert normwise(got[np.ix_(cols, rows)], B[cols] @ A[:, rows]) <= TOL
    for (i, j) in ((0, 0), (m - 1, 0), (0, n - 1), (m - 1, n - 1)):
        assert abs(got[j, i] - float(B[j] @ A[:, i])) <= TOL * np.sqrt(k) * 4
    want = B @ A
    scale = float(np.max(np.abs(want)))
    err = np.abs(got - want)
    worst = np.unravel_index(int(np.argmax(err)), err.shape)
    assert err[worst] <= TOL * scale, "largest error at column %d, row %d" % worst
    # per 128 x 128 output tile: no tile may stand out (an error that is small against the
    # largest element of the whole product but systematic inside one tile)
    tn, tm = (n + 127) // 128, (m + 127) // 128
    pad = np.zeros((tn * 128, tm * 128))
    pad[:n, :m] = err
    per_tile = pad.reshape(tn, 128, tm, 128).max(axis=(1, 3))
    assert float(per_tile.max()) <= 8 * max(float(np.median(per_tile)), 1e-7 * scale)


def test_sgemm_permutation_is_exact(gpu):
    # B = permutation matrix: C = A with permuted columns, exactly (x*1 + 0s)
    m, k = 1024, 1024
    a = _rand(m * k, 35)
    perm = np.random.default_rng(36).permutation(k)
    B = np.zeros((k, k), np.float32)      # B[j, l] (numpy view of column-major {k,n})
    B[np.arange(k), perm] = 1.0           # column j picks row perm[j]
    got = _gemm(gpu, a, B.ravel(), m, k, k).reshape(k, m)
    assert_bits_equal(got, a.reshape(k, m)[perm], "A * P")


def test_sgemm_linearity_full_size(gpu):
    m = n = k = 2048
    a, b1, b2 = _rand(m * k, 37), _rand(k * n, 38), _rand(k * n, 39)
    c1 = _gemm(gpu, a, b1, m, n, k)
    c2 = _gemm(gpu, a, b2, m, n, k)
    c12 = _gemm(gpu, a, b1 + b2, m, n, k)
    assert normwise(c12, c1.astype(np.float64) + c2) <= TOL
