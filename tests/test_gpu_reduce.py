"""GPU parity of reductions, arg-max, softmax and transpose against the CPU oracle.
Bit-exact: max, arg-max indices (ties, NaN), transpose.  Normwise <= 1e-4: sums and
softmax forward/backward."""
import numpy as np
import pytest

from gpu_util import Gpu, TOL, assert_bits_equal, normwise, say

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


def _rand(n, seed):
    return np.random.default_rng(seed).standard_normal(n).astype(np.float32)


def test_reference_closed_forms(gpu):
    # tests/unittest_reduction.cpp:6-149, {5,3} iota
    x = np.arange(15, dtype=np.float32)
    dx, do = gpu.up(x), gpu.empty(5)
    gpu.call("mnv_reduce_max_col", dx.p, do.p, 5, 3)
    np.testing.assert_array_equal(gpu.down(do, 3), [4, 9, 14])
    gpu.call("mnv_reduce_max_row", dx.p, do.p, 5, 3)
    np.testing.assert_array_equal(gpu.down(do, 5), [10, 11, 12, 13, 14])
    gpu.call("mnv_reduce_sum_col", dx.p, do.p, 5, 3)
    np.testing.assert_array_equal(gpu.down(do, 3), [10, 35, 60])
    gpu.call("mnv_reduce_sum_row", dx.p, do.p, 5, 3)
    np.testing.assert_array_equal(gpu.down(do, 5), [15, 18, 21, 24, 27])
    gpu.call("mnv_maxindex_col", dx.p, do.p, 5, 3)
    np.testing.assert_array_equal(gpu.down(do, 3), [4, 4, 4])
    gpu.call("mnv_maxindex_row", dx.p, do.p, 5, 3)
    np.testing.assert_array_equal(gpu.down(do, 5), [2, 2, 2, 2, 2])


SHAPES = [(1, 1), (1, 9), (9, 1), (5, 3), (10, 256), (1000, 256), (1000, 37), (4096, 256),
          (2050, 130), (64, 3000), (8192, 512), (515, 8192)]


@pytest.mark.parametrize("m,n", SHAPES)
def test_reductions(gpu, ora, m, n):
    x = _rand(m * n, 20)
    dx = gpu.up(x)
    dcol, drow = gpu.empty(n), gpu.empty(m)
    say("reduce", m, n)
    gpu.call("mnv_reduce_max_col", dx.p, dcol.p, m, n)
    assert_bits_equal(gpu.down(dcol), ora.reduction(ora.MAX, x, [m, n], [0]), "max_col")
    gpu.call("mnv_reduce_max_row", dx.p, drow.p, m, n)
    assert_bits_equal(gpu.down(drow), ora.reduction(ora.MAX, x, [m, n], [1]), "max_row")
    gpu.call("mnv_maxindex_col", dx.p, dcol.p, m, n)
    assert_bits_equal(gpu.down(dcol), ora.maxindex(x, [m, n], 0), "maxindex_col")
    gpu.call("mnv_maxindex_row", dx.p, drow.p, m, n)
    assert_bits_equal(gpu.down(drow), ora.maxindex(x, [m, n], 1), "maxindex_row")
    gpu.call("mnv_reduce_sum_col", dx.p, dcol.p, m, n)
    ref = ora.reduction(ora.SUM, x, [m, n], [0])
    x64 = x.reshape(n, m).astype(np.float64)
    assert normwise(gpu.down(dcol), ref) <= TOL
    assert normwise(gpu.down(dcol), x64.sum(axis=1)) <= TOL
    gpu.call("mnv_reduce_sum_row", dx.p, drow.p, m, n)
    ref = ora.reduction(ora.SUM, x, [m, n], [1])
    assert normwise(gpu.down(drow), ref) <= TOL
    assert normwise(gpu.down(drow), x64.sum(axis=0)) <= TOL


@pytest.mark.parametrize("m,n", [(8, 4), (1024, 64), (4100, 67), (300, 5000)])
def test_max_and_argmax_with_ties_nan_and_signed_zero(gpu, ora, m, n):
    rng = np.random.default_rng(21)
    x = rng.integers(-2, 3, size=m * n).astype(np.float32)  # heavy ties
    x[x == 0] = np.where(rng.random(np.count_nonzero(x == 0)) < 0.5, 0.0, -0.0)
    x[rng.random(m * n) < 0.05] = np.nan
    a = x.reshape(n, m)
    a[0, :] = np.nan           # a whole column of NaN; NaN first in every row
    if n > 2:
        a[1, 0] = np.nan       # NaN first in a column whose rest is finite
        a[2, :] = -np.inf      # all -inf column
    x = a.ravel().copy()
    dx, dcol, drow = gpu.up(x), gpu.empty(n), gpu.empty(m)
    for name, out, ref in (
            ("mnv_reduce_max_col", dcol, ora.reduction(ora.MAX, x, [m, n], [0])),
            ("mnv_reduce_max_row", drow, ora.reduction(ora.MAX, x, [m, n], [1])),
            ("mnv_maxindex_col", dcol, ora.maxindex(x, [m, n], 0)),
            ("mnv_maxindex_row", drow, ora.maxindex(x, [m, n], 1))):
        say(name, m, n)
        gpu.call(name, dx.p, out.p, m, n)
        assert_bits_equal(gpu.down(out), ref, name)


def test_max_and_argmax_full_size(gpu, ora):
    m = n = 8192
    x = _rand(m * n, 22)
    dx, dcol, drow = gpu.up(x), gpu.empty(n), gpu.empty(m)
    a = x.reshape(n, m)
    gpu.call("mnv_reduce_max_col", dx.p, dcol.p, m, n)
    assert_bits_equal(gpu.down(dcol), a.max(axis=1), "max_col 8192")
    gpu.call("mnv_reduce_max_row", dx.p, drow.p, m, n)
    assert_bits_equal(gpu.down(drow), a.max(axis=0), "max_row 8192")
    gpu.call("mnv_maxindex_col", dx.p, dcol.p, m, n)
    assert_bits_equal(gpu.down(dcol), ora.maxindex(x, [m, n], 0), "maxindex_col 8192")
    gpu.call("mnv_maxindex_row", dx.p, drow.p, m, n)
    assert_bits_equal(gpu.down(drow), a.argmax(axis=0).astype(np.float32), "maxindex_row 8192")
    gpu.call("mnv_reduce_sum_col", dx.p, dcol.p, m, n)
    assert normwise(gpu.down(dcol), a.astype(np.float64).sum(axis=1)) <= TOL
    gpu.call("mnv_reduce_sum_row", dx.p, drow.p, m, n)
    assert normwise(gpu.down(drow), a.astype(np.float64).sum(axis=0)) <= TOL


SOFTMAX = [(1, 1), (10, 256), (1000, 256), (7, 33), (256, 100), (2048, 64), (2052, 7), (4096, 16),
           (4100, 9), (8192, 48), (8193, 5), (9000, 3), (40000, 2)]


@pytest.mark.parametrize("length,lines", SOFTMAX)
def test_softmax_instance(gpu, ora, length, lines):
    x = _rand(length * lines, 23) * 4
    dy = _rand(length * lines, 24)
    dx, dout = gpu.up(x), gpu.empty(x.size)
    say("softmax instance", length, lines)
    gpu.call("mnv_softmax_instance_fwd", dx.p, dout.p, lines, length, 1, 1)
    y = gpu.down(dout)
    ref = ora.softmax_instance_fwd(x, lines, length, 1, 1)
    assert normwise(y, ref) <= TOL
    assert np.max(np.abs(y.reshape(lines, length).astype(np.float64).sum(axis=1) - 1)) < 1e-4
    # {W,H,C,N} with H, W > 1 is the same contiguous line
    if length % 6 == 0:
        gpu.call("mnv_softmax_instance_fwd", dx.p, dout.p, lines, length // 6, 2, 3)
        assert_bits_equal(gpu.down(dout), y, "instance chw")
    gpu.call("mnv_softmax_channel_fwd", dx.p, dout.p, lines, length, 1, 1)
    assert_bits_equal(gpu.down(dout), y, "channel with H=W=1 equals instance")
    dyd, dtop = gpu.up(dy), gpu.up(ref)
    gpu.call("mnv_softmax_instance_bwd", dyd.p, dtop.p, dout.p, lines, length, 1, 1)
    assert normwise(gpu.down(dout), ora.softmax_instance_bwd(dy, ref, lines, length, 1, 1)) <= TOL


@pytest.mark.parametrize("n,c,h,w", [
    (2, 5, 3, 4), (3, 10, 1, 7), (4, 21, 13, 13), (1, 2, 1, 2),
    (2, 64, 9, 15),      # the last channel count of the 64-position x 4-group kernel, ragged positions
    (3, 65, 7, 11),      # the first of the 32 x 32 kernel
    (2, 512, 5, 13),     # all channels in registers, forward and backward
    (1, 1000, 6, 7),     # in registers forward, re-read backward
    (1, 1024, 3, 33),
    (2, 1500, 2, 17),    # re-read in both passes
    (1, 1024, 256, 256),  # the 8192 x 8192-element case of the bandwidth table
])
def test_softmax_channel(gpu, ora, n, c, h, w):
    x = _rand(n * c * h * w, 25) * 3
    dy = _rand(x.size, 26)
    dx, dout = gpu.up(x), gpu.empty(x.size)
    gpu.call("mnv_softmax_channel_fwd", dx.p, dout.p, n, c, h, w)
    ref = ora.softmax_channel_fwd(x, n, c, h, w)
    assert normwise(gpu.down(dout), ref) <= TOL
    dyd, dtop = gpu.up(dy), gpu.up(ref)
    gpu.call("mnv_softmax_channel_bwd", dyd.p, dtop.p, dout.p, n, c, h, w)
    assert normwise(gpu.down(dout), ora.softmax_channel_bwd(dy, ref, n, c, h, w)) <= TOL


@pytest.mark.parametrize("m,n", [(1, 1), (3, 4), (64, 64), (65, 63), (1000, 37), (256, 784),
                                 (4096, 9216), (10, 256), (2052, 1500), (1500, 2052),
                                 (132, 16388),
                                 # rows of the result off the 64-byte grid (shifted runs): the last
                                 # tile reaching past n, both tile sizes, the benchmark's ragged shape
                                 (256, 8312), (64, 252), (68, 200), (8000, 8200)])
def test_transpose_bit_exact(gpu, ora, m, n):
    x = _rand(m * n, 27)       # a is {m,n}
    dx, dout = gpu.up(x), gpu.empty(m * n)
    say("transpose", m, n)
    gpu.call("mnv_transpose", dx.p, dout.p, m, n)
    # oracle: in{n_o,m_o} -> out{m_o,n_o}; here in = {m,n} so m_o = n, n_o = m
    assert_bits_equal(gpu.down(dout), ora.transpose(x, n, m), "transpose")
    # involution: transposing back restores the input
    dback = gpu.empty(m * n)
    gpu.call("mnv_transpose", dout.p, dback.p, n, m)
    assert_bits_equal(gpu.down(dback), x, "transpose twice")


@pytest.mark.parametrize("off", [4, 8, 12])
def test_transpose_into_a_result_off_the_64_byte_grid(gpu, off):
    """n % 16 == 0 but c starts `off` floats past a 64-byte boundary: shifted runs again, and
    nothing may be written in front of or behind the result."""
    m, n = 260, 2048
    x = _rand(m * n, 28)
    dx = gpu.up(x)
    dout = gpu.up(np.full(m * n + off + 20, np.nan, np.float32))
    say("transpose into offset", off)
    gpu.call("mnv_transpose", dx.p, dout.offset(off), m, n)
    got = gpu.down(dout)
    assert_bits_equal(got[off:off + m * n], np.ascontiguousarray(x.reshape(n, m).T).ravel(), "transpose")
    assert np.isnan(got[:off]).all() and np.isnan(got[off + m * n:]).all(), "wrote outside the result"


def _random_extents(count, seed, hi_m, hi_n, limit):
    """Seeded (m, n) pairs: half of the extents from the values the kernels branch on (vector
    width, wavefront, workgroup and tile sizes and their neighbours), half anywhere below hi."""
    rng = np.random.default_rng(seed)
    edge = [1, 2, 3, 4, 5, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513,
            1023, 1024, 1025, 2047, 2048, 2052, 4095, 4096, 4100]
    out = []
    while len(out) < count:
        m = int(rng.choice(edge)) if rng.random() < 0.5 else int(rng.integers(1, hi_m))
        n = int(rng.choice(edge)) if rng.random() < 0.5 else int(rng.integers(1, hi_n))
        if m * n <= limit:
            out.append((m, n))
    return out


@pytest.mark.parametrize("m,n", _random_extents(40, 5, 5000, 5000, 3_000_000))
def test_reductions_random_extents(gpu, ora, m, n):
    test_reductions(gpu, ora, m, n)


@pytest.mark.parametrize("length,lines", _random_extents(40, 6, 9000, 600, 2_000_000))
def test_softmax_instance_random_extents(gpu, ora, length, lines):
    test_softmax_instance(gpu, ora, length, lines)


@pytest.mark.parametrize("m,n", _random_extents(40, 7, 5000, 5000, 3_000_000))
def test_transpose_random_extents(gpu, ora, m, n):
    test_transpose_bit_exact(gpu, ora, m, n)


def test_large_operand_paths_8192x8192(gpu):
    """Inputs of 256 MB and more take the variants that read past the caches: softmax,
    transpose and the broadcast add at the size of the bandwidth benchmark."""
    m = n = 8192
    x = _rand(m * n, 23)
    dx, dz = gpu.up(x), gpu.empty(m * n)
    say("softmax 8192 lines of 8192")
    gpu.call("mnv_softmax_instance_fwd", dx.p, dz.p, n, m, 1, 1)  # lines of m contiguous floats
    y = gpu.down(dz).reshape(n, m)
    assert np.max(np.abs(y.astype(np.float64).sum(axis=1) - 1.0)) <= 1e-5
    for line in (0, 1, 4095, 8191):
        v = x.reshape(n, m)[line].astype(np.float64)
        ref = np.exp(v - v.max())
        ref /= ref.sum()
        assert normwise(y[line], ref) <= TOL
    say("transpose 8192 x 8192")
    gpu.call("mnv_transpose", dx.p, dz.p, m, n)
    assert_bits_equal(gpu.down(dz), np.ascontiguousarray(x.reshape(n, m).T).ravel(), "transpose 8192")
    say("broadcast add 8192 x 8192")
    vec = _rand(m, 24)
    dv = gpu.up(vec)
    gpu.call("mnv_norm_add_col", dx.p, dv.p, dz.p, m, n)   # res[r + c*m] = x[r + c*m] + vec[c]
    assert_bits_equal(gpu.down(dz), (x.reshape(n, m) + vec[:, None]).ravel(), "norm_add_col 8192")
    gpu.call("mnv_norm_add_row", dx.p, dv.p, dz.p, m, n)   # res[r + c*m] = x[r + c*m] + vec[r]
    assert_bits_equal(gpu.down(dz), (x.reshape(n, m) + vec[None, :]).ravel(), "norm_add_row 8192")
