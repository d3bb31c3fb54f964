"""mnv_sgemm_nn_static, the entry point that allocates nothing: its split-k partial sums
live in a fixed device array of the library instead of a caller's workspace.  Two calls in a
row through the C ABI, the second on a smaller problem (so that it finds the first call's
partial sums in the array), each bit-identical to mnv_sgemm_nn with a workspace of the same
size and within 1e-4 of an fp64 product; sizes beyond the array are refused."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, TOL, assert_bits_equal, normwise, say

pytestmark = pytest.mark.gpu
SCRATCH_BYTES = 32 << 20  # MNV_SGEMM_STATIC_SCRATCH_BYTES


def _rand(n, seed):
    return np.random.default_rng(seed).standard_normal(n).astype(np.float32)


def test_sgemm_static_matches_workspace_entry_point():
    gpu = Gpu()
    L = gpu.L
    ws = gpu.empty(SCRATCH_BYTES // 4)
    for (m, n, k, seed) in ((1000, 256, 4096, 70), (250, 60, 2050, 71), (1000, 256, 4096, 72)):
        a, b = _rand(m * k, seed), _rand(k * n, seed + 100)
        da, db = gpu.up(a), gpu.up(b)
        want_d = gpu.up(np.full(m * n, np.nan, np.float32))
        got_d = gpu.up(np.full(m * n, np.nan, np.float32))
        assert L.mnv_sgemm_nn_workspace_bytes(m, n, k) > 0, "the case must split its k range"
        say("mnv_sgemm_nn with a workspace", m, n, k)
        gpu.call("mnv_sgemm_nn", da.p, db.p, want_d.p, m, n, k, ws.p, ctypes.c_size_t(SCRATCH_BYTES))
        say("mnv_sgemm_nn_static", m, n, k)
        gpu.call("mnv_sgemm_nn_static", da.p, db.p, got_d.p, m, n, k)
        got, want = gpu.down(got_d), gpu.down(want_d)
        assert_bits_equal(got, want, "static scratch vs workspace %dx%dx%d" % (m, n, k))
        ref = a.reshape(k, m).T.astype(np.float64) @ b.reshape(n, k).T.astype(np.float64)
        assert normwise(got.reshape(n, m).T, ref) <= TOL
    # limits: an output whose two k ranges do not fit the array, and bad arguments
    d = gpu.empty(16)
    assert L.mnv_sgemm_nn_static(d.p, d.p, d.p, 4096, 4096, 16, gpu.dev.stream) == -3
    assert L.mnv_sgemm_nn_static(None, d.p, d.p, 4, 4, 4, gpu.dev.stream) == -1
    assert L.mnv_sgemm_nn_static(d.p, d.p, d.p, 0, 4, 4, gpu.dev.stream) == 0
    assert b"maximum" in L.mnv_error_string(-3)
