"""GPU parity of the implicit-GEMM convolutions and of pooling, through the C ABI:
the reference's golden vectors, the CPU oracle on small and AlexNet-layer shapes
(normwise <= 1e-4; bit-exact for max pooling values and gradient routing), and at
batch 256 the adjoint identities and sampled fp64 dot products."""
import ctypes
import json
import os

import numpy as np
import pytest

from gpu_util import Gpu, TOL, assert_bits_equal, normwise, say

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


@pytest.fixture
def direct(gpu):
    """The direct implicit-GEMM kernels for 3 x 3 layers too (tests that aim at one of their
    launch plans); the minimal-filtering path has tests of its own."""
    prev = gpu.L.mnv_conv_winograd_mode(0)
    yield
    gpu.L.mnv_conv_winograd_mode(prev)


def _rand(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def _out(H, R, s, p):
    return (H + 2 * p - R) // s + 1


class Conv:
    """Runs the three convolution passes of one geometry on the GPU."""

    def __init__(self, gpu, N, C, K, H, W, ph, pw, sv, sh, R, S):
        self.gpu, self.p = gpu, (N, C, K, H, W, ph, pw, sv, sh, R, S)
        self.Ho, self.Wo = _out(H, R, sv, ph), _out(W, S, sh, pw)

    def _ws(self, query, workspace):
        nbytes = getattr(self.gpu.L, query)(*self.p) if workspace else 0
        ws = self.gpu.empty(nbytes // 4 + 1) if nbytes else None
        return (ws.p if ws else None), ctypes.c_size_t(nbytes), ws

    def fwd(self, x, w, b, workspace=True):
        g, p = self.gpu, self.p
        N, C, K = p[0], p[1], p[2]
        dx, dw, db = g.up(x), g.up(w), g.up(b)
        dt = g.empty(N * K * self.Ho * self.Wo)
        wp, wb, keep = self._ws("mnv_conv_fwd_workspace_bytes", workspace)
        g.call("mnv_conv_fwd", dx.p, dw.p, db.p, dt.p, *p, wp, wb)
        return g.down(dt)

    def bwd_data(self, dy, w, workspace=True):
        g, p = self.gpu, self.p
        N, C, K, H, W = p[:5]
        ddy, dw = g.up(dy), g.up(w)
        dbd = g.up(np.full(N * C * H * W, np.nan, np.float32))  # every element must be written
        wp, wb, keep = self._ws("mnv_conv_bwd_data_workspace_bytes", workspace)
        g.call("mnv_conv_bwd_data", ddy.p, dw.p, dbd.p, *p, wp, wb)
        return g.down(dbd)

    def bwd_filter(self, dy, x, workspace=True):
        g, p = self.gpu, self.p
        N, C, K, H, W, ph, pw, sv, sh, R, S = p
        ddy, dx = g.up(dy), g.up(x)
        dfd = g.up(np.full(K * C * R * S, np.nan, np.float32))
        nbytes = g.L.mnv_conv_bwd_filter_workspace_bytes(*p) if workspace else 0
        ws = g.empty(nbytes // 4 + 1) if nbytes else None
        g.call("mnv_conv_bwd_filter", dx.p, ddy.p, dfd.p, *p, ws.p if ws else None,
               ctypes.c_size_t(nbytes))
        return g.down(dfd)

    def bwd_bias(self, dy, workspace=True):
        g, p = self.gpu, self.p
        ddy, db = g.up(dy), g.empty(p[2])
        nbytes = g.L.mnv_conv_bwd_bias_workspace_bytes(p[0], p[2]) if workspace else 0
        ws = g.empty(nbytes // 4 + 1) if nbytes else None
        g.call("mnv_conv_bwd_bias", ddy.p, db.p, p[0], p[2], self.Ho, self.Wo,
               ws.p if ws else None, ctypes.c_size_t(nbytes))
        return g.down(db)


@pytest.mark.parametrize("case", json.load(open(os.path.join(GOLD, "conv_forward.json"))),
                         ids=lambda c: c["name"])
def test_conv_forward_golden(gpu, case):
    W, H, C, N = case["input_size"]
    S, R, _, K = case["weight_size"]
    x = np.array(case["input"], np.float32)
    w = np.array(case["weight"], np.float32)
    b = np.array(case["bias"] or [0] * K, np.float32)
    cv = Conv(gpu, N, C, K, H, W, case["pad_height"], case["pad_width"], case["stride_vertical"],
              case["stride_horizontal"], R, S)
    got = cv.fwd(x, w, b)
    Wo, Ho, _, _ = case["correct_size"]
    idx = np.arange(got.size)
    want = np.array(case["correct_without_bias"], np.float32) + b[(idx // (Wo * Ho)) % K]
    assert np.max(np.abs(got - want)) < 1e-3   # tests/unittest_conv_forward.cpp:32,66
    assert np.max(np.abs(got - want)) < 2e-5


CASES = [
    # N, C, K, H, W, ph, pw, sv, sh, R, S
    (2, 3, 4, 7, 9, 0, 0, 1, 1, 3, 5),
    (2, 2, 3, 8, 7, 2, 1, 2, 3, 3, 2),      # strided, padded, ragged fit
    (1, 4, 2, 6, 6, 1, 1, 1, 1, 3, 3),
    (3, 5, 7, 11, 13, 2, 3, 1, 2, 5, 4),
    (1, 1, 1, 1, 1, 0, 0, 1, 1, 1, 1),
    (2, 1, 16, 28, 28, 0, 0, 1, 1, 5, 5),   # MNIST CNN layer 1
    (2, 16, 32, 12, 12, 0, 0, 1, 1, 5, 5),  # MNIST CNN layer 2
    (2, 16, 32, 12, 12, 2, 2, 1, 1, 5, 5),  # same with the reference app's padding
    (5, 130, 70, 9, 9, 1, 1, 1, 1, 3, 3),   # more than one tile in both GEMM dimensions
    (2, 8, 140, 20, 20, 1, 1, 2, 2, 3, 3),
    (3, 32, 48, 10, 11, 1, 2, 1, 1, 3, 5),  # channel counts that take the (tap, channel) order
    (2, 16, 16, 9, 9, 2, 2, 1, 1, 5, 5),
    (2, 48, 32, 12, 12, 1, 1, 2, 1, 3, 3),  # 16-multiple channels but a strided data gradient
    (8, 16, 96, 48, 48, 1, 1, 1, 1, 3, 3),  # 96 output channels on many tiles: 96-column tiles
    (8, 96, 16, 48, 48, 1, 1, 1, 1, 3, 3),  # 96 input channels: the same for the data gradient
    (4, 64, 96, 20, 20, 1, 1, 1, 1, 3, 3),  # 96-column tiles in the table-driven filter gradient
    (8, 4, 192, 46, 46, 0, 0, 1, 1, 3, 3),  # two 96-column tiles, channel-major reduction order
    (3, 20, 17, 13, 13, 1, 1, 1, 1, 3, 3),  # <= 32 channels either way: 128x32 tiles, ragged rows,
    (2, 24, 33, 15, 14, 0, 0, 1, 1, 4, 4),  #   and a reduction cut into k ranges on small tiles
]


@pytest.mark.parametrize("p", CASES)
def test_conv_all_passes_against_oracle(gpu, ora, p):
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 40), _rand(K * C * R * S, 41), _rand(K, 42)
    dy = _rand(N * K * cv.Ho * cv.Wo, 43)
    ref = ora.conv_fwd(x, w, b, *p)
    for ws in (True, False):
        say("conv fwd", p, ws)
        assert normwise(cv.fwd(x, w, b, ws), ref) <= TOL
    ref = ora.conv_bwd_data(dy, w, *p)
    for ws in (True, False):
        say("conv bwd data", p, ws)
        assert normwise(cv.bwd_data(dy, w, ws), ref) <= TOL
    ref = ora.conv_bwd_filter(dy, x, *p)
    for ws in (True, False):
        say("conv bwd filter", p, ws)
        assert normwise(cv.bwd_filter(dy, x, ws), ref) <= TOL
    ref = ora.conv_bwd_bias(dy, N, K, cv.Ho, cv.Wo)
    for ws in (True, False):
        say("conv bwd bias", p, ws)
        assert normwise(cv.bwd_bias(dy, ws), ref) <= TOL


def _random_geometries(count, seed):
    """Seeded geometries that mix what the launch plans branch on: channel counts below, at and
    off multiples of 16 / 96 / 128, unit and larger strides, padding up to the filter's reach,
    planes whose rows are not multiples of four."""
    rng = np.random.default_rng(seed)
    menu = [1, 2, 3, 5, 8, 16, 17, 24, 32, 33, 48, 64, 96, 100, 128, 130, 192]
    out = []
    while len(out) < count:
        N = int(rng.integers(1, 7))
        C, K = int(rng.choice(menu)), int(rng.choice(menu))
        H, W = int(rng.integers(4, 23)), int(rng.integers(4, 23))
        R, S = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        ph, pw = int(rng.integers(0, R)), int(rng.integers(0, S))
        sv, sh = int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2, 3]))
        if H + 2 * ph < R or W + 2 * pw < S:
            continue
        Ho, Wo = (H + 2 * ph - R) // sv + 1, (W + 2 * pw - S) // sh + 1
        if N * C * K * Ho * Wo * R * S > 150e6:
            continue
        out.append((N, C, K, H, W, ph, pw, sv, sh, R, S))
    return out


@pytest.mark.parametrize("p", _random_geometries(96, 2024), ids=lambda p: "x".join(map(str, p)))
def test_conv_random_geometries_against_oracle(gpu, ora, p):
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 50), _rand(K * C * R * S, 51), _rand(K, 52)
    dy = _rand(N * K * cv.Ho * cv.Wo, 53)
    say("conv, random geometry", p)
    assert normwise(cv.fwd(x, w, b), ora.conv_fwd(x, w, b, *p)) <= TOL
    assert normwise(cv.bwd_data(dy, w), ora.conv_bwd_data(dy, w, *p)) <= TOL
    assert normwise(cv.bwd_filter(dy, x), ora.conv_bwd_filter(dy, x, *p)) <= TOL
    assert normwise(cv.bwd_bias(dy), ora.conv_bwd_bias(dy, N, K, cv.Ho, cv.Wo)) <= TOL


@pytest.mark.parametrize("p", [(8, 16, 128, 127, 127, 1, 1, 1, 1, 3, 3),    # forward: 505 tiles of 256 x 128
                               (8, 128, 16, 127, 127, 1, 1, 1, 1, 3, 3)],   # the same for the data gradient
                         ids=["forward", "data gradient"])
def test_conv_on_256_row_tiles_against_oracle(gpu, ora, direct, p):
    """Outputs of about 2^24 elements whose 256 x 128 tiles fill two workgroup slots per CU:
    the (tap, channel) forward / data-gradient kernels then run eight wavefronts per
    workgroup.  Ragged last tile (8 x 127 x 127 positions)."""
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 70), _rand(K * C * R * S, 71), _rand(K, 72)
    dy = _rand(N * K * cv.Ho * cv.Wo, 73)
    say("conv on 256-row tiles", p)
    assert normwise(cv.fwd(x, w, b), ora.conv_fwd(x, w, b, *p)) <= TOL
    assert normwise(cv.bwd_data(dy, w), ora.conv_bwd_data(dy, w, *p)) <= TOL
    # the same geometry without a workspace runs the generic kernels on 128 x 128 tiles
    assert normwise(cv.fwd(x, w, b, False), cv.fwd(x, w, b).astype(np.float64)) <= 1e-5
    assert normwise(cv.bwd_data(dy, w, False), cv.bwd_data(dy, w).astype(np.float64)) <= 1e-5


def test_conv_with_a_cut_tail_against_oracle(gpu, ora, direct):
    """Launches of a few more large tiles than a multiple of the 256 CUs cut the tiles past
    that multiple into k ranges (partial tiles in the workspace, added by a second kernel):
    264 tiles forward, 526 tiles in the data gradient.  With and without a workspace (no
    workspace: no cut), against the oracle; the workspace query must ask for the partial
    tiles on top of the permuted filter."""
    p = (10, 32, 256, 41, 41, 1, 1, 1, 1, 3, 3)
    N, C, K, H, W = p[:5]
    cv = Conv(gpu, *p)
    assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) >= K * C * 9 * 4 + 8 * 2 * 128 * 128 * 4
    x, w, b = _rand(N * C * H * W, 50), _rand(K * C * 9, 51, 0.1), _rand(K, 52)
    ref = ora.conv_fwd(x, w, b, *p)
    for ws in (True, False):
        say("conv fwd, cut tail", p, ws)
        assert normwise(cv.fwd(x, w, b, ws), ref) <= TOL
    p = (20, 256, 32, 41, 41, 1, 1, 1, 1, 3, 3)
    N, C, K, H, W = p[:5]
    cv = Conv(gpu, *p)
    assert gpu.L.mnv_conv_bwd_data_workspace_bytes(*p) >= K * C * 9 * 4 + 14 * 2 * 128 * 128 * 4
    dy, w = _rand(N * K * H * W, 53), _rand(K * C * 9, 54, 0.1)
    ref = ora.conv_bwd_data(dy, w, *p)
    for ws in (True, False):
        say("conv bwd data, cut tail", p, ws)
        assert normwise(cv.bwd_data(dy, w, ws), ref) <= TOL


ALEXNET = [
    # name, N, C, K, H, W, ph, pw, sv, sh, R, S   (owl/apps/imagenet_alexnet/alexnet.py:9-32)
    ("conv1", 1, 3, 96, 227, 227, 0, 0, 4, 4, 11, 11),
    ("conv2", 1, 96, 256, 27, 27, 2, 2, 1, 1, 5, 5),
    ("conv3", 1, 256, 384, 13, 13, 1, 1, 1, 1, 3, 3),
    ("conv4", 1, 384, 384, 13, 13, 1, 1, 1, 1, 3, 3),
    ("conv5", 2, 384, 256, 13, 13, 1, 1, 1, 1, 3, 3),
]


@pytest.mark.parametrize("case", ALEXNET, ids=lambda c: c[0])
def test_conv_alexnet_layers_small_batch_against_oracle(gpu, ora, case):
    name, p = case[0], case[1:]
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    x, w = _rand(N * C * H * W, 44), _rand(K * C * R * S, 45, 0.01)
    b = _rand(K, 46, 0.1)
    dy = _rand(N * K * cv.Ho * cv.Wo, 47)
    say(name, "fwd")
    assert normwise(cv.fwd(x, w, b), ora.conv_fwd(x, w, b, *p)) <= TOL
    say(name, "bwd filter")
    assert normwise(cv.bwd_filter(dy, x), ora.conv_bwd_filter(dy, x, *p)) <= TOL
    say(name, "bwd data")
    assert normwise(cv.bwd_data(dy, w), ora.conv_bwd_data(dy, w, *p)) <= TOL


@pytest.mark.parametrize("case", [ALEXNET[1], ALEXNET[2], ALEXNET[3], ALEXNET[4], ALEXNET[0]],
                         ids=lambda c: c[0])
def test_conv_batch_256_properties(gpu, case):
    name, p = case[0], (256,) + case[2:]
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    x, w = _rand(N * C * H * W, 48), _rand(K * C * R * S, 49, 0.05)
    b = np.zeros(K, np.float32)
    dy = _rand(N * K * cv.Ho * cv.Wo, 50)
    say(name, "b256 fwd")
    y = cv.fwd(x, w, b)
    # sampled outputs against an fp64 dot product written from the definition
    X = x.reshape(N, C, H, W)
    Wt = w.reshape(K, C, R, S)[:, :, ::-1, ::-1].astype(np.float64)
    Y = y.reshape(N, K, cv.Ho, cv.Wo)
    rng = np.random.default_rng(51)
    worst = 0.0
    for _ in range(40):
        n, k = rng.integers(N), rng.integers(K)
        i, j = rng.integers(cv.Ho), rng.integers(cv.Wo)
        if _ < 8:  # borders, where padding and the last tile live
            n, i, j = (N - 1, cv.Ho - 1, cv.Wo - 1) if _ % 2 else (0, 0, 0)
        acc = 0.0
        for r in range(R):
            yy = i * sv - ph + r
            if not 0 <= yy < H:
                continue
            xs = np.arange(S) + j * sh - pw
            ok = (xs >= 0) & (xs < W)
            acc += float(np.sum(X[n, :, yy, xs[ok]].astype(np.float64).T * Wt[k, :, r, ok].T))
        worst = max(worst, abs(Y[n, k, i, j] - acc))
    assert worst <= TOL * np.max(np.abs(y))
    lhs = float(np.dot(y.astype(np.float64), dy.astype(np.float64)))
    scale = float(np.linalg.norm(y.astype(np.float64)) * np.linalg.norm(dy.astype(np.float64)))
    say(name, "b256 bwd filter")
    dw = cv.bwd_filter(dy, x)
    assert abs(float(np.dot(dw.astype(np.float64), w.astype(np.float64))) - lhs) <= 1e-5 * scale
    # sampled filter-gradient entries against fp64 sums over the 256 distinct images, written
    # from the definition (cuda_perform.cu:293-318 hands the same sum to cuDNN): corners of
    # the (k, c, tap) index space first, where tile edges, channel groups and padded taps
    # live, then random entries.  One scalar identity cannot see a wrong tap or an image
    # counted twice; one entry out of place fails here by its whole size.
    DY = dy.reshape(N, K, cv.Ho, cv.Wo)
    DW = dw.reshape(K, C, R, S)
    picks = [(k, c, r, s_) for k in (0, K - 1) for c in (0, C - 1) for r in (0, R - 1)
             for s_ in (0, S - 1)]
    picks += [(K // 2, C // 2, R // 2, S // 2), (127 % K, 15 % C, 0, S - 1), (128 % K, 16 % C, R - 1, 0)]
    while len(picks) < 72:
        picks.append((int(rng.integers(K)), int(rng.integers(C)), int(rng.integers(R)),
                      int(rng.integers(S))))
    worst, top = 0.0, float(np.max(np.abs(dw)))
    for (k, c, r, s_) in picks:
        rf, sf = R - 1 - r, S - 1 - s_          # the tap of the flipped filter
        i = np.arange(cv.Ho)
        j = np.arange(cv.Wo)
        i = i[(i * sv - ph + rf >= 0) & (i * sv - ph + rf < H)]
        j = j[(j * sh - pw + sf >= 0) & (j * sh - pw + sf < W)]
        xs = X[:, c][:, i * sv - ph + rf][:, :, j * sh - pw + sf].astype(np.float64)
        want = float(np.sum(xs * DY[:, k][:, i][:, :, j]))
        worst = max(worst, abs(float(DW[k, c, r, s_]) - want))
    assert worst <= TOL * top, "filter gradient entry off by %.3e of %.3e" % (worst, top)
    if name != "conv1":  # the network never asks for conv1's data gradient
        say(name, "b256 bwd data")
        dx = cv.bwd_data(dy, w)
        assert abs(float(np.dot(dx.astype(np.float64), x.astype(np.float64))) - lhs) <= 1e-5 * scale
        # sampled data-gradient entries (cuda_perform.cu:266-291), borders and corners included
        DX = dx.reshape(N, C, H, W)
        picks = [(n, c, y, x_) for n in (0, N - 1) for c in (0, C - 1) for y in (0, H - 1)
                 for x_ in (0, W - 1)]
        picks += [(N // 2, C // 2, H // 2, W // 2), (1, 1, 0, W // 2), (N - 2, C - 2, H - 1, 1)]
        while len(picks) < 72:
            picks.append((int(rng.integers(N)), int(rng.integers(C)), int(rng.integers(H)),
                          int(rng.integers(W))))
        worst, top = 0.0, float(np.max(np.abs(dx)))
        for (n, c, y, x_) in picks:
            want = 0.0
            for r in range(R):
                if (y + ph - r) % sv or not 0 <= (y + ph - r) // sv < cv.Ho:
                    continue
                for s_ in range(S):
                    if (x_ + pw - s_) % sh or not 0 <= (x_ + pw - s_) // sh < cv.Wo:
                        continue
                    want += float(np.dot(DY[n, :, (y + ph - r) // sv, (x_ + pw - s_) // sh].astype(np.float64),
                                         Wt[:, c, r, s_]))
            worst = max(worst, abs(float(DX[n, c, y, x_]) - want))
        assert worst <= TOL * top, "data gradient entry off by %.3e of %.3e" % (worst, top)
    db = cv.bwd_bias(dy)
    assert normwise(db, dy.reshape(N, K, -1).astype(np.float64).sum(axis=(0, 2))) <= TOL


def _filter_plan(gpu, p, nbytes):
    tile, ranges, wgs = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    rc = gpu.L.mnv_conv_bwd_filter_plan(*p, ctypes.c_size_t(nbytes), ctypes.byref(tile),
                                        ctypes.byref(ranges), ctypes.byref(wgs))
    assert rc == 0
    return tile.value, ranges.value, wgs.value


# Filter gradients whose launch is dealt to the chip in equal amounts of k-slabs per workgroup
# (few output tiles, a long reduction): every tile is cut into the same aligned k ranges, and
# what those leave goes to the workgroups that remain, in shares that cross tile boundaries.
# One case per way of fetching the gathered operand with remaining workgroups (True), and
# four whose tiles divide the workgroups' number or whose shares are too short to leave a
# rest (False): every tile is then cut evenly.
STREAMK = [
    ("one tap per tile", True, 5, 256, 1408, 13, 13, 1, 1, 1, 1, 3, 3),
    ("two taps per tile", True, 3, 96, 1792, 13, 13, 2, 2, 1, 1, 5, 5),
    ("a table row per row group", True, 7, 48, 1408, 13, 13, 2, 2, 1, 1, 5, 5),
    ("no padding", True, 17, 22, 1408, 17, 17, 0, 0, 1, 1, 5, 5),
    ("channels not in sixteens", True, 7, 24, 2816, 13, 13, 2, 2, 1, 1, 5, 5),
    ("96-column tile", True, 32, 1088, 192, 7, 7, 1, 1, 1, 1, 3, 3),
    ("strided, ragged tile edges", True, 5, 120, 1608, 23, 21, 1, 2, 2, 2, 3, 5),
    ("one tap per tile, even cuts", False, 84, 128, 128, 13, 13, 1, 1, 1, 1, 3, 3),
    ("two taps per tile, even cuts", False, 40, 96, 128, 13, 13, 2, 2, 1, 1, 5, 5),
    ("no padding, even cuts", False, 150, 22, 128, 17, 17, 0, 0, 1, 1, 5, 5),
    ("96-column tile, even cuts", False, 96, 128, 96, 13, 13, 1, 1, 1, 1, 3, 3),
]


@pytest.mark.parametrize("case", STREAMK, ids=lambda c: c[0])
def test_conv_bwd_filter_in_equal_shares_against_oracle(gpu, ora, direct, case):
    remaining, p = case[1], case[2:]
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    nbytes = gpu.L.mnv_conv_bwd_filter_workspace_bytes(*p)
    tile, ranges, wgs = _filter_plan(gpu, p, nbytes)
    tiles = ((C * R * S + 127) // 128) * ((K + (95 if K in (96, 192) else 127)) // (96 if K in (96, 192) else 128))
    say("filter gradient,", case[0], "tile", tile, "workgroups", wgs, "tiles", tiles)
    assert tile == 128 and ranges == 1 and wgs >= 256, "the case is meant to take the stream-k plan"
    # workgroups = tiles x aligned ranges + the remaining ones (fewer than the tiles)
    assert tiles < wgs and (wgs % tiles != 0) == remaining
    x, dy = _rand(N * C * H * W, 61), _rand(N * K * cv.Ho * cv.Wo, 62)
    got = cv.bwd_filter(dy, x)
    assert normwise(got, ora.conv_bwd_filter(dy, x, *p)) <= TOL
    # equal shares are added in a fixed order: identical bits on a second call
    assert_bits_equal(cv.bwd_filter(dy, x), got, "second call")
    # without a workspace the same problem runs in one k range per tile
    assert _filter_plan(gpu, p, 0)[1:] == (1, 0)
    assert normwise(cv.bwd_filter(dy, x, workspace=False), got.astype(np.float64)) <= 1e-5


def _random_streamk_geometries(count, seed):
    """Seeded mid-size geometries whose filter gradient takes the stream-k plan: hundreds of
    k-slabs per tile, a few to a few hundred tiles, every way of fetching the gathered operand."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        N = int(rng.integers(24, 100))
        C, K = int(rng.choice([48, 64, 96, 100, 128, 160, 256])), int(rng.choice([128, 192, 200, 256, 384]))
        H, W = int(rng.integers(8, 21)), int(rng.integers(8, 21))
        R = S = int(rng.choice([3, 5]))
        ph = pw = int(rng.choice([0, R // 2]))
        Ho, Wo = H + 2 * ph - R + 1, W + 2 * pw - S + 1
        bn = 96 if K in (96, 192) else 128
        tiles = ((C * R * S + 127) // 128) * ((K + bn - 1) // bn)
        if tiles * N * ((Ho * Wo + 15) // 16) < 8 * 1024:   # eight slabs for each of at most 1024 workgroups
            continue
        out.append((N, C, K, H, W, ph, pw, 1, 1, R, S))
    return out


@pytest.mark.parametrize("p", _random_streamk_geometries(40, 99), ids=lambda p: "x".join(map(str, p)))
def test_conv_bwd_filter_streamk_random_geometries_sampled_fp64(gpu, direct, p):
    """Beyond what the oracle reaches in seconds: 64 filter-gradient entries per geometry (the
    corners of the index space first) against fp64 sums written from the definition."""
    N, C, K, H, W, ph, pw, sv, sh, R, S = p
    cv = Conv(gpu, *p)
    tile, ranges, wgs = _filter_plan(gpu, p, gpu.L.mnv_conv_bwd_filter_workspace_bytes(*p))
    say("filter gradient, random stream-k geometry", p, "tile", tile, "k ranges", ranges, "workgroups", wgs)
    assert wgs > 0, "the geometry is meant to take the stream-k plan"
    x, dy = _rand(N * C * H * W, 80), _rand(N * K * cv.Ho * cv.Wo, 81)
    dw = cv.bwd_filter(dy, x)
    X, DY, DW = x.reshape(N, C, H, W), dy.reshape(N, K, cv.Ho, cv.Wo), dw.reshape(K, C, R, S)
    rng = np.random.default_rng(82)
    picks = [(k, c, r, s_) for k in (0, K - 1) for c in (0, C - 1) for r in (0, R - 1) for s_ in (0, S - 1)]
    while len(picks) < 64:
        picks.append((int(rng.integers(K)), int(rng.integers(C)), int(rng.integers(R)), int(rng.integers(S))))
    worst, top = 0.0, float(np.max(np.abs(dw)))
    for (k, c, r, s_) in picks:
        rf, sf = R - 1 - r, S - 1 - s_
        i, j = np.arange(cv.Ho), np.arange(cv.Wo)
        i = i[(i - ph + rf >= 0) & (i - ph + rf < H)]
        j = j[(j - pw + sf >= 0) & (j - pw + sf < W)]
        xs = X[:, c][:, i - ph + rf][:, :, j - pw + sf].astype(np.float64)
        worst = max(worst, abs(float(DW[k, c, r, s_]) - float(np.sum(xs * DY[:, k][:, i][:, :, j]))))
    assert worst <= TOL * top, "filter gradient entry off by %.3e of %.3e" % (worst, top)
    assert_bits_equal(cv.bwd_filter(dy, x), dw, "second call")


# ------------------------------------------------------------------- pooling

@pytest.mark.parametrize("case", json.load(open(os.path.join(GOLD, "pooling_forward.json"))),
                         ids=lambda c: c["name"])
def test_pooling_forward_golden(gpu, case):
    W, H, C, N = case["input_size"]
    Wo, Ho, _, _ = case["correct_size"]
    geo = (N, C, H, W, case["stride_vertical"], case["stride_horizontal"], case["height"],
           case["width"], case["pad_height"], case["pad_width"])
    assert gpu.L.mnv_pooled_size(H, case["height"], case["stride_vertical"], case["pad_height"]) == Ho
    assert gpu.L.mnv_pooled_size(W, case["width"], case["stride_horizontal"], case["pad_width"]) == Wo
    dx, dt = gpu.up(np.array(case["input"], np.float32)), gpu.empty(Wo * Ho * C * N)
    gpu.call("mnv_maxpool_fwd", dx.p, dt.p, *geo)
    np.testing.assert_array_equal(gpu.down(dt), np.array(case["correct"], np.float32))


POOL = [
    # N, C, H, W, sv, sh, kh, kw, ph, pw
    (2, 3, 7, 9, 2, 2, 3, 3, 0, 0),
    (1, 2, 6, 5, 2, 3, 3, 2, 1, 1),
    (2, 2, 8, 8, 2, 2, 2, 2, 0, 0),
    (1, 1, 5, 5, 1, 1, 3, 3, 1, 1),
    (2, 96, 55, 55, 2, 2, 3, 3, 0, 0),    # AlexNet pool1
    (2, 256, 27, 27, 2, 2, 3, 3, 0, 0),   # pool2
    (3, 256, 13, 13, 2, 2, 3, 3, 0, 0),   # pool5
    (4, 16, 24, 24, 2, 2, 2, 2, 0, 0),    # MNIST CNN pools
    (4, 32, 12, 12, 3, 3, 3, 3, 0, 0),
    (1, 3, 100, 95, 2, 2, 3, 3, 1, 1),    # planes too large for the LDS-staged kernels
    (70, 33, 5, 7, 1, 2, 2, 3, 1, 1),     # many tiny planes per workgroup, odd plane size
    (3, 5, 9, 11, 2, 2, 3, 3, 1, 1),      # padded 3x3/2 and 2x2/2: the 2x2-block gradient
    (3, 5, 8, 10, 2, 2, 2, 2, 1, 1),      #   path with blocks that start outside the plane
    (2, 7, 10, 9, 2, 2, 3, 3, 0, 0),      # even height: clipped last window
    (5000, 1, 6, 6, 2, 2, 3, 3, 0, 0),    # more groups than resident workgroups
]


@pytest.mark.parametrize("p", POOL)
@pytest.mark.parametrize("ties", [False, True])
def test_pooling_against_oracle(gpu, ora, p, ties):
    N, C, H, W, sv, sh, kh, kw, ph, pw = p
    rng = np.random.default_rng(52)
    if ties:   # relu-like data: many equal values, whole windows of zeros
        x = np.maximum(rng.integers(-3, 3, size=N * C * H * W), 0).astype(np.float32)
    else:
        x = rng.standard_normal(N * C * H * W).astype(np.float32)
    Ho, Wo = ora.pooled_size(H, kh, sv, ph), ora.pooled_size(W, kw, sh, pw)
    dy = rng.standard_normal(N * C * Ho * Wo).astype(np.float32)
    dx, dt = gpu.up(x), gpu.empty(dy.size)
    say("pool", p, "ties" if ties else "")
    gpu.call("mnv_maxpool_fwd", dx.p, dt.p, *p)
    top = gpu.down(dt)
    assert_bits_equal(top, ora.pool_fwd(ora.POOL_MAX, x, *p), "maxpool fwd")
    ddy, dbd = gpu.up(dy), gpu.up(np.full(x.size, np.nan, np.float32))
    gpu.call("mnv_maxpool_bwd", dx.p, dt.p, ddy.p, dbd.p, *p)
    ref, mask = ora.pool_bwd(ora.POOL_MAX, dy, top, x, *p, want_mask=True)
    assert_bits_equal(gpu.down(dbd), ref, "maxpool bwd (same accumulation order)")
    # routing mask: a gradient of all ones counts, per position, the windows it wins
    ones = gpu.up(np.ones(dy.size, np.float32))
    gpu.call("mnv_maxpool_bwd", dx.p, dt.p, ones.p, dbd.p, *p)
    counts = np.zeros(x.size, np.float32)
    plane = np.repeat(np.arange(N * C), Ho * Wo) * (H * W)
    np.add.at(counts, plane + mask.astype(np.int64), 1.0)
    assert_bits_equal(gpu.down(dbd), counts, "maxpool routing mask")
    gpu.call("mnv_avgpool_fwd", dx.p, dt.p, *p)
    avg = gpu.down(dt)
    assert normwise(avg, ora.pool_fwd(ora.POOL_AVG, x, *p)) <= TOL
    gpu.call("mnv_avgpool_bwd", dx.p, dt.p, ddy.p, dbd.p, *p)
    assert normwise(gpu.down(dbd), ora.pool_bwd(ora.POOL_AVG, dy, avg, x, *p)) <= TOL


def _random_pools(count, seed):
    """Seeded pooling geometries: windows of 1..4 with strides up to the window, padding below
    the window, planes from one row to 30, a few and many planes."""
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        N, C = int(rng.integers(1, 5)), int(rng.choice([1, 2, 3, 16, 33, 96]))
        H, W = int(rng.integers(1, 31)), int(rng.integers(1, 31))
        kh, kw = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        if rng.random() < 0.5:   # the square windows the fast kernels take
            kw = kh = int(rng.choice([2, 3]))
        sv, sh = int(rng.integers(1, kh + 1)), int(rng.integers(1, kw + 1))
        if rng.random() < 0.5:
            sv = sh = 2
        ph, pw = int(rng.integers(0, kh)), int(rng.integers(0, kw))
        if H + 2 * ph < kh or W + 2 * pw < kw:
            continue
        out.append((N, C, H, W, sv, sh, kh, kw, ph, pw))
    return out


@pytest.mark.parametrize("p", _random_pools(48, 11), ids=lambda p: "x".join(map(str, p)))
def test_pooling_random_geometries_against_oracle(gpu, ora, p):
    test_pooling_against_oracle(gpu, ora, p, True)
    test_pooling_against_oracle(gpu, ora, p, False)


def test_pooling_batch_256_properties(gpu):
    p = (256, 96, 55, 55, 2, 2, 3, 3, 0, 0)
    N, C, H, W = p[:4]
    x = _rand(N * C * H * W, 53)
    dx, dt = gpu.up(x), gpu.empty(N * C * 27 * 27)
    gpu.call("mnv_maxpool_fwd", dx.p, dt.p, *p)
    top = gpu.down(dt).reshape(N * C, 27, 27)
    X = x.reshape(N * C, H, W)
    want = np.full((N * C, 27, 27), -np.inf, np.float32)
    for r in range(3):
        for s in range(3):
            want = np.maximum(want, X[:, r:r + 53:2, s:s + 53:2])
    assert_bits_equal(top, want, "pool1 b256")
    dy = _rand(top.size, 54)
    ddy, dbd = gpu.up(dy), gpu.empty(x.size)
    gpu.call("mnv_maxpool_bwd", dx.p, dt.p, ddy.p, dbd.p, *p)
    g = gpu.down(dbd)
    # continuous data has no ties: every window routes to exactly one position
    assert abs(float(g.astype(np.float64).sum()) - float(dy.astype(np.float64).sum())) < 1e-2
    assert np.count_nonzero(g) <= dy.size


# ----------------------------------------------------------------------- LRN
LRN = [
    # N, C, H, W, local_size, alpha, beta
    (2, 8, 3, 5, 5, 1e-1, 0.75),
    (3, 7, 4, 4, 3, 1e-2, 0.5),
    (2, 9, 5, 3, 4, 2e-1, 0.75),      # even window: forward and backward windows differ
    (1, 3, 6, 6, 5, 1e-1, 0.75),      # fewer channels than the window
    (2, 4, 2, 2, 1, 1e-1, 0.75),
    (2, 96, 27, 27, 5, 1e-4, 0.75),   # AlexNet norm1 (after pool1) and its constants
    (2, 256, 13, 13, 5, 1e-4, 0.75),  # norm2
    (70, 5, 9, 7, 5, 1e-1, 0.75),     # image boundaries inside a wavefront
    (3, 20, 55, 55, 5, 1e-4, 0.75),   # odd planes: whole wavefronts re-cut their runs, others straddle planes
    (2, 33, 31, 33, 3, 1e-2, 0.75),   # every channel starts at a different offset from a 64-byte boundary
    (2, 24, 28, 28, 7, 1e-2, 0.75),   # planes that start on 64-byte boundaries
    (2, 24, 25, 23, 7, 1e-2, 0.75),   # window of 7 on odd planes: re-cut stores, segments of 8 / 16 channels
    (3, 5, 41, 37, 5, 1e-2, 0.75),    # fewer channels than a segment, seven wavefronts per plane
]


@pytest.mark.parametrize("p", LRN)
def test_lrn_against_oracle(gpu, ora, p):
    N, C, H, W, size, alpha, beta = p
    x = _rand(N * C * H * W, 60) * 3
    dy = _rand(x.size, 61)
    say("lrn", p)
    dx, ds, dt = gpu.up(x), gpu.up(np.full(x.size, np.nan, np.float32)), gpu.up(np.full(x.size, np.nan, np.float32))
    gpu.call("mnv_lrn_fwd", dx.p, ds.p, dt.p, size, ctypes.c_float(alpha), ctypes.c_float(beta), N, C, H, W)
    top, scale = ora.lrn_fwd(x, size, alpha, beta, N, C, H, W)
    assert normwise(gpu.down(ds), scale) <= 1e-6      # same operations in the same order
    assert normwise(gpu.down(dt), top) <= TOL
    # backward from the oracle's forward results, so that only the backward kernel is compared
    dtop, dsc, ddy = gpu.up(top), gpu.up(scale), gpu.up(dy)
    dbd = gpu.up(np.full(x.size, np.nan, np.float32))
    gpu.call("mnv_lrn_bwd", dx.p, dtop.p, dsc.p, ddy.p, dbd.p, size, ctypes.c_float(alpha),
             ctypes.c_float(beta), N, C, H, W)
    assert normwise(gpu.down(dbd), ora.lrn_bwd(x, top, scale, dy, size, alpha, beta, N, C, H, W)) <= TOL


@pytest.mark.parametrize("offset", [1, 5, 16])
def test_lrn_tensors_off_their_natural_alignment(gpu, ora, offset):
    """scale / top (and the inputs) `offset` floats into their allocations."""
    N, C, H, W, size, alpha, beta = 2, 12, 23, 23, 5, 1e-2, 0.75
    n = N * C * H * W
    x = _rand(n, 64) * 3
    dy = _rand(n, 65)
    pad = np.full(offset, np.nan, np.float32)
    say("lrn offset", offset)
    dx = gpu.up(np.concatenate([pad, x]))
    ds, dt = gpu.up(np.full(n + offset + 3, np.nan, np.float32)), gpu.up(np.full(n + offset + 7, np.nan, np.float32))
    f = ctypes.c_float
    gpu.call("mnv_lrn_fwd", dx.offset(offset), ds.offset(offset), dt.offset(offset), size, f(alpha), f(beta), N, C, H, W)
    top, scale = ora.lrn_fwd(x, size, alpha, beta, N, C, H, W)
    got_s, got_t = gpu.down(ds), gpu.down(dt)
    assert normwise(got_s[offset:offset + n], scale) <= 1e-6 and normwise(got_t[offset:offset + n], top) <= TOL
    assert np.isnan(got_s[:offset]).all() and np.isnan(got_s[offset + n:]).all(), "wrote outside scale"
    assert np.isnan(got_t[:offset]).all() and np.isnan(got_t[offset + n:]).all(), "wrote outside top"
    dtop, dsc, ddy = gpu.up(np.concatenate([pad, top])), gpu.up(np.concatenate([pad, scale])), gpu.up(np.concatenate([pad, dy]))
    dbd = gpu.up(np.full(n + offset + 5, np.nan, np.float32))
    gpu.call("mnv_lrn_bwd", dx.offset(offset), dtop.offset(offset), dsc.offset(offset), ddy.offset(offset),
             dbd.offset(offset), size, f(alpha), f(beta), N, C, H, W)
    got = gpu.down(dbd)
    assert normwise(got[offset:offset + n], ora.lrn_bwd(x, top, scale, dy, size, alpha, beta, N, C, H, W)) <= TOL
    assert np.isnan(got[:offset]).all() and np.isnan(got[offset + n:]).all(), "wrote outside bottom_diff"


def test_lrn_batch_256_properties(gpu):
    """AlexNet norm1 at batch 256: the closed form in fp64 on sampled positions."""
    N, C, H, W, size, alpha, beta = 256, 96, 27, 27, 5, 1e-4, 0.75
    x = _rand(N * C * H * W, 62) * 10
    dxb, ds, dt = gpu.up(x), gpu.empty(x.size), gpu.empty(x.size)
    gpu.call("mnv_lrn_fwd", dxb.p, ds.p, dt.p, size, ctypes.c_float(alpha), ctypes.c_float(beta), N, C, H, W)
    top = gpu.down(dt).reshape(N, C, H * W)
    X = x.reshape(N, C, H * W).astype(np.float64)
    rng = np.random.default_rng(63)
    worst = 0.0
    for _ in range(400):
        n, c, p = int(rng.integers(N)), int(rng.integers(C)), int(rng.integers(H * W))
        lo, hi = max(c - 2, 0), min(c + 2, C - 1)
        s = 1.0 + alpha / size * np.sum(X[n, lo:hi + 1, p] ** 2)
        worst = max(worst, abs(top[n, c, p] - X[n, c, p] * s ** (-beta)))
    assert worst <= TOL * np.max(np.abs(top))


def test_lrn_benchmark_shape_properties(gpu):
    """The shape the bandwidth table times (Caffe-style norm1 on conv1's output, batch 256: the
    re-cut, non-temporal kernels with short channel segments): forward and backward against
    the closed forms in fp64 on sampled positions, and every element written."""
    N, C, H, W, size, alpha, beta = 256, 96, 55, 55, 5, 1e-4, 0.75
    hw, n = H * W, N * C * H * W
    rng = np.random.default_rng(66)
    x = (rng.standard_normal(n, dtype=np.float32) * 10).astype(np.float32)
    dy = rng.standard_normal(n, dtype=np.float32)
    say("lrn at the benchmark shape")
    dx_, ds, dt = gpu.up(x), gpu.up(np.full(n, np.nan, np.float32)), gpu.up(np.full(n, np.nan, np.float32))
    f = ctypes.c_float
    gpu.call("mnv_lrn_fwd", dx_.p, ds.p, dt.p, size, f(alpha), f(beta), N, C, H, W)
    top, scale = gpu.down(dt), gpu.down(ds)
    assert np.isfinite(top).all() and np.isfinite(scale).all(), "an element was not written"
    ddy, dbd = gpu.up(dy), gpu.up(np.full(n, np.nan, np.float32))
    gpu.call("mnv_lrn_bwd", dx_.p, dt.p, ds.p, ddy.p, dbd.p, size, f(alpha), f(beta), N, C, H, W)
    bd = gpu.down(dbd)
    assert np.isfinite(bd).all(), "an element of the gradient was not written"
    X = x.reshape(N, C, hw).astype(np.float64)
    DY = dy.reshape(N, C, hw).astype(np.float64)
    T, S, B = top.reshape(N, C, hw), scale.reshape(N, C, hw), bd.reshape(N, C, hw)
    worst_t = worst_s = worst_b = 0.0
    picks = [(0, 0, 0), (N - 1, C - 1, hw - 1), (1, 0, hw - 1), (0, C - 1, 0), (7, 5, 239), (7, 5, 240),
             (7, 6, 241), (3, 95, 3024), (200, 47, 1008)]
    picks += [(int(rng.integers(N)), int(rng.integers(C)), int(rng.integers(hw))) for _ in range(600)]
    for nn, c, p in picks:
        lo, hi = max(c - 2, 0), min(c + 2, C - 1)
        col = X[nn, :, p]
        sc = 1.0 + alpha / size * np.array([np.sum(col[max(k - 2, 0):min(k + 2, C - 1) + 1] ** 2)
                                             for k in range(lo, hi + 1)])
        s_c = sc[c - lo]
        worst_s = max(worst_s, abs(S[nn, c, p] - s_c) / s_c)
        worst_t = max(worst_t, abs(T[nn, c, p] - col[c] * s_c ** (-beta)))
        # bottom_diff = dy * s^-beta - 2 alpha beta / size * x * sum_k dy_k * y_k / s_k over the window
        yk = col[lo:hi + 1] * sc ** (-beta)
        acc = np.sum(DY[nn, lo:hi + 1, p] * yk / sc)
        want = DY[nn, c, p] * s_c ** (-beta) - 2.0 * alpha * beta / size * col[c] * acc
        worst_b = max(worst_b, abs(B[nn, c, p] - want))
    assert worst_s <= 1e-6
    assert worst_t <= TOL * np.max(np.abs(top))
    assert worst_b <= TOL * np.max(np.abs(bd))
