"""GPU parity of the minimal-filtering paths of the 3 x 3 unit-stride convolutions (forward
and data gradient by F(m x m, 3 x 3), filter gradient by F(3 x 3, m x m), m = 2, 4 and 5; 5 x 5
filters on 8 x 8 tiles), through the C ABI: against the CPU oracle's direct
sums on geometries that exercise odd and even extents, every padding, ragged tile counts and
channel counts off the tile width; in groups of images under a small workspace (same bits as
in one group); with the fused epilogues (same bits as the operator chain); and the switch
that selects the path."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, assert_bits_equal, normwise, say
from test_gpu_conv import Conv, _rand

pytestmark = pytest.mark.gpu
# The transforms are short sums with small constants: against the direct sum a few 1e-6 of the
# output's norm in fp32 with 2 x 2 tiles, up to about 6e-6 with 4 x 4 tiles (measured on the
# batch-256 layers); the bound of the convolutions is 1e-4
TIGHT = 2e-5
# 7 x 7 tiles (5 x 5 outputs under 3 x 3 filters) and 8 x 8 tiles (4 x 4 outputs under 5 x 5
# filters): seven and eight points make the transforms less well conditioned; up to 2.6e-5
# measured on the batch-256 layers
TIGHT5 = 5e-5
F2, F4, F5 = 3, 4, 5   # modes that pin the tile size (2: the library picks it); 5 x 5 filters run with 4
POINTS = {F2: 4, F4: 6, F5: 7}
BOUND = {F2: TIGHT, F4: TIGHT, F5: TIGHT5}


@pytest.fixture(scope="module")
def gpu():
    return Gpu()


class mode:
    """The path switch set for a block, the previous mode restored after it."""

    def __init__(self, gpu, m):
        self.L, self.m = gpu.L, m

    def __enter__(self):
        self.prev = self.L.mnv_conv_winograd_mode(self.m)

    def __exit__(self, *exc):
        self.L.mnv_conv_winograd_mode(self.prev)


GEOMS = [
    # N, C, K, H, W, ph, pw
    (2, 16, 16, 6, 6, 1, 1),        # even outputs, one tile row of the product
    (3, 32, 48, 13, 13, 1, 1),      # odd outputs: the last tile row and column are half empty
    (2, 16, 128, 8, 8, 0, 0),       # no padding
    (2, 16, 16, 5, 6, 2, 2),        # full padding (the data gradient then has none)
    (1, 16, 32, 3, 3, 0, 0),        # a single output per plane
    (2, 48, 20, 9, 11, 1, 0),       # unequal paddings; 20 output channels (data gradient: direct)
    (5, 64, 144, 7, 7, 1, 1),       # 144 output channels in two 128-wide column tiles per point
    (1, 16, 16, 4, 3, 0, 1),        # tiles in all: 1, rounded up to 4
    (7, 32, 32, 10, 9, 2, 1),
    (4, 144, 160, 13, 13, 1, 1),    # 9 and 10 k-slabs
    (3, 16, 16, 21, 2, 1, 1),       # two-pixel-wide planes
    (2, 20, 24, 5, 6, 2, 2),        # channel counts off 16: only the filter gradient takes the path
    (9, 130, 40, 9, 9, 1, 1),       # 130 input channels: two row tiles in the filter gradient
]
GEOMS5 = [
    # N, C, K, H, W, ph, pw under 5 x 5 filters
    (2, 16, 16, 9, 9, 2, 2),        # one tile row of the product
    (3, 32, 48, 13, 12, 2, 2),      # odd and even outputs
    (2, 16, 128, 11, 11, 0, 0),     # no padding
    (2, 16, 16, 8, 7, 4, 4),        # full padding (the data gradient then has none)
    (1, 16, 32, 5, 5, 0, 0),        # a single output per plane
    (2, 48, 20, 9, 11, 1, 3),       # unequal paddings; 20 output channels (data gradient: direct)
    (3, 96, 144, 27, 27, 2, 2),     # the planes and input channels of the AlexNet shape's conv2
    (2, 20, 24, 7, 8, 2, 1),        # channel counts off 16: only the filter gradient takes the path
]


@pytest.mark.parametrize("p7", GEOMS5, ids=lambda p: "x".join(map(str, p)))
def test_winograd_5x5_passes_against_oracle(gpu, ora, p7):
    _passes_against_oracle(gpu, ora, p7, F4, 5, TIGHT5)


@pytest.mark.parametrize("tile", [F2, F4, F5], ids=["2x2", "4x4", "5x5"])
@pytest.mark.parametrize("p7", GEOMS, ids=lambda p: "x".join(map(str, p)))
def test_winograd_passes_against_oracle(gpu, ora, p7, tile):
    _passes_against_oracle(gpu, ora, p7, tile, 3, BOUND[tile])


def _passes_against_oracle(gpu, ora, p7, tile, R, TIGHT):
    N, C, K, H, W, ph, pw = p7
    p = (N, C, K, H, W, ph, pw, 1, 1, R, R)
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 80), _rand(K * C * R * R, 81, 0.2), _rand(K, 82)
    dy = _rand(N * K * cv.Ho * cv.Wo, 83)
    want_y, want_dx = ora.conv_fwd(x, w, b, *p), ora.conv_bwd_data(dy, w, *p)
    want_dw = ora.conv_bwd_filter(dy, x, *p)
    with mode(gpu, 0):
        direct_y, direct_dx, direct_dw = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
        direct_bare, direct_bare_dw = cv.fwd(x, w, b, False), cv.bwd_filter(dy, x, False)
        direct_bytes = gpu.L.mnv_conv_fwd_workspace_bytes(*p)
    with mode(gpu, tile):
        say("winograd bwd filter", p)
        dw = cv.bwd_filter(dy, x)
        assert normwise(dw, want_dw) <= TIGHT
        assert np.any(dw.view(np.uint32) != direct_dw.view(np.uint32))
        assert_bits_equal(cv.bwd_filter(dy, x), dw, "second call")
        assert_bits_equal(cv.bwd_filter(dy, x, False), direct_bare_dw, "no workspace: the direct kernels")
        if C % 16:
            assert_bits_equal(cv.fwd(x, w, b), direct_y, "bottom channel count off 16: the direct kernels")
            assert_bits_equal(cv.bwd_data(dy, w), direct_dx, "top channel count off 16")
            return
        say("winograd fwd", p)
        # the size query covers the transformed tensors, and the path really ran: its bits
        # are not those of the direct kernels
        al = 8 if R == 5 else POINTS[tile]
        assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) == max(direct_bytes, _wino_bytes(N, C, K, cv.Ho, cv.Wo, al))
        y = cv.fwd(x, w, b)
        assert normwise(y, want_y) <= TIGHT
        assert np.any(y.view(np.uint32) != direct_y.view(np.uint32))
        say("winograd bwd data", p)
        dx = cv.bwd_data(dy, w)
        assert normwise(dx, want_dx) <= TIGHT
        if K % 16 == 0:
            assert np.any(dx.view(np.uint32) != direct_dx.view(np.uint32))
        else:
            assert_bits_equal(dx, direct_dx, "top channel count off 16: the direct kernels")
        # without a workspace the direct kernels run
        assert_bits_equal(cv.fwd(x, w, b, False), direct_bare, "no workspace")


def test_winograd_needs_a_16_byte_aligned_workspace(gpu, ora):
    """The transformed tensors are moved in 16-byte vectors: a workspace that starts 4 bytes
    off runs the direct kernels (same bits as with the path switched off)."""
    p = (3, 32, 48, 9, 9, 1, 1, 1, 1, 3, 3)
    N, C, K, H, W = p[:5]
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 70), _rand(K * C * 9, 71, 0.2), _rand(K, 72)
    with mode(gpu, 0):
        direct = cv.fwd(x, w, b)
    with mode(gpu, 2):
        nbytes = gpu.L.mnv_conv_fwd_workspace_bytes(*p)
        ws = gpu.empty(nbytes // 4 + 64)
        dxb, dwb, dbb, top = gpu.up(x), gpu.up(w), gpu.up(b), gpu.empty(direct.size)
        say("winograd, workspace off the 16-byte grid", p)
        gpu.call("mnv_conv_fwd", dxb.p, dwb.p, dbb.p, top.p, *p, ws.offset(1),
                 ctypes.c_size_t(nbytes))
        assert_bits_equal(gpu.down(top), direct, "unaligned workspace")
        gpu.call("mnv_conv_fwd", dxb.p, dwb.p, dbb.p, top.p, *p, ws.p, ctypes.c_size_t(nbytes))
        assert np.any(gpu.down(top).view(np.uint32) != direct.view(np.uint32))


def _random_winograd_geometries(count, seed):
    """Seeded geometries for the forced path: both filter extents, every tile size, planes from
    one output to 40 x 40 (past what the transform kernels stage in LDS), paddings up to the
    filter's reach, channel counts around 16 and 128."""
    rng = np.random.default_rng(seed)
    menu = [16, 16, 32, 48, 64, 80, 128, 144]
    out = []
    while len(out) < count:
        R = int(rng.choice([3, 3, 5]))
        tile = F4 if R == 5 else int(rng.choice([F2, F4, F5]))
        N = int(rng.integers(1, 6))
        C, K = int(rng.choice(menu)), int(rng.choice(menu + [20, 130]))
        H, W = int(rng.integers(1, 41)), int(rng.integers(1, 41))
        ph, pw = int(rng.integers(0, R)), int(rng.integers(0, R))
        if H + 2 * ph < R or W + 2 * pw < R:
            continue
        Ho, Wo = H + 2 * ph - R + 1, W + 2 * pw - R + 1
        if N * C * K * Ho * Wo * R * R > 120e6:
            continue
        out.append((N, C, K, H, W, ph, pw, R, tile))
    return out


@pytest.mark.parametrize("q", _random_winograd_geometries(36, 7), ids=lambda q: "x".join(map(str, q)))
def test_winograd_random_geometries_against_oracle(gpu, ora, q):
    N, C, K, H, W, ph, pw, R, tile = q
    p = (N, C, K, H, W, ph, pw, 1, 1, R, R)
    cv = Conv(gpu, *p)
    bound = TIGHT5 if R == 5 else BOUND[tile]
    x, w, b = _rand(N * C * H * W, 60), _rand(K * C * R * R, 61, 0.2), _rand(K, 62)
    dy = _rand(N * K * cv.Ho * cv.Wo, 63)
    with mode(gpu, tile):
        say("winograd, random geometry", q)
        assert normwise(cv.fwd(x, w, b), ora.conv_fwd(x, w, b, *p)) <= bound
        assert normwise(cv.bwd_data(dy, w), ora.conv_bwd_data(dy, w, *p)) <= bound
        assert normwise(cv.bwd_filter(dy, x), ora.conv_bwd_filter(dy, x, *p)) <= bound


def _points(Ho, Wo):
    """Points per dimension the library picks by itself under 3 x 3 filters: a larger tile (4 x 4,
    then 5 x 5 outputs) when it takes at most 85% of the products of the best smaller one."""
    best, al = 16 * ((Ho + 1) // 2) * ((Wo + 1) // 2), 4
    six = 36 * ((Ho + 3) // 4) * ((Wo + 3) // 4)
    if six * 100 <= best * 85:
        best, al = six, 6
    if 49 * ((Ho + 4) // 5) * ((Wo + 4) // 5) * 100 <= best * 85:
        al = 7
    return al


def _wino_bytes(images, C, K, Ho, Wo, al=None):
    """The workspace the path wants for `images` images at once (U, V, M from 256-byte
    boundaries; tiles rounded up to 4, output channels to 128).  al = 8: 5 x 5 filters."""
    al = al or _points(Ho, Wo)
    m = {4: 2, 6: 4, 7: 5, 8: 4}[al]
    a256 = lambda v: (v + 255) // 256 * 256
    kp = (K + 127) // 128 * 128
    pp = (images * ((Ho + m - 1) // m) * ((Wo + m - 1) // m) + 3) // 4 * 4
    return a256(al * al * kp * C * 4) + a256(al * al * pp * C * 4) + a256(al * al * pp * kp * 4)


@pytest.mark.parametrize("tile", [F2, F4, F5], ids=["2x2", "4x4", "5x5"])
@pytest.mark.parametrize("N", [12, 13])
def test_winograd_in_groups_of_images_has_the_same_bits(gpu, N, tile):
    """A workspace that holds five images: 12 images run as three groups of four, 13 as five,
    five and three.  Every output element is the same sum in the same order."""
    C, K, H, W = 32, 64, 13, 13
    p = (N, C, K, H, W, 1, 1, 1, 1, 3, 3)
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 84), _rand(K * C * 9, 85, 0.2), _rand(K, 86)
    dy = _rand(N * K * H * W, 87)
    al = POINTS[tile]
    with mode(gpu, tile):
        assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) == _wino_bytes(N, C, K, H, W, al)
        whole_y, whole_dx = cv.fwd(x, w, b), cv.bwd_data(dy, w)
        small = _wino_bytes(5, C, K, H, W, al) + 1024
        assert small < _wino_bytes(N, C, K, H, W, al)
        ws = gpu.empty(small // 4 + 64)
        dxb, dwb, dbb, dyb = gpu.up(x), gpu.up(w), gpu.up(b), gpu.up(dy)
        top, bd = gpu.empty(whole_y.size), gpu.empty(whole_dx.size)
        say("winograd in groups, fwd", p)
        gpu.call("mnv_conv_fwd", dxb.p, dwb.p, dbb.p, top.p, *p, ws.p, ctypes.c_size_t(small))
        assert_bits_equal(gpu.down(top), whole_y, "forward in groups")
        say("winograd in groups, bwd data", p)
        small = _wino_bytes(5, K, C, H, W, al) + 1024
        gpu.call("mnv_conv_bwd_data", dyb.p, dwb.p, bd.p, *p, ws.p, ctypes.c_size_t(small))
        assert_bits_equal(gpu.down(bd), whole_dx, "data gradient in groups")
        # the filter gradient sums over the images: in groups the 16 products accumulate group
        # by group, the same sum in another order
        say("winograd in groups, bwd filter", p)
        whole_dw = cv.bwd_filter(dy, x)
        full = gpu.L.mnv_conv_bwd_filter_workspace_bytes(*p)
        small = full - (_wino_bytes(N, C, K, H, W, al) - _wino_bytes(5, C, K, H, W, al)) + 1024
        big = gpu.empty(small // 4 + 64)
        fd = gpu.up(np.full(K * C * 9, np.nan, np.float32))
        gpu.call("mnv_conv_bwd_filter", dxb.p, dyb.p, fd.p, *p, big.p, ctypes.c_size_t(small))
        got = gpu.down(fd)
        assert normwise(got, whole_dw.astype(np.float64)) <= 1e-5
        assert np.any(got.view(np.uint32) != whole_dw.view(np.uint32))


@pytest.mark.parametrize("tile", [F2, F4, F5], ids=["2x2", "4x4", "5x5"])
def test_winograd_fused_epilogues_have_the_bits_of_the_chain(gpu, tile):
    """conv + ReLU and data gradient + ReLU gradient in one call against the separate
    operators, both on the minimal-filtering path."""
    p = (6, 32, 48, 11, 12, 1, 1, 1, 1, 3, 3)
    N, C, K, H, W = p[:5]
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 88), _rand(K * C * 9, 89, 0.2), _rand(K, 90)
    dy = _rand(N * K * cv.Ho * cv.Wo, 91)
    with mode(gpu, tile):
        nbytes = gpu.L.mnv_conv_fwd_workspace_bytes(*p)
        nbytes = max(nbytes, gpu.L.mnv_conv_bwd_data_workspace_bytes(*p))
        ws = gpu.empty(nbytes // 4 + 64)
        dxb, dwb, dbb, dyb = gpu.up(x), gpu.up(w), gpu.up(b), gpu.up(dy)
        top, bd = gpu.empty(N * K * cv.Ho * cv.Wo), gpu.empty(x.size)
        say("winograd conv + relu", p)
        gpu.call("mnv_conv_fwd_relu", dxb.p, dwb.p, dbb.p, top.p, *p, ws.p, ctypes.c_size_t(nbytes))
        assert_bits_equal(gpu.down(top), np.maximum(cv.fwd(x, w, b), np.float32(0)), "conv + relu")
        say("winograd data gradient + relu gradient", p)
        gpu.call("mnv_conv_bwd_data_relu", dyb.p, dwb.p, dxb.p, bd.p, *p, ws.p, ctypes.c_size_t(nbytes))
        assert_bits_equal(gpu.down(bd), np.where(x > 0, cv.bwd_data(dy, w), np.float32(0)),
                          "data gradient + relu gradient")
        say("winograd filter gradient + update", p)
        nbytes = gpu.L.mnv_conv_bwd_filter_workspace_bytes(*p)
        ws = gpu.empty(nbytes // 4 + 64)
        scale = np.float32(0.0123)
        want = w - scale * cv.bwd_filter(dy, x)
        out = gpu.empty(w.size)
        gpu.call("mnv_conv_bwd_filter_sgd", dxb.p, dyb.p, dwb.p, ctypes.c_float(scale), out.p, *p, ws.p,
                 ctypes.c_size_t(nbytes))
        assert_bits_equal(gpu.down(out), want, "filter gradient + update")
        gpu.call("mnv_conv_bwd_filter_sgd", dxb.p, dyb.p, dwb.p, ctypes.c_float(scale), dwb.p, *p, ws.p,
                 ctypes.c_size_t(nbytes))
        assert_bits_equal(gpu.down(dwb), want, "filter gradient + update in place")


def _profile_read(gpu, kind):
    n, ms, gf = ctypes.c_int(), ctypes.c_double(), ctypes.c_double()
    assert gpu.L.mnv_conv_winograd_profile_read(kind, ctypes.byref(n), ctypes.byref(ms), ctypes.byref(gf)) == 0
    return n.value, ms.value, gf.value


def test_winograd_product_profile_counts_launches_and_flops(gpu):
    """The measurement aid brackets the products of a pass with events: one record per group
    of images, of the pass's kind, carrying 2 x points x Cout x Cin x tiles flops; results
    have the same bits with and without it; enabling drops earlier records, disabling keeps
    them readable."""
    N, C, K, H, W = 12, 32, 64, 13, 13
    p = (N, C, K, H, W, 1, 1, 1, 1, 3, 3)
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 60), _rand(K * C * 9, 61, 0.2), _rand(K, 62)
    dy = _rand(N * K * H * W, 63)
    points, tiles = 36, N * 4 * 4        # 4 x 4 outputs per tile on 13 x 13 planes
    with mode(gpu, F4):
        plain = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
        assert gpu.L.mnv_conv_winograd_profile(1) == 0
        try:
            assert _profile_read(gpu, 0) == (0, 0.0, 0.0) and _profile_read(gpu, 1) == (0, 0.0, 0.0)
            timed = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
            n0, ms0, gf0 = _profile_read(gpu, 0)
            n1, ms1, gf1 = _profile_read(gpu, 1)
            assert (n0, n1) == (2, 1) and ms0 > 0 and ms1 > 0
            assert gf0 == pytest.approx(2 * 2.0 * points * K * C * tiles / 1e9, rel=1e-12)
            assert gf1 == pytest.approx(2.0 * points * K * C * tiles / 1e9, rel=1e-12)
            for got, want, what in zip(timed, plain, ("forward", "data gradient", "filter gradient")):
                assert_bits_equal(got, want, what + " with the profile on")
            # a workspace of five images: three groups, a record each
            nbytes = _wino_bytes(5, C, K, H, W, POINTS[F4]) + 1024
            ws, dxb, dwb, dbb = gpu.empty(nbytes // 4 + 64), gpu.up(x), gpu.up(w), gpu.up(b)
            top = gpu.empty(N * K * H * W)
            assert gpu.L.mnv_conv_winograd_profile(1) == 0      # drops the three records
            assert _profile_read(gpu, 0)[0] == 0
            gpu.call("mnv_conv_fwd", dxb.p, dwb.p, dbb.p, top.p, *p, ws.p, ctypes.c_size_t(nbytes))
            n0, _, gf0 = _profile_read(gpu, 0)
            assert n0 == 3 and gf0 == pytest.approx(2.0 * points * K * C * tiles / 1e9, rel=1e-12)
            assert_bits_equal(gpu.down(top), plain[0], "forward in three groups")
        finally:
            assert gpu.L.mnv_conv_winograd_profile(0) == 0
        assert _profile_read(gpu, 0)[0] == 3          # still readable after switching off
        cv.fwd(x, w, b)
        assert _profile_read(gpu, 0)[0] == 3          # and nothing is recorded while it is off
        assert gpu.L.mnv_conv_winograd_profile(1) == 0 and gpu.L.mnv_conv_winograd_profile(0) == 0
        assert _profile_read(gpu, 0)[0] == 0


def test_winograd_is_taken_by_itself_where_it_pays(gpu):
    """In the initial mode a 3 x 3 layer whose multiplies outweigh the transformed tensors'
    traffic takes the path without being asked (256 -> 256 channels, 72 images of 13 x 13); the
    same layer with 128 channels, on 8 images, at stride 2 or under 7 x 7 filters does not."""
    assert gpu.L.mnv_conv_winograd_mode(-1) == 1
    p = (72, 256, 256, 13, 13, 1, 1, 1, 1, 3, 3)
    N, C, K, H, W = p[:5]
    cv = Conv(gpu, *p)
    x, w, b = _rand(N * C * H * W, 92), _rand(K * C * 9, 93, 0.05), _rand(K, 94)
    assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) == _wino_bytes(N, C, K, H, W)
    say("winograd in the initial mode", p)
    y = cv.fwd(x, w, b)
    with mode(gpu, 0):
        assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) < _wino_bytes(N, C, K, H, W)
        direct = cv.fwd(x, w, b)
    assert np.any(y.view(np.uint32) != direct.view(np.uint32))
    assert normwise(y, direct) <= TIGHT
    for q in [(72, 128, 128, 13, 13, 1, 1, 1, 1, 3, 3), (72, 256, 256, 13, 13, 1, 1, 2, 2, 3, 3),
              (72, 256, 256, 13, 13, 3, 3, 1, 1, 7, 7), (8, 256, 256, 13, 13, 1, 1, 1, 1, 3, 3)]:
        with mode(gpu, 0):
            want = gpu.L.mnv_conv_fwd_workspace_bytes(*q)
        assert gpu.L.mnv_conv_fwd_workspace_bytes(*q) == want, q


ALEX3 = [("conv3", 256, 384), ("conv4", 384, 384), ("conv5", 384, 256)]


def test_direct_and_winograd_agree_on_conv2_at_batch_256(gpu):
    """The 5 x 5 layer of the AlexNet shape at batch 256 (96 -> 256 channels on 27 x 27 planes,
    padding 2) on the direct kernels and by minimal filtering on 8 x 8 tiles, all three
    passes: two independent algorithms over the same 256 distinct images."""
    p = (256, 96, 256, 27, 27, 2, 2, 1, 1, 5, 5)
    N, C, K, H, W = p[:5]
    cv = Conv(gpu, *p)
    x, w, b = np.maximum(_rand(N * C * H * W, 95), 0), _rand(K * C * 25, 96, 0.05), _rand(K, 97)
    dy = _rand(N * K * H * W, 98)
    say("conv2 b256 both paths")
    with mode(gpu, 0):
        direct_y, direct_dx, direct_dw = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
    with mode(gpu, 1):
        assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) == _wino_bytes(N, C, K, H, W, 8)
        y, dx, dw = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
        assert np.any(y.view(np.uint32) != direct_y.view(np.uint32))
        errs = normwise(y, direct_y), normwise(dx, direct_dx), normwise(dw, direct_dw)
        say("conv2 b256, minimal filtering against direct:", errs)
        assert max(errs) <= TIGHT5


@pytest.mark.parametrize("case", ALEX3, ids=lambda c: c[0])
def test_direct_and_winograd_agree_at_batch_256(gpu, case):
    """The 13 x 13 layers of the AlexNet shape at batch 256 on both paths (two independent
    algorithms over the same 256 distinct images), as the host layer runs them (5 x 5 output
    tiles, the library's choice for 13 x 13 planes): with the whole-batch workspace and in
    groups under 128 MB; and the 2 x 2 and 4 x 4 tiles beside them."""
    name, C, K = case
    p = (256, C, K, 13, 13, 1, 1, 1, 1, 3, 3)
    N, H, W = 256, 13, 13
    cv = Conv(gpu, *p)
    x, w, b = np.maximum(_rand(N * C * H * W, 95), 0), _rand(K * C * 9, 96, 0.05), _rand(K, 97)
    dy = _rand(N * K * H * W, 98)
    say(name, "b256 both paths")
    with mode(gpu, 0):
        direct_y, direct_dx, direct_dw = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
    with mode(gpu, 1):
        assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) == _wino_bytes(N, C, K, H, W)
        # the filter gradient's 16 products as one equal-shares launch: as many workgroups as
        # the chip holds
        nbytes = gpu.L.mnv_conv_bwd_filter_workspace_bytes(*p)
        assert nbytes > _wino_bytes(N, C, K, H, W)
        tile, ranges, wgs = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        assert gpu.L.mnv_conv_bwd_filter_plan(*p, ctypes.c_size_t(nbytes), ctypes.byref(tile),
                                              ctypes.byref(ranges), ctypes.byref(wgs)) == 0
        assert (tile.value, ranges.value) == (128, 1) and wgs.value >= 512
        dw = cv.bwd_filter(dy, x)
        assert np.any(dw.view(np.uint32) != direct_dw.view(np.uint32))
        assert normwise(dw, direct_dw) <= TIGHT5
        y, dx = cv.fwd(x, w, b), cv.bwd_data(dy, w)
        assert np.any(y.view(np.uint32) != direct_y.view(np.uint32))
        say(name, "5 x 5 tiles against direct:", normwise(y, direct_y), normwise(dx, direct_dx), normwise(dw, direct_dw))
        assert normwise(y, direct_y) <= TIGHT5 and normwise(dx, direct_dx) <= TIGHT5
        small = 128 << 20
        ws = gpu.empty(small // 4)
        dxb, dwb, dbb, dyb = gpu.up(x), gpu.up(w), gpu.up(b), gpu.up(dy)
        top, bd = gpu.empty(y.size), gpu.empty(dx.size)
        gpu.call("mnv_conv_fwd", dxb.p, dwb.p, dbb.p, top.p, *p, ws.p, ctypes.c_size_t(small))
        assert_bits_equal(gpu.down(top), y, "forward in groups")
        gpu.call("mnv_conv_bwd_data", dyb.p, dwb.p, bd.p, *p, ws.p, ctypes.c_size_t(small))
        assert_bits_equal(gpu.down(bd), dx, "data gradient in groups")
    assert _points(13, 13) == 7
    for tile in (F2, F4):
        with mode(gpu, tile):
            assert gpu.L.mnv_conv_fwd_workspace_bytes(*p) == _wino_bytes(N, C, K, H, W, POINTS[tile])
            y2, dx2, dw2 = cv.fwd(x, w, b), cv.bwd_data(dy, w), cv.bwd_filter(dy, x)
            assert np.any(y2.view(np.uint32) != y.view(np.uint32))
            assert normwise(y2, direct_y) <= TIGHT and normwise(dx2, direct_dx) <= TIGHT
            assert normwise(dw2, direct_dw) <= TIGHT
