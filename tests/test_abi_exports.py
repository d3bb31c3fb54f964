"""The C ABI library loads and exports every symbol that include/mnv_hip.h declares,
and the ctypes binding covers all of them (no compute calls: runs without a GPU)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mnv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mnv_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_a_sane_number_of_entry_points():
    names = _declared()
    assert len(names) >= 70
    for must in ("mnv_sgemm_nn", "mnv_conv_fwd", "mnv_conv_bwd_data", "mnv_conv_bwd_filter",
                 "mnv_conv_bwd_bias", "mnv_maxpool_bwd", "mnv_softmax_instance_fwd",
                 "mnv_maxindex_col", "mnv_norm_add_row", "mnv_reduce_sum_row"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from minerva_amd import capi
    assert os.path.exists(capi.LIB_PATH), "build the library first: python -m minerva_amd.build"
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [n for n in _declared() if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_covers_every_declared_symbol():
    from minerva_amd import capi
    declared = set(_declared())
    bound = set(capi.PROTOTYPES)
    assert declared == bound, (sorted(declared - bound), sorted(bound - declared))
    capi.load()  # attaches argtypes; raises if a symbol is absent


def test_pure_host_entry_points():
    from minerva_amd import capi
    L = capi.lib()
    # pooled-size rule of narray/convolution.cpp:107-114 (golden sizes of the reference tests)
    assert L.mnv_pooled_size(4, 3, 1, 0) == 2
    assert L.mnv_pooled_size(4, 3, 1, 1) == 4
    assert L.mnv_pooled_size(4, 3, 2, 1) == 3
    assert L.mnv_pooled_size(4, 4, 3, 2) == 2
    assert L.mnv_pooled_size(55, 3, 2, 0) == 27
    assert L.mnv_error_string(0) == b"ok"
    assert b"invalid" in L.mnv_error_string(-1)
    # workspace queries are pure arithmetic
    assert L.mnv_sgemm_nn_workspace_bytes(4096, 4096, 4096) == 0
    assert L.mnv_sgemm_nn_workspace_bytes(1000, 256, 4096) > 0
    assert L.mnv_conv_bwd_filter_workspace_bytes(256, 256, 384, 13, 13, 1, 1, 1, 1, 3, 3) > 0


def test_winograd_switch_and_size_queries():
    """The path switch is process-wide host state and the size queries follow it (pure
    arithmetic): the 384 -> 384 channel layer on 13 x 13 planes at batch 256 asks for its
    transformed tensors only while the path is on (49 values per 7 x 7 tile and channel on
    3 x 3 tiles per plane, 376 MB; 16 per 4 x 4 tile on 7 x 7 tiles, 597 MB, or 36 per 6 x 6 tile
    on 4 x 4 tiles, 474 MB, with the tile size pinned); the 5 x 5 layer (96 -> 256 channels on 27 x 27 planes) 64 values per 8 x 8 tile
    on 7 x 7 tiles per plane, 1137 MB, unless the tile is pinned to 2 x 2 outputs."""
    from minerva_amd import capi
    L = capi.lib()
    conv4 = (256, 384, 384, 13, 13, 1, 1, 1, 1, 3, 3)
    conv2 = (256, 96, 256, 27, 27, 2, 2, 1, 1, 5, 5)
    assert L.mnv_conv_winograd_mode(-1) == 1
    try:
        on = L.mnv_conv_fwd_workspace_bytes(*conv4)
        tiles = 256 * 3 * 3
        assert on == 49 * 384 * 384 * 4 + 2 * 49 * tiles * 384 * 4
        assert L.mnv_conv_bwd_data_workspace_bytes(*conv4) == on
        five = L.mnv_conv_fwd_workspace_bytes(*conv2)
        assert five == 64 * 256 * 96 * 4 + 64 * 256 * 49 * (96 + 256) * 4
        assert L.mnv_conv_winograd_mode(0) == 1
        assert L.mnv_conv_fwd_workspace_bytes(*conv4) < on // 4
        direct_five = L.mnv_conv_fwd_workspace_bytes(*conv2)
        assert direct_five < five // 4
        assert L.mnv_conv_winograd_mode(2) == 0
        assert L.mnv_conv_fwd_workspace_bytes(*conv4) == on
        assert L.mnv_conv_fwd_workspace_bytes(*conv2) == five
        assert L.mnv_conv_winograd_mode(3) == 2      # 2 x 2 output tiles only
        assert L.mnv_conv_fwd_workspace_bytes(*conv4) == 16 * 384 * 384 * 4 + 2 * 16 * 256 * 49 * 384 * 4
        assert L.mnv_conv_fwd_workspace_bytes(*conv2) == direct_five
        assert L.mnv_conv_winograd_mode(4) == 3      # 4 x 4 output tiles only
        assert L.mnv_conv_fwd_workspace_bytes(*conv4) == 36 * 384 * 384 * 4 + 2 * 36 * 256 * 16 * 384 * 4
        assert L.mnv_conv_fwd_workspace_bytes(*conv2) == five
        assert L.mnv_conv_winograd_mode(5) == 4      # 5 x 5 output tiles only
        assert L.mnv_conv_fwd_workspace_bytes(*conv4) == on
        assert L.mnv_conv_winograd_mode(7) == 5      # out of range: a query
    finally:
        L.mnv_conv_winograd_mode(1)


def _plan(m, n, k, workspace=True):
    import ctypes
    from minerva_amd import capi
    L = capi.lib()
    ws = L.mnv_sgemm_nn_workspace_bytes(m, n, k) if workspace else 0
    tile, ranges, groups = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    assert L.mnv_sgemm_nn_plan(m, n, k, ctypes.c_size_t(ws), ctypes.byref(tile), ctypes.byref(ranges),
                               ctypes.byref(groups)) == 0
    return tile.value, ranges.value, groups.value, ws


def test_sgemm_plans_of_the_benchmark_shapes():
    """The launch plan is host arithmetic on the extents alone.  Square and short-k products
    run one tile per workgroup without k ranges (the large square one on 256 x 128 tiles, which
    fill the chip's two-per-CU slots exactly); the skinny inner products of the AlexNet
    shape run as workgroups of four wavefront groups; the workspace the query asks for is
    exactly what the plan's partial results need; without a workspace nothing is split in
    memory."""
    assert _plan(4096, 4096, 4096)[:3] == (256, 1, 1)
    assert _plan(4096, 4096, 256)[:3] == (128, 1, 1)
    assert _plan(4096, 9216, 256)[:3] == (128, 1, 1)
    assert _plan(4096, 256, 9216)[:3] == (128, 4, 4)
    assert _plan(4096, 256, 4096)[:3] == (64, 1, 4)
    assert _plan(1000, 256, 4096)[:3] == (64, 4, 4)
    assert _plan(9216, 256, 4096)[2] == 1
    for (m, n, k) in [(4096, 256, 9216), (1000, 256, 4096), (9216, 256, 4096), (256, 256, 784),
                      (10, 256, 256), (4, 4, 4096), (130, 70, 1000)]:
        tile, ranges, groups, ws = _plan(m, n, k)
        assert tile in (64, 128) and groups in (1, 4) and 1 <= ranges <= 16
        assert ws == (ranges * m * n * 4 if ranges > 1 else 0)
        assert _plan(m, n, k, workspace=False)[1] == 1


def test_host_library_exports_every_declared_symbol():
    """include/mnv_host.h against libmnv_host.so (loading it needs no GPU either)."""
    from minerva_amd import capi, hostapi
    text = open(os.path.join(ROOT, "include", "mnv_host.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(mnvh_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 30
    assert os.path.exists(hostapi.LIB_PATH), "build the library first: python -m minerva_amd.build"
    capi.lib()  # libmnv_hip.so first, from the same directory
    lib = ctypes.CDLL(hostapi.LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_narray_front_end_has_the_names_of_the_reference_binding():
    """Every public name of the reference's Python binding that belongs to the operator path
    (owl/owl/__init__.py, owl/owl/libowl.pyx:51-444, owl/owl/elewise.py, owl/owl/conv.py)
    exists in minerva_amd.owl; importing it needs no GPU."""
    from minerva_amd import owl
    from minerva_amd.owl import conv, elewise
    module = ("has_cuda wait_for_all create_cpu_device create_gpu_device get_gpu_device_count "
              "set_device zeros ones randn randb from_numpy concat slice NArray").split()
    narray = ("mult exp ln sigm sigm_back relu relu_back tanh tanh_back conv_forward "
              "conv_backward_data conv_backward_filter conv_backward_bias softmax_forward "
              "softmax_backward activation_forward activation_backward pooling_forward "
              "pooling_backward lrn_forward lrn_backward sum max max_index count_zero trans "
              "reshape wait_for_eval shape zeros ones randn randb concat slice from_numpy "
              "to_numpy __add__ __sub__ __mul__ __truediv__ __iadd__ __isub__ __imul__ "
              "__itruediv__ __radd__ __rsub__ __rmul__ __rtruediv__").split()
    assert not [n for n in module if not hasattr(owl, n)]
    assert not [n for n in narray if not hasattr(owl.NArray, n)]
    assert not [n for n in "mult exp ln sigm relu tanh sigm_back relu_back tanh_back".split()
                if not hasattr(elewise, n)]
    assert not [n for n in "softmax Lrner Convolver Pooler soft_op pool_op".split()
                if not hasattr(conv, n)]
    assert conv.soft_op.instance != conv.soft_op.channel and conv.pool_op.max != conv.pool_op.avg
    for cls, methods in ((conv.Convolver, "ff bp weight_grad bias_grad"), (conv.Pooler, "ff bp"),
                         (conv.Lrner, "ff bp")):
        assert not [m for m in methods.split() if not hasattr(cls, m)]
