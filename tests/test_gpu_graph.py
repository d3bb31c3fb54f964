"""Recorded steps (HIP graphs): a replay must give bit for bit what the same operators
give when they are launched one by one.  Every recording is replayed several times, with
eager work, host copies and synchronisations between the replays, and every replay is
checked, not only the first."""
import ctypes

import numpy as np
import pytest

from gpu_util import Gpu, assert_bits_equal, net_batches, net_state, run_steps, say

pytestmark = pytest.mark.gpu


_batches, _state = net_batches, net_state


def _eager(kind, batch, variant, lr, params, batches):
    return run_steps(kind, batch, variant, lr, params, batches)


@pytest.mark.parametrize("kind,batch,variant", [("mlp", 256, 0), ("cnn", 64, 0), ("cnn", 32, 1),
                                                ("alexnet", 2, 0)])
def test_replay_equals_eager_steps(kind, batch, variant):
    from minerva_amd import hostapi
    lr = 0.05
    params, batches = _batches(kind, batch, 4)
    say("eager steps", kind, batch, variant)
    want = _eager(kind, batch, variant, lr, params, batches)

    say("record + replay", kind, batch, variant)
    r = hostapi.Runtime(0, sync_each_op=True)
    net = hostapi.Net(r, kind, batch, variant)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(*batches[0])
    ops_before = r.ops_issued()
    nodes = net.capture_step(lr)
    ops_per_step = (r.ops_issued() - ops_before) // 2  # the eager pass and the recording pass
    # one node per kernel: at least one per operator plus one copy per parameter
    assert nodes >= ops_per_step + len(net.params), (nodes, ops_per_step)
    # recording applied nothing
    for k, n in net.params.items():
        assert_bits_equal(net.read(k, n), params[k], "parameter %s after recording" % k)
    x = np.arange(1000, dtype=np.float32)
    for i, (d, l) in enumerate(batches):
        net.load_batch(d, l)  # in place: the recording reads these buffers
        net.replay(1)
        got = _state(net, l.size)
        for k in want[i]:
            assert_bits_equal(got[k], want[i][k], "%s after replay %d" % (k, i))
        # the program's own eager work between two replays
        y = r.op("arithmetic", [(x, [1000]), (x, [1000])], [0])[0]
        assert_bits_equal(y, x + x, "eager add between replays")
    net.close()
    r.close()


def test_back_to_back_replays_equal_eager_steps():
    """Several replays launched without waiting in between, on one resident batch."""
    from minerva_amd import hostapi
    kind, batch, lr, steps = "mlp", 128, 0.1, 5
    params, batches = _batches(kind, batch, 1)
    want = _eager(kind, batch, 0, lr, params, batches * steps)[-1]
    r = hostapi.Runtime(0, sync_each_op=False)
    net = hostapi.Net(r, kind, batch)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(*batches[0])
    net.capture_step(lr)
    say("back-to-back replays")
    net.replay(steps, sync_each_step=False)
    got = _state(net, batches[0][1].size)
    for k in want:
        assert_bits_equal(got[k], want[k], k)
    net.close()
    r.close()


def test_recording_rules():
    from minerva_amd import hostapi
    r = hostapi.Runtime(0, sync_each_op=True)
    params, batches = _batches("mlp", 32, 1)
    net = hostapi.Net(r, "mlp", 32)
    with pytest.raises(hostapi.HostError, match="load a batch"):
        net.capture_step(0.1)
    with pytest.raises(hostapi.HostError, match="record a step"):
        net.replay(1)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(*batches[0])
    net.capture_step(0.1)
    with pytest.raises(hostapi.HostError, match="recorded"):
        net.step(0.1)
    with pytest.raises(hostapi.HostError, match="already recorded"):
        net.capture_step(0.1)
    # parameters set while the recording exists are the ones the next replay starts from
    net.set_param("b1", np.full(10, 0.25, np.float32))
    net.replay(1)
    with_graph = net.read("w1", net.params["w1"])
    net.release_graph()
    # after the release the network steps eagerly again, from the replayed parameters
    net.step(0.1)
    assert np.max(np.abs(net.read("w1", net.params["w1"]) - with_graph)) > 0
    net.close()
    want = _eager("mlp", 32, 0, 0.1, dict(params, b1=np.full(10, 0.25, np.float32)), batches)[0]
    assert_bits_equal(with_graph, want["w1"], "replay after set_param")
    # a network with dropout draws fresh seeds on the host in every step
    drop = hostapi.Net(r, "alexnet", 1, 1)
    drop.load_batch(np.zeros(227 * 227 * 3, np.float32), np.zeros(1000, np.float32))
    with pytest.raises(hostapi.HostError, match="random seeds"):
        drop.capture_step(0.1)
    drop.close()
    r.close()


def test_c_abi_graph_capture_and_replay(ora):
    """The five graph entry points by themselves: c = a @ b, e = c + d recorded once and
    replayed on changing inputs (a skinny product, so the split-k workspace path with its
    second kernel is part of the recording)."""
    gpu = Gpu()
    L = gpu.L
    m, n, k = 64, 48, 4096
    rng = np.random.default_rng(5)
    da, db, dd = gpu.empty(m * k), gpu.empty(k * n), gpu.empty(m * n)
    dc, de = gpu.empty(m * n), gpu.empty(m * n)
    ws_bytes = L.mnv_sgemm_nn_workspace_bytes(m, n, k)
    assert ws_bytes > 0
    ws = gpu.empty(ws_bytes // 4 + 1)
    s = gpu.dev.stream

    def launch():
        assert L.mnv_sgemm_nn(da.p, db.p, dc.p, m, n, k, ws.p, ctypes.c_size_t(ws_bytes), s) == 0
        assert L.mnv_add(dc.p, dd.p, de.p, ctypes.c_size_t(m * n), s) == 0

    def load(seed):
        r = np.random.default_rng(seed)
        a, b, d = (r.standard_normal(x).astype(np.float32) for x in (m * k, k * n, m * n))
        for buf, h in ((da, a), (db, b), (dd, d)):
            assert L.mnv_memcpy_h2d(buf.p, h.ctypes.data_as(ctypes.c_void_p), h.size * 4, s) == 0
        gpu.dev.sync()
        return a, b, d

    load(1)
    launch()  # one-time set-up outside the recording
    gpu.dev.sync()
    say("c-abi capture")
    assert L.mnv_graph_begin_capture(None) == -1  # the default stream cannot be recorded
    assert L.mnv_graph_begin_capture(s) == 0
    launch()
    exe, nodes = ctypes.c_void_p(), ctypes.c_size_t()
    assert L.mnv_graph_end_capture(s, ctypes.byref(exe), ctypes.byref(nodes)) == 0
    assert exe.value and nodes.value >= 2  # product (+ split-k reduction), addition
    for seed in (2, 3, 4):
        load(seed)
        launch()
        gpu.dev.sync()
        eager = gpu.down(de)
        assert L.mnv_fill(de.p, ctypes.c_size_t(m * n), ctypes.c_float(-1.0), s) == 0
        assert L.mnv_fill(dc.p, ctypes.c_size_t(m * n), ctypes.c_float(-1.0), s) == 0
        say("c-abi replay", seed)
        assert L.mnv_graph_launch(exe, s) == 0
        gpu.dev.sync()
        assert_bits_equal(gpu.down(de), eager, "replay with inputs of seed %d" % seed)
    a, b, d = load(9)
    assert L.mnv_graph_launch(exe, s) == 0
    gpu.dev.sync()
    ref = ora.matmult(a, b, m, n, k, fast=True) + d
    assert np.max(np.abs(gpu.down(de) - ref)) <= 1e-4 * np.max(np.abs(ref))
    assert L.mnv_graph_destroy(exe) == 0
    assert L.mnv_graph_launch(None, s) == -1
    # aborting a recording leaves the stream usable
    assert L.mnv_graph_begin_capture(s) == 0
    launch()
    assert L.mnv_graph_abort_capture(s) == 0
    launch()
    gpu.dev.sync()
