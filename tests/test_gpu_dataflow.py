"""Dataflow mode of the device: operators spread over four streams and ordered by events
on the GPU instead of a host wait after every operator.  Results must be bit-identical to
the one-stream order, also when a consumer sits on another stream than its producer and
when a pool block is recycled on another stream while its last reader is still queued."""
import numpy as np
import pytest

from gpu_util import assert_bits_equal, net_batches, run_steps, say

pytestmark = pytest.mark.gpu


def _rand(n, seed):
    return np.random.default_rng(seed).standard_normal(n).astype(np.float32)


@pytest.mark.parametrize("kind,batch,variant", [("mlp", 256, 0), ("cnn", 64, 0), ("cnn", 32, 1),
                                                ("alexnet", 2, 0)])
def test_training_steps_identical_to_stream_order(kind, batch, variant):
    params, batches = net_batches(kind, batch, 3)
    say("one stream", kind, batch, variant)
    want = run_steps(kind, batch, variant, 0.05, params, batches)
    say("dataflow", kind, batch, variant)
    got = run_steps(kind, batch, variant, 0.05, params, batches, dataflow=True)
    for i, (g, w) in enumerate(zip(got, want)):
        for k in w:
            assert_bits_equal(g[k], w[k], "%s after step %d" % (k, i))


def test_consumer_on_another_stream_waits_for_its_producer():
    from minerva_amd import hostapi
    n = 2048
    a, b = _rand(n * n, 1) / np.float32(45), _rand(n * n, 2) / np.float32(45)
    results = {}
    for mode in ("order", "dataflow"):
        r = hostapi.Runtime(0, sync_each_op=False, dataflow=(mode == "dataflow"))
        ta, tb = r.tensor(a, [n, n]), r.tensor(b, [n, n])
        say("producer chain", mode)
        chain = [r.top("matmult", [ta, tb])]
        for _ in range(7):  # ~0.15 ms each: the host is several products ahead of the GPU
            chain.append(r.top("matmult", [chain[-1], tb]))
        mid = chain[3]
        # a side branch off the middle of the chain, declared independent of what follows `mid`:
        # placed on another stream, it must wait for `mid` on the GPU
        if mode == "dataflow":
            r.set_stream((chain[0].stream + 1) % 4)
        side = r.top("arithmetic", [mid, mid], [0])
        if mode == "dataflow":
            r.set_stream(-1)
        side2 = r.top("arithmetic_const", [side], [2, 0.5, 0])   # follows `side` by itself
        if mode == "dataflow":
            assert all(c.stream == chain[0].stream for c in chain), "a chain shares one stream"
            assert side.stream != mid.stream, "the side branch must sit on another stream"
            assert side2.stream == side.stream
            assert r.dataflow_stats()[0] >= 1, "the side branch must wait for its producer"
        results[mode] = (side2.read(), chain[-1].read())
        r.close()
    assert_bits_equal(results["dataflow"][0], results["order"][0], "side branch")
    assert_bits_equal(results["dataflow"][1], results["order"][1], "main chain")
    assert np.isfinite(results["order"][1]).all() and np.abs(results["order"][0]).max() > 0


def test_block_recycled_on_another_stream_waits_for_its_last_reader():
    from minerva_amd import hostapi
    n = 4096
    x = _rand(n * n, 3) / np.float32(64)
    results = {}
    for mode in ("order", "dataflow"):
        # four live 64 MiB tensors make half of this pool's threshold: from there on a
        # stream recycles a block that another stream still uses rather than allocating
        r = hostapi.Runtime(0, sync_each_op=False, dataflow=(mode == "dataflow"),
                            pool_bytes=512 << 20)
        tx = r.tensor(x, [n, n])
        say("long reader", mode)
        y = r.top("arithmetic_const", [tx], [2, 1.0, 0])    # y = x on the device, own block
        prod = r.top("matmult", [y, y])                       # ~1 ms, reads y throughout
        prod2 = r.top("matmult", [prod, tx])
        total_before, _ = r.pool_stats()
        y.free()                                              # y's block goes back to the pool
        z = r.top("fill", [], [7.0, n, n])                    # 64 MiB, no inputs: a stream of its own;
        total_after, _ = r.pool_stats()                       # same size: takes y's block
        assert total_after == total_before, "the fill must recycle the freed block"
        if mode == "dataflow":
            assert z.stream != prod.stream, "the fill must sit on another stream than the reader"
            assert r.dataflow_stats()[1] >= 1, "the fill's stream must have been made to wait"
        results[mode] = (prod.read(), prod2.read())
        assert_bits_equal(z.read(), np.full(n * n, 7.0, np.float32), "fill")
        r.close()
    # the reader saw y, not the fill that recycled y's block
    assert_bits_equal(results["dataflow"][0], results["order"][0], "product that read the freed block")
    assert_bits_equal(results["dataflow"][1], results["order"][1], "its successor")
    s = np.float64(x[:n]) @ np.float64(x.reshape(n, n)[:, 0])  # entry (0, 0) of x @ x, column-major
    assert abs(results["order"][0][0] - s) <= 1e-3 * max(1.0, abs(s))


def test_random_operator_graph_with_frees():
    """A few hundred operators over a changing set of live tensors, tensors freed while
    their consumers are queued: dataflow placement against the one-stream order."""
    from minerva_amd import hostapi
    m = 2048   # 16 MiB tensors: large enough for an operator to start a chain of its own
    rng_ops = np.random.default_rng(11)
    plan = []
    live = 4
    for _ in range(120):
        kind = int(rng_ops.integers(0, 5))
        i, j = int(rng_ops.integers(0, live)), int(rng_ops.integers(0, live))
        drop = int(rng_ops.integers(0, live + 1)) if live > 6 else -1
        plan.append((kind, i, j, drop, int(rng_ops.integers(-1, 4))))
        live += 1
        if 0 <= drop < live - 1:
            live -= 1
    outs = {}
    for mode in ("order", "dataflow"):
        r = hostapi.Runtime(0, sync_each_op=False, dataflow=(mode == "dataflow"))
        ts = [r.tensor(_rand(m * m, 20 + k) / np.float32(16), [m, m]) for k in range(4)]
        streams = set()
        say("random graph", mode)
        for kind, i, j, drop, where in plan:
            if mode == "dataflow":
                r.set_stream(where)     # -1: automatic (follows the newest input in flight)
            if kind == 0:
                t = r.top("matmult", [ts[i], ts[j]])
                t2 = r.top("arithmetic_const", [t], [2, 1.0 / 16, 0])  # keep magnitudes bounded
                t.free()
                t = t2
            elif kind == 1:
                t = r.top("arithmetic", [ts[i], ts[j]], [1])
            elif kind == 2:
                t = r.top("trans", [ts[i]])
            elif kind == 3:
                t = r.top("tanh_forward", [ts[i]])
            else:
                t = r.top("arithmetic", [ts[i], ts[j]], [2])
            streams.add(t.stream)
            ts.append(t)
            if 0 <= drop < len(ts) - 1:
                ts.pop(drop).free()
        outs[mode] = [t.read() for t in ts]
        if mode == "dataflow":
            assert len(streams) >= 3, "the graph must spread over the streams: %r" % streams
        r.close()
    assert len(outs["order"]) == len(outs["dataflow"])
    for k, (g, w) in enumerate(zip(outs["dataflow"], outs["order"])):
        assert np.isfinite(w).all()
        assert_bits_equal(g, w, "live tensor %d" % k)


def test_recording_is_refused_in_dataflow_mode():
    from minerva_amd import hostapi
    params, batches = net_batches("mlp", 32, 1)
    r = hostapi.Runtime(0, dataflow=True)
    net = hostapi.Net(r, "mlp", 32)
    for k, v in params.items():
        net.set_param(k, v)
    net.load_batch(*batches[0])
    with pytest.raises(hostapi.HostError, match="dataflow"):
        net.capture_step(0.1)
    net.step(0.1)  # the refusal left the network usable
    r.sync()
    net.close()
    r.close()


def test_reader_of_lrn_scale_waits_for_the_forward_pass(ora):
    """LRNForward fills its `scale` INPUT (as the reference's does): in dataflow mode a later
    reader of `scale` alone, on another stream, must wait for the forward pass and not only
    for the fill that created the tensor."""
    from minerva_amd import hostapi
    N, C, H, W = 64, 96, 27, 27
    x = _rand(N * C * H * W, 5)
    want_top, want_scale = ora.lrn_fwd(x, 5, 1e-4, 0.75, N, C, H, W)
    r = hostapi.Runtime(0, sync_each_op=False, dataflow=True)
    dims = [W, H, C, N]
    tx = r.tensor(x, dims)
    big = r.tensor(_rand(2048 * 2048, 6) / np.float32(45), [2048, 2048])
    crossed = 0
    for rep in range(3):
        say("lrn scale reader, repetition", rep)
        busy = r.top("matmult", [big, big])          # keeps the producer's stream busy first
        busy = r.top("matmult", [busy, big])
        scale = r.top("fill", [], [0.0] + dims)
        top = r.top("lrn_forward", [tx, scale], [5, 1e-4, 0.75])
        # four more operators behind the forward pass on its stream: the reader of `scale`
        # then starts a chain of its own on another stream
        tail = top
        for _ in range(4):
            tail = r.top("arithmetic_const", [tail], [2, 1.0, 0])
            assert tail.stream == top.stream, "a chain stays on its stream"
        waits_before = r.dataflow_stats()[0]
        r.set_stream((top.stream + 1 + rep) % 4 if (top.stream + 1 + rep) % 4 != top.stream else (top.stream + 1) % 4)
        twice = r.top("arithmetic_const", [scale], [2, 2.0, 0])   # reads `scale` alone
        r.set_stream(-1)
        if twice.stream == top.stream:
            continue  # placement put both on one stream this time: stream order covers it
        crossed += 1
        assert r.dataflow_stats()[0] > waits_before, "the reader must wait for the forward pass"
        got = twice.read()
        assert float(np.max(np.abs(got - 2 * want_scale))) <= 1e-4 * float(np.max(np.abs(want_scale)))
        assert float(np.max(np.abs(top.read() - want_top))) <= 1e-4 * float(np.max(np.abs(want_top)))
    assert crossed >= 1, "no repetition placed the reader on another stream than the forward pass"
    r.close()


def test_mode_switched_on_live_data_tracks_readers_of_older_tensors():
    """Tensors created in the one-stream order have no producer on record.  After the switch
    to dataflow mode a long reader of such a tensor must still be known when the tensor's block
    is freed and taken by another stream: that stream has to wait for the reader."""
    from minerva_amd import hostapi
    n = 4096
    x = _rand(n * n, 8) / np.float32(64)
    results = {}
    for mode in ("order", "switched"):
        r = hostapi.Runtime(0, sync_each_op=False, pool_bytes=512 << 20)
        tx = r.tensor(x, [n, n])
        y = r.top("arithmetic_const", [tx], [2, 1.0, 0])      # created before the switch
        r.sync()
        if mode == "switched":
            r.set_dataflow(True)
        say("reader of a tensor older than the mode", mode)
        prod = r.top("matmult", [y, y])                         # ~1 ms, reads y throughout
        prod2 = r.top("matmult", [prod, tx])
        waits_before = r.dataflow_stats()[1]
        total_before, _ = r.pool_stats()
        y.free()
        z = r.top("fill", [], [7.0, n, n])                      # takes y's block
        assert r.pool_stats()[0] == total_before, "the fill must recycle the freed block"
        if mode == "switched":
            assert z.stream != prod.stream, "the fill must sit on another stream than the reader"
            assert r.dataflow_stats()[1] > waits_before, "the fill's stream must wait for the reader"
        results[mode] = prod.read()
        assert_bits_equal(z.read(), np.full(n * n, 7.0, np.float32), "fill")
        if mode == "switched":   # and back: everything on one stream again
            r.set_dataflow(False)
            again = r.top("matmult", [tx, tx])
            assert again.stream == 0
            again.read()
        r.close()
    assert_bits_equal(results["switched"], results["order"], "product that read the freed block")


@pytest.mark.parametrize("kind,batch", [("mlp", 256), ("cnn", 64), ("alexnet", 2)])
def test_batches_prefetched_under_the_running_step_train_the_same(kind, batch):
    """The next batch loaded on a second stream while a step is in flight (what the
    reference's trainer gets from its data provider, owl/owl/net/trainer.py:118-145): five
    different batches, every parameter, gradient and probability bit-identical to loading each
    batch in stream order before its step."""
    params, batches = net_batches(kind, batch, 5)
    say("batches loaded in stream order", kind, batch)
    want = run_steps(kind, batch, 0, 0.05, params, batches)
    say("batches prefetched under the step before", kind, batch)
    got = run_steps(kind, batch, 0, 0.05, params, batches, prefetch=True)
    for i, (g, w) in enumerate(zip(got, want)):
        for k in w:
            assert_bits_equal(g[k], w[k], "%s after step %d" % (k, i))
    # the batches differ, so a step that trained on a stale batch would show
    assert not np.array_equal(want[1]["prob"], want[2]["prob"])
