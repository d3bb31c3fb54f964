"""Helpers shared by the GPU parity tests: every call goes through the C ABI
(minerva_amd.capi -> libmnv_hip.so); the oracle is only the checker."""
import sys

import numpy as np

from minerva_amd import capi

TOL = 1e-4  # normwise bound for the floating-point ops: max|gpu - ref| / max|ref|


def say(*a):
    """Name the case before the GPU step, flushed, so a fault can be attributed."""
    print(*a)
    sys.stdout.flush()


def normwise(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    denom = max(np.max(np.abs(ref)), 1e-30)
    return float(np.max(np.abs(got - ref)) / denom)


def assert_bits_equal(got, ref, what=""):
    got = np.ascontiguousarray(got, np.float32)
    ref = np.ascontiguousarray(ref, np.float32)
    assert got.shape == ref.shape, what
    same = got.view(np.uint32) == ref.view(np.uint32)
    both_nan = np.isnan(got) & np.isnan(ref)
    bad = ~(same | both_nan)
    assert not bad.any(), "%s: %d of %d elements differ, first at %d: %r vs %r" % (
        what, int(bad.sum()), bad.size, int(np.argmax(bad)), got.ravel()[np.argmax(bad)],
        ref.ravel()[np.argmax(bad)])


class Gpu:
    def __init__(self):
        self.L = capi.lib()
        self.dev = capi.Device(0)

    def up(self, a):
        return self.dev.upload(a)

    def down(self, b, n=None):
        return self.dev.download(b, n)

    def empty(self, n):
        return self.dev.empty(n)

    def call(self, name, *args):
        rc = getattr(self.L, name)(*args, self.dev.stream)
        capi.check(rc, name)
        self.dev.sync()


def net_batches(kind, batch, count):
    """The seeded parameters and `count` different batches of one network configuration."""
    from oracle import nets
    params, data, label = nets.make_inputs(kind, batch)
    per_d, per_l = data.size // batch, label.size // batch
    out = []
    for i in range(count):  # rotate the images against the labels: new batches, same statistics
        d = np.roll(data.reshape(batch, per_d), i, axis=0).ravel()
        l = np.roll(label.reshape(batch, per_l), 2 * i, axis=0).ravel()
        out.append((d.copy(), l.copy()))
    return params, out


def net_state(net, label_floats, weight_gradients=True):
    s = {k: net.read(k, n) for k, n in net.params.items()}
    s.update({"g_" + k: net.read("g_" + k, n) for k, n in net.params.items()
              if weight_gradients or not k.startswith("w")})
    s["prob"] = net.read("prob", label_floats)
    return s


def run_steps(kind, batch, variant, lr, params, batches, fused=False, fused_updates=False,
              prefetch=False, **runtime_args):
    """One step per batch, operator by operator (fused: with the fused operators;
    fused_updates: weight updates in the gradient kernels' stores as well, which leaves no
    weight gradients to read; prefetch: every batch but the first is loaded on a second
    stream while the step before it is in flight); the state after every step."""
    from minerva_amd import hostapi
    runtime_args.setdefault("sync_each_op", False)
    r = hostapi.Runtime(0, **runtime_args)
    net = hostapi.Net(r, kind, batch, variant)
    if fused or fused_updates:
        net.set_fused(updates=fused_updates)
    for k, v in params.items():
        net.set_param(k, v)
    states = []
    for i, (d, l) in enumerate(batches):
        if not prefetch or i == 0:
            net.load_batch(d, l)
        net.step(lr)
        if prefetch and i + 1 < len(batches):
            net.prefetch_batch(*batches[i + 1])   # under the step that was just queued
        states.append(net_state(net, l.size, weight_gradients=not fused_updates))
    run_steps.ops_issued = r.ops_issued()  # of the run that just ended
    net.close()
    r.close()
    return states


# A whole training step chains ~20 fp32 operators and both sides round at every one of them.
# For the shallow networks (MLP, MNIST CNN, batch 16 to 256) the chain is continuous enough
# that every probability, gradient and updated parameter agrees with the oracle normwise to
# 1e-4 (measured: <= 1.1e-5).
def rel_l2(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30))


def compare_step(got, newp, res):
    """Probabilities, every gradient and every updated parameter of one step, normwise 1e-4."""
    worst = {"prob": normwise(got["prob"], res["prob"])}
    for k, v in sorted(newp.items()):
        worst["g_" + k] = normwise(got["g_" + k], res["g_" + k])
        worst[k] = normwise(got[k], v)
    say("  step: worst normwise error %.2e (%s)" % (max(worst.values()), max(worst, key=worst.get)))
    bad = {k: v for k, v in worst.items() if not v <= TOL}
    assert not bad, bad


# The 12-layer AlexNet step is NOT continuous in that sense: a pre-activation that rounds to
# different sides of 0 on the two sides flips its ReLU gate (and two near-equal values in a
# pooling window can swap the arg-max), which adds or drops one full-size term in every
# gradient below it; at batch 2 a single flipped gate among ~10^6 moves the gradients of the
# layers below by 1e-3 to 1e-2.  So the step is compared in two halves, each at 1e-4:
#   forward : every activation and the probabilities against the oracle's forward pass;
#   backward: every gradient against the oracle's backward pass evaluated AT THE GPU's
#             activations (same gates and routes on both sides);
# and the update against w - lr/batch * g on the GPU's own gradient, bit for bit.
ALEX_ACT_ELEMS = {1: 96 * 55 * 55, 2: 96 * 27 * 27, 3: 256 * 27 * 27, 4: 256 * 13 * 13,
                  5: 384 * 13 * 13, 6: 384 * 13 * 13, 7: 256 * 13 * 13, 8: 9216, 9: 4096,
                  10: 4096}


def compare_alexnet_step(got, gpu_acts, params, data, label, batch, lr, ora_acts, ora_prob,
                         masks=None):
    """got: parameters, "g_*" and "prob" of the GPU step; gpu_acts: {1..10: activations}."""
    from oracle import nets
    worst = {"prob": normwise(got["prob"], ora_prob)}
    flips = 0
    for i, a in gpu_acts.items():
        worst["act%d" % i] = normwise(a, ora_acts[i])
        flips += int(np.count_nonzero((a > 0) != (ora_acts[i] > 0)))
    acts = [data] + [gpu_acts[i] for i in range(1, 11)] + [None]
    g, _, _ = nets.alexnet_backward(params, acts, got["prob"], label, batch, masks=masks)
    for k in sorted(params):
        worst["g_" + k] = normwise(got["g_" + k], g[k])
        step = (np.float32(lr) / np.float32(batch)) * got["g_" + k]
        assert_bits_equal(got[k], params[k] - step, "SGD update of " + k)
    say("  alexnet step: %d of %d gates differ from the oracle's; worst normwise error %.2e (%s)"
        % (flips, sum(a.size for a in gpu_acts.values()), max(worst.values()),
           max(worst, key=worst.get)))
    bad = {k: v for k, v in worst.items() if not v <= TOL}
    assert not bad, bad
    return flips
