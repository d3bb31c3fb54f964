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


def net_state(net, label_floats):
    s = {k: net.read(k, n) for k, n in net.params.items()}
    s.update({"g_" + k: net.read("g_" + k, n) for k, n in net.params.items()})
    s["prob"] = net.read("prob", label_floats)
    return s


def run_steps(kind, batch, variant, lr, params, batches, **runtime_args):
    """One step per batch, operator by operator; the state after every step."""
    from minerva_amd import hostapi
    runtime_args.setdefault("sync_each_op", False)
    r = hostapi.Runtime(0, **runtime_args)
    net = hostapi.Net(r, kind, batch, variant)
    for k, v in params.items():
        net.set_param(k, v)
    states = []
    for d, l in batches:
        net.load_batch(d, l)
        net.step(lr)
        states.append(net_state(net, l.size))
    net.close()
    r.close()
    return states


# A whole training step chains ~20 fp32 operators and both sides round at every one of
# them.  Besides ordinary rounding noise there is one discontinuous effect: a pre-activation
# that rounds to different sides of 0 on the two sides flips its ReLU gate, which adds or
# drops one full-size term in the gradients downstream (seen on conv bias gradients: an
# error of exactly one term).  So a step is compared this way: probabilities and updated
# weights normwise at 1e-4; every weight gradient in relative L2 norm at 1e-3 with at least
# 99.9 % of its entries within 1e-4 of the largest entry; every bias gradient -- a sum of
# hundreds to thousands of signed, largely cancelling terms -- within 3e-3 of the L1 mass
# of its terms (one flipped term of a 338-term sum is 3e-3 of that mass), the updated bias
# within the same bound scaled by lr / batch.  The operators themselves are held to 1e-4
# (or bit-exactness) one by one in the other test files.
def rel_l2(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-30))


def compare_step(got, newp, res, lr=0.01, batch=1, deep=False):
    """deep=True (the 12-layer network at batch 2, where a handful of flipped gates among
    ~10^6 tiny activations is a visible fraction of the gradient signal): gradients are held
    to 1e-2 in relative L2 norm and 1e-3 in their norms instead of the entrywise rule."""
    for k, v in newp.items():
        g, r = got["g_" + k], res["g_" + k]
        if k.startswith("w") and deep:
            assert rel_l2(g, r) <= 1e-2, "gradient %s: relative L2 error %.3e" % (k, rel_l2(g, r))
            ng, nr = np.linalg.norm(g.astype(np.float64)), np.linalg.norm(r.astype(np.float64))
            assert abs(ng - nr) <= 1e-3 * nr, "gradient norm %s: %.6e vs %.6e" % (k, ng, nr)
            assert normwise(got[k], v) <= TOL, "updated " + k
        elif k.startswith("w"):
            assert rel_l2(g, r) <= 1e-3, "gradient %s: relative L2 error %.3e" % (k, rel_l2(g, r))
            close = np.abs(g.astype(np.float64) - r) <= TOL * np.max(np.abs(r))
            assert close.mean() >= 0.999, "gradient %s: %.5f of entries within 1e-4" % (k, close.mean())
            assert normwise(got[k], v) <= TOL, "updated " + k
        else:
            scale = 3e-3 * float(np.max(res["l1_" + k]))
            err = float(np.max(np.abs(g.astype(np.float64) - r)))
            assert err <= scale, "gradient %s: error %.3e, bound %.3e" % (k, err, scale)
            err = float(np.max(np.abs(got[k].astype(np.float64) - v)))
            assert err <= scale * lr / batch + 1e-12, "updated " + k
    assert normwise(got["prob"], res["prob"]) <= TOL
