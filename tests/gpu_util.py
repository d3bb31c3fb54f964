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
