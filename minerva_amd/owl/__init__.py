"""NArray front end over the HIP operator path, with the names, argument order and shape
conventions of Minerva's Python binding (reference owl/owl/__init__.py:1-221 for the
module functions, owl/owl/libowl.pyx:51-444 for the NArray class).

A program written against the reference's `owl` runs on this package after
`from minerva_amd import owl` (and `from minerva_amd.owl import elewise, conv`):

    gpu = owl.create_gpu_device(0); owl.set_device(gpu)
    w = owl.randn([256, 784], 0.0, 0.01); x = owl.from_numpy(batch)
    a = elewise.relu(w * x + b)          # `*` of two NArrays is the matrix product

What differs, on purpose:
 * operators are queued on the device's stream in program order instead of being recorded
   in a lazy dataflow graph; `wait_for_all` / `wait_for_eval` / `to_numpy` wait for them.
   Results are the same, the reference's scheduler is not part of this path;
 * there is no CPU device: `create_cpu_device` raises (every operator here runs as a HIP
   kernel and nothing falls back to the host);
 * `has_cuda` reports whether a GPU operator path exists (it does: HIP).

Shapes follow Minerva: `shape[0]` is the fastest dimension, so `from_numpy` of a C-ordered
array of shape (a, b, c) gives an NArray of shape [c, b, a] over the same bytes
(reference owl/owl/__init__.py:137-160).
"""
import numpy as np

from .. import capi, hostapi

_ARITH = {"add": 0, "sub": 1, "mul": 2, "div": 3}  # ArithmeticType (reference op/closure.h:8-13)
_ELEWISE = {"exp": 0, "ln": 1, "neg": 2}           # ElewiseType (op/closure.h:15-19)
_REDUCE = {"sum": 0, "max": 1}                     # ReductionType (op/closure.h:21-24)

_devices = {}   # device id -> hostapi.Runtime
_current = None


def _runtime():
    if _current is None:
        raise RuntimeError("no device selected: call create_gpu_device and set_device first")
    return _devices[_current]


def initialize():
    """The reference parses its command-line flags here; nothing to do."""


def has_cuda():
    """1 when GPU operators are available (reference owl/owl/__init__.py:31-37)."""
    return 1 if get_gpu_device_count() > 0 else 0


def wait_for_all():
    """Blocks until every operator issued so far has finished (owl/__init__.py:39-47)."""
    for rt in _devices.values():
        rt.sync()


def create_cpu_device():
    raise NotImplementedError("this build has no CPU operator path: create a GPU device")


def create_gpu_device(which):
    """A device on GPU `which`; returns its id (owl/__init__.py:62-73).  The first device
    created becomes the current one."""
    global _current
    rt = hostapi.Runtime(gpu=int(which), sync_each_op=False)
    dev = (max(_devices) + 1) if _devices else 0
    _devices[dev] = rt
    if _current is None:
        _current = dev
    return dev


def get_gpu_device_count():
    import ctypes
    n = ctypes.c_int()
    capi.check(capi.lib().mnv_device_count(ctypes.byref(n)), "mnv_device_count")
    return n.value


def set_device(dev):
    """Operators issued from now on run on `dev` (owl/__init__.py:83-91)."""
    global _current
    if dev not in _devices:
        raise ValueError("unknown device id %r" % (dev,))
    _current = dev


def close_devices():
    """Releases every device (not in the reference, whose system lives until exit)."""
    global _current
    for rt in _devices.values():
        rt.close()
    _devices.clear()
    _current = None


def _dims(shape):
    d = [int(x) for x in shape]
    if not d or any(x <= 0 for x in d):
        raise ValueError("bad shape %r" % (shape,))
    return d


class NArray(object):
    """A dense fp32 array on the current device (reference libowl.pyx:51-444)."""

    __array_priority__ = 1000  # numpy scalars defer to the reflected operators below

    def __init__(self, runtime, tensor):
        self._rt, self._t = runtime, tensor

    def __del__(self):
        try:
            if self._t is not None and self._rt.h:
                self._t.free()
        except Exception:
            pass

    # ---- helpers
    def _op(self, name, others=(), params=()):
        ins = [self._t] + [o._t for o in others]
        return NArray(self._rt, self._rt.top(name, ins, params))

    def _binary(self, rhs, kind):
        """NArray (op) NArray: same shape -> element-wise; otherwise rhs is replicated along
        its dimensions of size 1 (reference narray_elewise.cpp:17-27, narray.cpp:195-214)."""
        if self.shape == rhs.shape:
            return self._op("arithmetic", [rhs], [_ARITH[kind]])
        return self._op("norm_arithmetic", [rhs], [_ARITH[kind]])

    def _const(self, val, kind, side):
        # side 0: val (op) x, side 1: x (op) val (reference op/closure.h:94-98)
        return self._op("arithmetic_const", params=[_ARITH[kind], float(val), side])

    def _assign(self, other):
        old, self._t = self._t, other._t
        other._t = None
        old.free()
        return self

    # ---- arithmetic (libowl.pyx:60-179); `*` of two arrays is the matrix product
    def __add__(self, rhs):
        return self._binary(rhs, "add") if isinstance(rhs, NArray) else self._const(rhs, "add", 1)

    def __radd__(self, lhs):
        return self._const(lhs, "add", 0)

    def __sub__(self, rhs):
        return self._binary(rhs, "sub") if isinstance(rhs, NArray) else self._const(rhs, "sub", 1)

    def __rsub__(self, lhs):
        return self._const(lhs, "sub", 0)

    def __mul__(self, rhs):
        return self._op("matmult", [rhs]) if isinstance(rhs, NArray) else self._const(rhs, "mul", 1)

    def __rmul__(self, lhs):
        return self._const(lhs, "mul", 0)

    def __truediv__(self, rhs):
        return self._binary(rhs, "div") if isinstance(rhs, NArray) else self._const(rhs, "div", 1)

    def __rtruediv__(self, lhs):
        return self._const(lhs, "div", 0)

    __div__, __rdiv__ = __truediv__, __rtruediv__

    def __neg__(self):
        return self._op("elewise", params=[_ELEWISE["neg"]])

    def __iadd__(self, rhs):
        return self._assign(self + rhs)

    def __isub__(self, rhs):
        return self._assign(self - rhs)

    def __imul__(self, rhs):
        return self._assign(self * rhs)

    def __itruediv__(self, rhs):
        return self._assign(self / rhs)

    __idiv__ = __itruediv__

    # ---- static operator functions of the binding (libowl.pyx:181-343)
    @staticmethod
    def mult(lhs, rhs):
        return lhs._binary(rhs, "mul")

    @staticmethod
    def exp(x):
        return x._op("elewise", params=[_ELEWISE["exp"]])

    @staticmethod
    def ln(x):
        return x._op("elewise", params=[_ELEWISE["ln"]])

    @staticmethod
    def sigm(x):
        return x._op("sigmoid_forward")

    @staticmethod
    def relu(x):
        return x._op("relu_forward")

    @staticmethod
    def tanh(x):
        return x._op("tanh_forward")

    @staticmethod
    def sigm_back(diff, top, bottom):
        return diff._op("sigmoid_backward", [top, bottom])

    @staticmethod
    def relu_back(diff, top, bottom):
        return diff._op("relu_backward", [top, bottom])

    @staticmethod
    def tanh_back(diff, top, bottom):
        return diff._op("tanh_backward", [top, bottom])

    @staticmethod
    def activation_forward(src, algo):
        return src._op("activation_forward", params=[int(algo)])

    @staticmethod
    def activation_backward(diff, top, bottom, algo):
        return diff._op("activation_backward", [top, bottom], [int(algo)])

    @staticmethod
    def softmax_forward(src, algo):
        return src._op("softmax_forward", params=[int(algo)])

    @staticmethod
    def softmax_backward(diff, top, algo):
        return diff._op("softmax_backward", [top], [int(algo)])

    @staticmethod
    def conv_forward(src, filt, bias, info):
        return src._op("conv_forward", [filt, bias], info.params())

    @staticmethod
    def conv_backward_data(diff, bottom, filt, info):
        return diff._op("conv_backward_data", [bottom, filt], info.params())

    @staticmethod
    def conv_backward_filter(diff, bottom, filt, info):
        return diff._op("conv_backward_filter", [bottom, filt], info.params())

    @staticmethod
    def conv_backward_bias(diff):
        return diff._op("conv_backward_bias")

    @staticmethod
    def pooling_forward(src, info):
        return src._op("pooling_forward", params=info.params())

    @staticmethod
    def pooling_backward(diff, top, bottom, info):
        return diff._op("pooling_backward", [top, bottom], info.params())

    @staticmethod
    def lrn_forward(src, scale, local_size, alpha, beta):
        return src._op("lrn_forward", [scale], [int(local_size), float(alpha), float(beta)])

    @staticmethod
    def lrn_backward(bottom_data, top_data, scale, top_diff, local_size, alpha, beta):
        return bottom_data._op("lrn_backward", [top_data, scale, top_diff],
                               [int(local_size), float(alpha), float(beta)])

    # ---- reductions and shape (libowl.pyx:345-387)
    def _reduce(self, dims, kind):
        dims = [dims] if isinstance(dims, int) else list(dims)
        out = self
        for d in dims:  # one dimension per operator: the device path reduces 2-D arrays
            out = out._op("reduction", params=[_REDUCE[kind], int(d)])
        return out

    def sum(self, dims):
        """Sum over dimension `dims` (an int or a list); reduced dimensions keep size 1."""
        return self._reduce(dims, "sum")

    def max(self, dims):
        return self._reduce(dims, "max")

    def max_index(self, dim):
        """Index (as a float) of the first maximum along `dim`."""
        return self._op("maxindex", params=[int(dim)])

    def count_zero(self):
        """Number of elements equal to zero (waits for the array)."""
        values = self._t.read()
        return int(values.size - np.count_nonzero(values))

    def trans(self):
        return self._op("trans")

    def reshape(self, shape):
        return self._op("reshape", params=_dims(shape))

    def wait_for_eval(self):
        self._rt.sync()

    @property
    def shape(self):
        return list(self._t.dims)

    # ---- creation (libowl.pyx:388-444)
    @staticmethod
    def zeros(shape):
        rt = _runtime()
        return NArray(rt, rt.top("fill", [], [0.0] + _dims(shape)))

    @staticmethod
    def ones(shape):
        rt = _runtime()
        return NArray(rt, rt.top("fill", [], [1.0] + _dims(shape)))

    @staticmethod
    def randn(shape, mean, var):
        rt = _runtime()
        return NArray(rt, rt.top("randn", [], [float(mean), float(var)] + _dims(shape)))

    @staticmethod
    def randb(shape, prob):
        rt = _runtime()
        return NArray(rt, rt.top("rand_bernoulli", [], [float(prob)] + _dims(shape)))

    @staticmethod
    def concat(arrays, dim):
        arrays = list(arrays)
        return arrays[0]._op("concat", arrays[1:], [int(dim)])

    @staticmethod
    def slice(src, slice_dim, st_off, slice_count):
        return src._op("slice", params=[int(slice_dim), int(st_off), int(slice_count)])

    @staticmethod
    def from_numpy(arr):
        arr = np.require(arr, dtype=np.float32, requirements=["C"])
        rt = _runtime()
        shape = list(reversed(arr.shape)) if arr.ndim else [1]
        return NArray(rt, rt.tensor(arr, shape))

    def to_numpy(self):
        """The array as numpy, dimensions reversed back (waits for it)."""
        return self._t.read().reshape(list(reversed(self.shape)))


def zeros(shape):
    return NArray.zeros(shape)


def ones(shape):
    return NArray.ones(shape)


def randn(shape, mu, var):
    """Normal random array; `var` is handed to the generator as its spread exactly as the
    reference does (owl/__init__.py:113-123 -> RandnOp closure)."""
    return NArray.randn(shape, mu, var)


def randb(shape, prob):
    return NArray.randb(shape, prob)


def from_numpy(nparr):
    return NArray.from_numpy(nparr)


def concat(narrays, concat_dim):
    return NArray.concat(narrays, concat_dim)


def slice(src, slice_dim, st_off, slice_count):
    return NArray.slice(src, slice_dim, st_off, slice_count)


def set_random_seed(seed):
    """Seeds the device generators (the reference seeds from the clock; a fixed seed makes
    `randn` / `randb` reproducible)."""
    hostapi.Runtime.set_random_seed(int(seed))
