"""ctypes binding of the C++ host layer (include/mnv_host.h -> lib/libmnv_host.so).

`Runtime.op` runs one Minerva operator on numpy tensors through the complete host
stack (closure -> Task -> HipDevice -> FnBundle -> hip::<Op> -> C ABI -> HIP kernel);
`Net` drives the training graphs.  Tensors are (flat float32 data, Minerva dims) pairs:
dims[0] is the fastest dimension, so a numpy array of shape dims[::-1] has the same bytes.
"""
import ctypes
import os

import numpy as np

from . import capi

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libmnv_host.so")
MAX_DIMS = 8


class _Tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.POINTER(ctypes.c_float)), ("ndims", ctypes.c_int),
                ("dims", ctypes.c_int * MAX_DIMS)]


class HostError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError("%s is missing: run `python -m minerva_amd.build`" % LIB_PATH)
        capi.lib()  # libmnv_hip.so first, from the same directory
        L = ctypes.CDLL(LIB_PATH)
        L.mnvh_last_error.restype = ctypes.c_char_p
        _lib = L
    return _lib


def _check(rc, what):
    if rc != 0:
        raise HostError("%s: %s" % (what, lib().mnvh_last_error().decode()))


class DeviceTensor:
    """A tensor resident on the device (a handle of the host layer)."""

    def __init__(self, runtime, handle):
        self.rt, self.h = runtime, handle
        nd, st = ctypes.c_int(), ctypes.c_int()
        dims = (ctypes.c_int * MAX_DIMS)()
        _check(lib().mnvh_tensor_info(self.h, ctypes.byref(nd), dims, ctypes.byref(st)), "tensor_info")
        self.dims = [dims[i] for i in range(nd.value)]
        self.stream = st.value  # worker stream the producer was placed on

    def read(self):
        n = int(np.prod(self.dims))
        out = np.empty(n, np.float32)
        _check(lib().mnvh_tensor_read(self.rt.h, self.h,
                                      out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                      ctypes.c_size_t(n)), "tensor_read")
        return out

    def free(self):
        if self.h:
            _check(lib().mnvh_tensor_free(self.h), "tensor_free")
            self.h = None


class Runtime:
    def __init__(self, gpu=0, sync_each_op=True, dataflow=False, pool_bytes=None):
        """sync_each_op: wait after every operator (the reference's behaviour); dataflow:
        four streams ordered by events instead (implies no per-operator wait); pool_bytes:
        threshold of the pooled allocator."""
        self.h = ctypes.c_void_p()
        mode = 2 if dataflow else (1 if sync_each_op else 0)
        if pool_bytes is None:
            _check(lib().mnvh_runtime_create(gpu, mode, ctypes.byref(self.h)), "runtime_create")
        else:
            _check(lib().mnvh_runtime_create_pool(gpu, mode, ctypes.c_size_t(pool_bytes),
                                                  ctypes.byref(self.h)), "runtime_create_pool")

    def tensor(self, a, dims):
        a = np.ascontiguousarray(a, dtype=np.float32).ravel()
        assert a.size == int(np.prod(dims))
        t = _Tensor()
        t.data = a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
        t.ndims = len(dims)
        for j, d in enumerate(dims):
            t.dims[j] = int(d)
        h = ctypes.c_void_p()
        _check(lib().mnvh_tensor_create(self.h, ctypes.byref(t), ctypes.byref(h)), "tensor_create")
        return DeviceTensor(self, h)

    def top(self, name, inputs, params=()):
        """One operator on device tensors; returns a DeviceTensor (nothing is synchronised)."""
        arr = (ctypes.c_void_p * max(len(inputs), 1))(*[t.h for t in inputs])
        p = (ctypes.c_double * max(len(params), 1))(*[float(x) for x in params])
        h = ctypes.c_void_p()
        _check(lib().mnvh_tensor_op(self.h, name.encode(), arr, len(inputs), p, len(params),
                                    ctypes.byref(h)), name)
        return DeviceTensor(self, h)

    def close(self):
        if self.h:
            _check(lib().mnvh_runtime_destroy(self.h), "runtime_destroy")
            self.h = None

    def sync(self):
        _check(lib().mnvh_runtime_sync(self.h), "runtime_sync")

    def ops_issued(self):
        n = ctypes.c_ulonglong()
        _check(lib().mnvh_runtime_ops_issued(self.h, ctypes.byref(n)), "ops_issued")
        return n.value

    def pool_stats(self):
        t, c = ctypes.c_size_t(), ctypes.c_size_t()
        _check(lib().mnvh_runtime_pool_stats(self.h, ctypes.byref(t), ctypes.byref(c)), "pool_stats")
        return t.value, c.value

    def set_stream(self, stream):
        """Dataflow mode: the following operators go to worker stream `stream` (-1: automatic)."""
        _check(lib().mnvh_runtime_set_stream(self.h, int(stream)), "set_stream")

    def set_dataflow(self, on):
        """Switches a live runtime between the one-stream order and dataflow placement."""
        _check(lib().mnvh_runtime_set_dataflow(self.h, 1 if on else 0), "set_dataflow")

    def dataflow_stats(self):
        """(waits for a producer on another stream, waits before reusing a recycled block)"""
        a, b = ctypes.c_ulonglong(), ctypes.c_ulonglong()
        _check(lib().mnvh_runtime_dataflow_stats(self.h, ctypes.byref(a), ctypes.byref(b)),
               "dataflow_stats")
        return a.value, b.value

    def profile(self, enable, only=""):
        """Per-operator device timing; `only`: time just the operators whose name contains it."""
        _check(lib().mnvh_runtime_profile_filter(self.h, only.encode()), "profile_filter")
        _check(lib().mnvh_runtime_profile(self.h, 1 if enable else 0), "profile")

    def profile_read(self):
        """{operator name: (launches, total device ms)} since the last read."""
        buf = ctypes.create_string_buffer(1 << 16)
        _check(lib().mnvh_runtime_profile_read(self.h, buf, ctypes.c_size_t(len(buf))), "profile_read")
        out = {}
        for line in buf.value.decode().splitlines():
            name, cnt, ms = line.split("\t")
            out[name] = (int(cnt), float(ms))
        return out

    def op(self, name, inputs, params=(), out_capacity=None):
        """inputs: list of (array, dims).  Returns (flat float32 result, dims)."""
        keep = []
        arr = (_Tensor * max(len(inputs), 1))()
        for i, (a, dims) in enumerate(inputs):
            a = np.ascontiguousarray(a, dtype=np.float32).ravel()
            assert a.size == int(np.prod(dims)), (name, a.size, dims)
            keep.append(a)
            arr[i].data = a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
            arr[i].ndims = len(dims)
            for j, d in enumerate(dims):
                arr[i].dims[j] = int(d)
        if out_capacity is None:
            out_capacity = max([int(np.prod(d)) for _, d in inputs] + [1]) * 4 + 1024
        out = np.empty(out_capacity, dtype=np.float32)
        nd = ctypes.c_int()
        od = (ctypes.c_int * MAX_DIMS)()
        p = (ctypes.c_double * max(len(params), 1))(*[float(x) for x in params])
        _check(lib().mnvh_op(self.h, name.encode(), arr, len(inputs), p, len(params),
                             out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                             ctypes.c_size_t(out_capacity), ctypes.byref(nd), od), name)
        dims = [od[i] for i in range(nd.value)]
        return out[:int(np.prod(dims))].copy(), dims

    @staticmethod
    def set_random_seed(seed):
        _check(lib().mnvh_set_random_seed(ctypes.c_uint64(seed)), "set_random_seed")

    def concurrent_adds(self, a, b, count):
        a = np.ascontiguousarray(a, np.float32)
        b = np.ascontiguousarray(b, np.float32)
        out = np.empty(count * a.size, np.float32)
        fp = ctypes.POINTER(ctypes.c_float)
        _check(lib().mnvh_concurrent_adds(self.h, a.ctypes.data_as(fp), b.ctypes.data_as(fp),
                                          ctypes.c_size_t(a.size), count, out.ctypes.data_as(fp)),
               "concurrent_adds")
        return out.reshape(count, a.size)


class Net:
    def __init__(self, runtime, kind, batch, variant=0):
        self.rt = runtime
        self.h = ctypes.c_void_p()
        _check(lib().mnvh_net_create(runtime.h, kind.encode(), batch, variant, ctypes.byref(self.h)),
               "net_create")
        n = ctypes.c_int()
        _check(lib().mnvh_net_num_params(self.h, ctypes.byref(n)), "net_num_params")
        self.params = {}
        for i in range(n.value):
            name = ctypes.create_string_buffer(16)
            sz = ctypes.c_size_t()
            _check(lib().mnvh_net_param_info(self.h, i, name, ctypes.byref(sz)), "net_param_info")
            self.params[name.value.decode()] = sz.value

    def close(self):
        if self.h:
            _check(lib().mnvh_net_destroy(self.h), "net_destroy")
            self.h = None

    def set_param(self, name, a):
        a = np.ascontiguousarray(a, np.float32).ravel()
        _check(lib().mnvh_net_set_param(self.h, name.encode(),
                                        a.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                        ctypes.c_size_t(a.size)), "net_set_param " + name)

    def read(self, name, floats):
        out = np.empty(floats, np.float32)
        _check(lib().mnvh_net_read(self.h, name.encode(),
                                   out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                   ctypes.c_size_t(floats)), "net_read " + name)
        return out

    def load_batch(self, data, label):
        d = np.ascontiguousarray(data, np.float32).ravel()
        l = np.ascontiguousarray(label, np.float32).ravel()
        fp = ctypes.POINTER(ctypes.c_float)
        _check(lib().mnvh_net_load_batch(self.h, d.ctypes.data_as(fp), ctypes.c_size_t(d.size),
                                         l.ctypes.data_as(fp), ctypes.c_size_t(l.size)),
               "net_load_batch")

    def prefetch_batch(self, data, label):
        """Loads the batch of the NEXT step while the step in flight keeps the GPU busy (a second
        worker stream, pinned staging); the next `step` trains on it."""
        d = np.ascontiguousarray(data, np.float32).ravel()
        l = np.ascontiguousarray(label, np.float32).ravel()
        fp = ctypes.POINTER(ctypes.c_float)
        _check(lib().mnvh_net_prefetch_batch(self.h, d.ctypes.data_as(fp), ctypes.c_size_t(d.size),
                                             l.ctypes.data_as(fp), ctypes.c_size_t(l.size)),
               "net_prefetch_batch")

    def set_fused(self, on=True, updates=False):
        """Opt-in fast path: fused epilogues instead of separate ReLU / bias / update operators.
        `updates`: the weight updates are also applied where the weight gradients are produced;
        the parameters keep their bits, but no "g_w<i>" can be read after a step."""
        _check(lib().mnvh_net_set_fused(self.h, (2 if updates else 1) if on else 0), "net_set_fused")

    def keep_activations(self, on=True):
        """The following steps also keep "act1" ... "act10" readable (AlexNet only)."""
        _check(lib().mnvh_net_keep_activations(self.h, 1 if on else 0), "net_keep_activations")

    def step(self, lr):
        _check(lib().mnvh_net_step(self.h, ctypes.c_float(lr)), "net_step")

    def capture_step(self, lr):
        """Records one step into a HIP graph; returns the number of graph nodes."""
        n = ctypes.c_size_t()
        _check(lib().mnvh_net_capture_step(self.h, ctypes.c_float(lr), ctypes.byref(n)),
               "net_capture_step")
        return n.value

    def replay(self, steps=1, sync_each_step=True):
        _check(lib().mnvh_net_replay(self.h, int(steps), 1 if sync_each_step else 0), "net_replay")

    def release_graph(self):
        _check(lib().mnvh_net_release_graph(self.h), "net_release_graph")
