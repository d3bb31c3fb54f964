"""ctypes binding of the C ABI declared in include/mnv_hip.h.

Loading fails loudly (ImportError / OSError) if the HIP library has not been built;
nothing here computes on the CPU.  `Device` is a small convenience layer for tests
and the benchmark: device buffers, uploads/downloads of numpy arrays, streams, events.
"""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libmnv_hip.so")

c_f = ctypes.c_float
c_i = ctypes.c_int
c_sz = ctypes.c_size_t
c_p = ctypes.c_void_p

_I = c_i
_P = c_p
_S = c_p  # stream

# name -> argument types (return type is int unless listed in _RESTYPES)
PROTOTYPES = {
    "mnv_device_count": [ctypes.POINTER(c_i)],
    "mnv_device_set": [_I],
    "mnv_device_info": [_I, ctypes.c_char_p, ctypes.POINTER(c_i), ctypes.POINTER(c_i),
                        ctypes.POINTER(c_sz)],
    "mnv_stream_create": [ctypes.POINTER(c_p)],
    "mnv_stream_destroy": [_S],
    "mnv_stream_sync": [_S],
    "mnv_device_sync": [],
    "mnv_malloc": [ctypes.POINTER(c_p), c_sz],
    "mnv_free": [_P],
    "mnv_host_malloc": [ctypes.POINTER(c_p), c_sz],
    "mnv_host_free": [_P],
    "mnv_memcpy_h2d": [_P, _P, c_sz, _S],
    "mnv_memcpy_d2h": [_P, _P, c_sz, _S],
    "mnv_memcpy_d2d": [_P, _P, c_sz, _S],
    "mnv_event_create": [ctypes.POINTER(c_p)],
    "mnv_event_create_ordering": [ctypes.POINTER(_P)],
    "mnv_stream_wait_event": [_S, _P],
    "mnv_event_destroy": [_P],
    "mnv_event_record": [_P, _S],
    "mnv_event_sync": [_P],
    "mnv_event_elapsed_ms": [_P, _P, ctypes.POINTER(c_f)],
    "mnv_graph_begin_capture": [_S],
    "mnv_graph_end_capture": [_S, ctypes.POINTER(_P), ctypes.POINTER(c_sz)],
    "mnv_graph_abort_capture": [_S],
    "mnv_graph_launch": [_P, _S],
    "mnv_graph_destroy": [_P],
    "mnv_error_string": [_I],
    "mnv_sgemm_nn_workspace_bytes": [_I, _I, _I],
    "mnv_sgemm_nn": [_P, _P, _P, _I, _I, _I, _P, c_sz, _S],
    "mnv_sgemm_nn_static": [_P, _P, _P, _I, _I, _I, _S],
    "mnv_transpose": [_P, _P, _I, _I, _S],
    "mnv_copy": [_P, _P, c_sz, _S],
    "mnv_fill": [_P, c_sz, c_f, _S],
    "mnv_conv_fwd_workspace_bytes": [_I] * 11,
    "mnv_conv_fwd": [_P, _P, _P, _P] + [_I] * 11 + [_P, c_sz, _S],
    "mnv_conv_bwd_data_workspace_bytes": [_I] * 11,
    "mnv_conv_bwd_data": [_P, _P, _P] + [_I] * 11 + [_P, c_sz, _S],
    "mnv_conv_bwd_filter_workspace_bytes": [_I] * 11,
    "mnv_conv_bwd_filter": [_P, _P, _P] + [_I] * 11 + [_P, c_sz, _S],
    "mnv_conv_bwd_bias": [_P, _P, _I, _I, _I, _I, _P, c_sz, _S],
    "mnv_conv_bwd_bias_workspace_bytes": [_I, _I],
    "mnv_pooled_size": [_I, _I, _I, _I],
}
for _n in ("add", "sub", "mul", "div"):
    PROTOTYPES["mnv_" + _n] = [_P, _P, _P, c_sz, _S]
for _n in ("add", "sub", "rsub", "mul", "div", "rdiv"):
    PROTOTYPES["mnv_const_" + _n] = [_P, _P, c_f, c_sz, _S]
for _n in ("exp", "ln", "neg", "sigmoid_fwd", "relu_fwd", "tanh_fwd"):
    PROTOTYPES["mnv_" + _n] = [_P, _P, c_sz, _S]
for _n in ("sigmoid_bwd", "relu_bwd", "tanh_bwd"):
    PROTOTYPES["mnv_" + _n] = [_P, _P, _P, _P, c_sz, _S]
for _op in ("add", "sub", "mul", "div"):
    for _d in ("col", "row"):
        PROTOTYPES["mnv_norm_%s_%s" % (_op, _d)] = [_P, _P, _P, _I, _I, _S]
for _op in ("reduce_sum", "reduce_max", "maxindex"):
    for _d in ("col", "row"):
        PROTOTYPES["mnv_%s_%s" % (_op, _d)] = [_P, _P, _I, _I, _S]
for _m in ("instance", "channel"):
    PROTOTYPES["mnv_softmax_%s_fwd" % _m] = [_P, _P, _I, _I, _I, _I, _S]
    PROTOTYPES["mnv_softmax_%s_bwd" % _m] = [_P, _P, _P, _I, _I, _I, _I, _S]
for _k in ("max", "avg"):
    PROTOTYPES["mnv_%spool_fwd" % _k] = [_P, _P] + [_I] * 10 + [_S]
    PROTOTYPES["mnv_%spool_bwd" % _k] = [_P, _P, _P, _P] + [_I] * 10 + [_S]
PROTOTYPES["mnv_conv_fwd_relu"] = PROTOTYPES["mnv_conv_fwd"]
PROTOTYPES["mnv_conv_bwd_data_relu"] = [_P, _P, _P, _P] + [_I] * 11 + [_P, c_sz, _S]
PROTOTYPES["mnv_maxpool_bwd_relu"] = PROTOTYPES["mnv_maxpool_bwd"]
PROTOTYPES["mnv_sgemm_nn_bias"] = [_P, _P, _P, _P, _I, _I, _I, _I, _P, c_sz, _S]
PROTOTYPES["mnv_sgemm_nn_relu_bwd"] = [_P, _P, _P, _P, _I, _I, _I, _P, c_sz, _S]
PROTOTYPES["mnv_sgd_update"] = [_P, _P, c_f, _P, c_sz, _S]
PROTOTYPES["mnv_sgemm_tn"] = [_P, _P, _P, _P, _I, _I, _I, _P, c_sz, _S]
PROTOTYPES["mnv_sgemm_nn_plan"] = [_I, _I, _I, c_sz, _P, _P, _P]
PROTOTYPES["mnv_sgemm_nt"] = [_P, _P, _P, _I, _I, _I, _P, c_sz, _S]
PROTOTYPES["mnv_sgemm_nt_sgd"] = [_P, _P, _P, c_f, _P, _I, _I, _I, _P, c_sz, _S]
PROTOTYPES["mnv_conv_bwd_filter_plan"] = [_I] * 11 + [c_sz, _P, _P, _P]
PROTOTYPES["mnv_conv_winograd_mode"] = [_I]
PROTOTYPES["mnv_conv_winograd_profile"] = [_I]
PROTOTYPES["mnv_conv_winograd_profile_read"] = [_I, _P, _P, _P]
PROTOTYPES["mnv_conv_bwd_filter_sgd"] = [_P, _P, _P, c_f, _P] + [_I] * 11 + [_P, c_sz, _S]
PROTOTYPES["mnv_copy_2d"] = [_P, _P, c_sz, c_sz, c_sz, c_sz, _S]
PROTOTYPES["mnv_select_workspace_bytes"] = [_I]
PROTOTYPES["mnv_select"] = [_P, _P, _P, _I, _I, _I, _P, c_sz, _S]
PROTOTYPES["mnv_threshold_norm"] = [_P, _P, c_f, c_sz, _S]
PROTOTYPES["mnv_randn"] = [_P, c_sz, ctypes.c_uint64, c_f, c_f, _S]
PROTOTYPES["mnv_rand_bernoulli"] = [_P, c_sz, ctypes.c_uint64, c_f, _S]
PROTOTYPES["mnv_lrn_fwd"] = [_P, _P, _P, _I, c_f, c_f, _I, _I, _I, _I, _S]
PROTOTYPES["mnv_lrn_bwd"] = [_P, _P, _P, _P, _P, _I, c_f, c_f, _I, _I, _I, _I, _S]

_RESTYPES = {
    "mnv_error_string": ctypes.c_char_p,
    "mnv_sgemm_nn_workspace_bytes": c_sz,
    "mnv_conv_bwd_filter_workspace_bytes": c_sz,
    "mnv_conv_fwd_workspace_bytes": c_sz,
    "mnv_conv_bwd_data_workspace_bytes": c_sz,
    "mnv_conv_bwd_bias_workspace_bytes": c_sz,
    "mnv_select_workspace_bytes": c_sz,
}


class MnvError(RuntimeError):
    pass


def load(path=LIB_PATH):
    """dlopen the library and attach prototypes.  Raises OSError if it is not built."""
    if not os.path.exists(path):
        raise OSError("%s is missing: run `python -m minerva_amd.build` (there is no CPU "
                      "fallback)" % path)
    lib = ctypes.CDLL(path)
    for name, args in PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.argtypes = args
        fn.restype = _RESTYPES.get(name, c_i)
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load()
    return _lib


def check(status, what=""):
    if status != 0:
        msg = lib().mnv_error_string(status)
        raise MnvError("%s failed: status %d (%s)" % (what or "mnv call", status,
                                                      msg.decode() if msg else "?"))


class Buffer:
    """A device allocation of `n` floats."""

    def __init__(self, dev, n):
        self.dev, self.n = dev, int(n)
        p = c_p()
        check(lib().mnv_malloc(ctypes.byref(p), max(self.n, 1) * 4), "mnv_malloc")
        self.ptr = p.value

    @property
    def p(self):
        return c_p(self.ptr)

    def offset(self, floats):
        return c_p(self.ptr + 4 * floats)

    def free(self):
        if self.ptr:
            check(lib().mnv_free(c_p(self.ptr)), "mnv_free")
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Device:
    """GPU `index` with one work stream."""

    def __init__(self, index=0, own_stream=True):
        L = lib()
        n = c_i()
        check(L.mnv_device_count(ctypes.byref(n)), "mnv_device_count")
        if n.value <= index:
            raise MnvError("no GPU %d (device count %d)" % (index, n.value))
        check(L.mnv_device_set(index), "mnv_device_set")
        self.index = index
        self.stream = c_p(None)
        if own_stream:
            s = c_p()
            check(L.mnv_stream_create(ctypes.byref(s)), "mnv_stream_create")
            self.stream = s

    def info(self):
        name = ctypes.create_string_buffer(256)
        cu, khz, mem = c_i(), c_i(), c_sz()
        check(lib().mnv_device_info(self.index, name, ctypes.byref(cu), ctypes.byref(khz),
                                    ctypes.byref(mem)), "mnv_device_info")
        return {"name": name.value.decode(), "cu_count": cu.value, "clock_khz": khz.value,
                "hbm_bytes": mem.value}

    def empty(self, n):
        return Buffer(self, n)

    def upload(self, arr):
        arr = np.ascontiguousarray(arr, dtype=np.float32)
        buf = Buffer(self, arr.size)
        if arr.size:
            check(lib().mnv_memcpy_h2d(buf.p, arr.ctypes.data_as(c_p), arr.size * 4, self.stream),
                  "mnv_memcpy_h2d")
            self.sync()
        return buf

    def download(self, buf, n=None):
        n = buf.n if n is None else int(n)
        out = np.empty(n, dtype=np.float32)
        if n:
            check(lib().mnv_memcpy_d2h(out.ctypes.data_as(c_p), buf.p, n * 4, self.stream),
                  "mnv_memcpy_d2h")
            self.sync()
        return out

    def sync(self):
        check(lib().mnv_stream_sync(self.stream), "mnv_stream_sync")

    def event(self):
        e = c_p()
        check(lib().mnv_event_create(ctypes.byref(e)), "mnv_event_create")
        return e

    def record(self, ev):
        check(lib().mnv_event_record(ev, self.stream), "mnv_event_record")

    def elapsed_ms(self, e0, e1):
        check(lib().mnv_event_sync(e1), "mnv_event_sync")
        ms = c_f()
        check(lib().mnv_event_elapsed_ms(e0, e1, ctypes.byref(ms)), "mnv_event_elapsed_ms")
        return ms.value

    def time_ms(self, fn, iters=20, warmup=5, reps=1):
        """Milliseconds per call of fn(), measured with events on this stream: the median over
        `reps` batches of `iters` back-to-back calls.  fn() returns the status of the call it
        makes (or None); any non-zero status raises instead of being timed."""
        def run(count):
            for _ in range(count):
                rc = fn()
                if rc is not None:
                    check(rc, "timed call")
        run(warmup)
        e0, e1 = self.event(), self.event()
        batches = []
        for _ in range(max(reps, 1)):
            self.record(e0)
            run(iters)
            self.record(e1)
            batches.append(self.elapsed_ms(e0, e1) / iters)
        lib().mnv_event_destroy(e0)
        lib().mnv_event_destroy(e1)
        batches.sort()
        mid = len(batches) // 2
        return batches[mid] if len(batches) % 2 else 0.5 * (batches[mid - 1] + batches[mid])
