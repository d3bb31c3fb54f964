"""ctypes front end of the CPU oracle (oracle/mnv_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import
this module; the shipped library never does.  Every function takes and returns
numpy float32 arrays whose *memory* is the reference's column-major layout: an
array created as ``np.empty(shape[::-1])`` (C order) for a Minerva ``Scale`` of
``shape`` has identical bytes (reference owl/owl/__init__.py:137-159 reverses the
shape list in the same way).  To keep call sites readable every function here
works on flat buffers plus explicit Minerva dims (dim 0 fastest).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmnv_oracle.so")

ADD, SUB, MUL, DIV = 0, 1, 2, 3
EXP, LN, NEG = 0, 1, 2
SUM, MAX = 0, 1
SIGMOID, RELU, TANH = 0, 1, 2
POOL_MAX, POOL_AVG = 0, 1


def build(force=False):
    """Compile the oracle with the recipe in oracle/Makefile."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "mnv_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmnv_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ora_pooled_size.restype = ctypes.c_int
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _ints(v):
    arr = (ctypes.c_int * len(v))(*[int(x) for x in v])
    return arr


def _chk(rc, name):
    if rc != 0:
        raise RuntimeError("oracle %s failed with status %d" % (name, rc))


def arithmetic(typ, a, b):
    a, b = _f(a), _f(b)
    out = np.empty_like(a)
    _chk(lib().ora_arithmetic(typ, _p(a), _p(b), _p(out), ctypes.c_size_t(a.size)), "arithmetic")
    return out


def arithmetic_const(typ, side, val, x):
    x = _f(x)
    out = np.empty_like(x)
    _chk(lib().ora_arithmetic_const(typ, side, ctypes.c_float(val), _p(x), _p(out),
                                    ctypes.c_size_t(x.size)), "arithmetic_const")
    return out


def elewise(typ, x):
    x = _f(x)
    out = np.empty_like(x)
    _chk(lib().ora_elewise(typ, _p(x), _p(out), ctypes.c_size_t(x.size)), "elewise")
    return out


def matmult(a, b, m, n, k, fast=False):
    """C{m,n} = A{m,k} * B{k,n}; flat column-major buffers."""
    a, b = _f(a), _f(b)
    assert a.size == m * k and b.size == k * n
    out = np.empty(m * n, dtype=np.float32)
    fn = lib().ora_matmult_fast if fast else lib().ora_matmult
    _chk(fn(_p(a), _p(b), _p(out), m, n, k), "matmult")
    return out


def transpose(x, m, n):
    """in{n,m} -> out{m,n}."""
    x = _f(x)
    assert x.size == m * n
    out = np.empty(m * n, dtype=np.float32)
    _chk(lib().ora_transpose(_p(x), _p(out), m, n), "transpose")
    return out


def reduction(typ, x, dims, rdims):
    x = _f(x)
    assert x.size == int(np.prod(dims))
    osize = int(np.prod([1 if i in rdims else d for i, d in enumerate(dims)]))
    out = np.empty(osize, dtype=np.float32)
    _chk(lib().ora_reduction(typ, _p(x), _ints(dims), len(dims), _ints(rdims), len(rdims),
                             _p(out)), "reduction")
    return out


def maxindex(x, dims, dim):
    x = _f(x)
    assert x.size == int(np.prod(dims))
    osize = int(np.prod([1 if i == dim else d for i, d in enumerate(dims)]))
    out = np.empty(osize, dtype=np.float32)
    _chk(lib().ora_maxindex(_p(x), _ints(dims), len(dims), dim, _p(out)), "maxindex")
    return out


def norm_arithmetic(typ, x, dims, v, rep):
    x, v = _f(x), _f(v)
    assert x.size == int(np.prod(dims))
    assert v.size == int(np.prod([1 if i in rep else d for i, d in enumerate(dims)]))
    out = np.empty_like(x)
    _chk(lib().ora_norm_arithmetic(typ, _p(x), _ints(dims), len(dims), _p(v), _ints(rep),
                                   len(rep), _p(out)), "norm_arithmetic")
    return out


def softmax_dim0(x, length):
    x = _f(x)
    out = np.empty_like(x)
    _chk(lib().ora_softmax_dim0(_p(x), _p(out), int(length),
                                ctypes.c_size_t(x.size // length)), "softmax_dim0")
    return out


def softmax_instance_fwd(x, n, c, h, w):
    return softmax_dim0(x, c * h * w)


def softmax_channel_fwd(x, n, c, h, w):
    x = _f(x)
    out = np.empty_like(x)
    _chk(lib().ora_softmax_channel_fwd(_p(x), _p(out), n, c, h, w), "softmax_channel_fwd")
    return out


def softmax_instance_bwd(dy, y, n, c, h, w):
    dy, y = _f(dy), _f(y)
    out = np.empty_like(dy)
    _chk(lib().ora_softmax_instance_bwd(_p(dy), _p(y), _p(out), c * h * w,
                                        ctypes.c_size_t(n)), "softmax_instance_bwd")
    return out


def softmax_channel_bwd(dy, y, n, c, h, w):
    dy, y = _f(dy), _f(y)
    out = np.empty_like(dy)
    _chk(lib().ora_softmax_channel_bwd(_p(dy), _p(y), _p(out), n, c, h, w),
         "softmax_channel_bwd")
    return out


def activation_fwd(alg, x):
    x = _f(x)
    out = np.empty_like(x)
    _chk(lib().ora_activation_fwd(alg, _p(x), _p(out), ctypes.c_size_t(x.size)), "activation_fwd")
    return out


def activation_bwd(alg, dy, y, x):
    dy, y, x = _f(dy), _f(y), _f(x)
    out = np.empty_like(dy)
    _chk(lib().ora_activation_bwd(alg, _p(dy), _p(y), _p(x), _p(out),
                                  ctypes.c_size_t(dy.size)), "activation_bwd")
    return out


def conv_out_size(h, r, stride, pad):
    """narray/convolution.cpp:13-18."""
    return (h + 2 * pad - r) // stride + 1


def conv_fwd(bottom, filt, bias, N, C, K, H, W, ph, pw, sv, sh, R, S):
    bottom, filt = _f(bottom), _f(filt)
    Ho, Wo = conv_out_size(H, R, sv, ph), conv_out_size(W, S, sh, pw)
    assert bottom.size == N * C * H * W and filt.size == K * C * R * S
    out = np.empty(N * K * Ho * Wo, dtype=np.float32)
    bp = _p(_f(bias)) if bias is not None else None
    _chk(lib().ora_conv_fwd(_p(bottom), _p(filt), bp, _p(out), N, C, K, H, W, ph, pw, sv, sh,
                            R, S), "conv_fwd")
    return out


def conv_bwd_data(top_diff, filt, N, C, K, H, W, ph, pw, sv, sh, R, S):
    top_diff, filt = _f(top_diff), _f(filt)
    out = np.empty(N * C * H * W, dtype=np.float32)
    _chk(lib().ora_conv_bwd_data(_p(top_diff), _p(filt), _p(out), N, C, K, H, W, ph, pw, sv,
                                 sh, R, S), "conv_bwd_data")
    return out


def conv_bwd_filter(top_diff, bottom, N, C, K, H, W, ph, pw, sv, sh, R, S):
    top_diff, bottom = _f(top_diff), _f(bottom)
    out = np.empty(K * C * R * S, dtype=np.float32)
    _chk(lib().ora_conv_bwd_filter(_p(top_diff), _p(bottom), _p(out), N, C, K, H, W, ph, pw,
                                   sv, sh, R, S), "conv_bwd_filter")
    return out


def conv_bwd_bias(top_diff, N, K, Ho, Wo):
    top_diff = _f(top_diff)
    out = np.empty(K, dtype=np.float32)
    _chk(lib().ora_conv_bwd_bias(_p(top_diff), _p(out), N, K, Ho, Wo), "conv_bwd_bias")
    return out


def pooled_size(size, win, stride, pad):
    return lib().ora_pooled_size(size, win, stride, pad)


def pool_fwd(alg, bottom, N, C, H, W, sv, sh, kh, kw, ph, pw):
    bottom = _f(bottom)
    Ho, Wo = pooled_size(H, kh, sv, ph), pooled_size(W, kw, sh, pw)
    out = np.empty(N * C * Ho * Wo, dtype=np.float32)
    _chk(lib().ora_pool_fwd(alg, _p(bottom), _p(out), N, C, H, W, sv, sh, kh, kw, ph, pw),
         "pool_fwd")
    return out


def pool_bwd(alg, top_diff, top, bottom, N, C, H, W, sv, sh, kh, kw, ph, pw, want_mask=False):
    top_diff, top, bottom = _f(top_diff), _f(top), _f(bottom)
    out = np.empty(N * C * H * W, dtype=np.float32)
    mask = np.empty(top_diff.size, dtype=np.float32) if want_mask else None
    _chk(lib().ora_pool_bwd(alg, _p(top_diff), _p(top), _p(bottom), _p(out),
                            _p(mask) if want_mask else None, N, C, H, W, sv, sh, kh, kw, ph,
                            pw), "pool_bwd")
    return (out, mask) if want_mask else out


def lrn_fwd(bottom, local_size, alpha, beta, N, C, H, W):
    """Returns (top, scale)."""
    bottom = _f(bottom)
    scale = np.empty(bottom.size, dtype=np.float32)
    top = np.empty(bottom.size, dtype=np.float32)
    _chk(lib().ora_lrn_fwd(_p(bottom), _p(scale), _p(top), local_size, ctypes.c_float(alpha),
                           ctypes.c_float(beta), N, C, H, W), "lrn_fwd")
    return top, scale


def lrn_bwd(bottom, top, scale, top_diff, local_size, alpha, beta, N, C, H, W):
    bottom, top, scale, top_diff = _f(bottom), _f(top), _f(scale), _f(top_diff)
    out = np.empty(bottom.size, dtype=np.float32)
    _chk(lib().ora_lrn_bwd(_p(bottom), _p(top), _p(scale), _p(top_diff), _p(out), local_size,
                           ctypes.c_float(alpha), ctypes.c_float(beta), N, C, H, W), "lrn_bwd")
    return out


# Concat / Slice / Select are pure data movement on column-major tensors (reference
# minerva/op/impl/cuda.cpp:80-155, 644-655; extents minerva/narray/narray.cpp:129-192):
# numpy's own indexing on Fortran-ordered views is the closed form.
def concat(arrays, dims_list, catdim):
    views = [_f(a).reshape(d, order="F") for a, d in zip(arrays, dims_list)]
    return np.concatenate(views, axis=catdim).ravel(order="F")


def slice_(x, dims, slice_dim, st_off, slice_count):
    v = _f(x).reshape(dims, order="F")
    idx = [slice(None)] * len(dims)
    idx[slice_dim] = slice(st_off, st_off + slice_count)
    return v[tuple(idx)].ravel(order="F")


def select(x, rows, cols, indices):
    return _f(x).reshape((rows, cols), order="F")[:, list(indices)].ravel(order="F")


def philox4x32_10(ctr, key):
    c = (ctypes.c_uint32 * 4)(*ctr)
    k = (ctypes.c_uint32 * 2)(*key)
    out = (ctypes.c_uint32 * 4)()
    lib().ora_philox4x32_10(c, k, out)
    return [int(v) for v in out]


def randn(n, seed, mean, stddev):
    out = np.empty(n, dtype=np.float32)
    _chk(lib().ora_randn(_p(out), ctypes.c_size_t(n), ctypes.c_uint64(seed), ctypes.c_float(mean),
                         ctypes.c_float(stddev)), "randn")
    return out


def rand_bernoulli(n, seed, p):
    out = np.empty(n, dtype=np.float32)
    _chk(lib().ora_rand_bernoulli(_p(out), ctypes.c_size_t(n), ctypes.c_uint64(seed),
                                  ctypes.c_float(p)), "rand_bernoulli")
    return out


def threshold_norm(x, threshold):
    x = _f(x)
    out = np.empty(x.size, dtype=np.float32)
    _chk(lib().ora_threshold_norm(_p(x), _p(out), ctypes.c_size_t(x.size), ctypes.c_float(threshold)),
         "threshold_norm")
    return out
