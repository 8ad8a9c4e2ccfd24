"""ctypes binding of the CPU oracle (oracle/oracle.cpp).

Test infrastructure only: tests, the smoke check and the benchmark's
cpu_baseline leg import this; the shipped package never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")

ADD, SUB, MUL, DIV, POW = 0, 1, 2, 3, 4
SQRT, ERF, GELU, SIGMOID, HARDSIGMOID, RELU, TANH = 0, 1, 2, 3, 4, 5, 6
REDUCE_MEAN, REDUCE_MAX = 0, 1

OK, ERR_BROADCAST, ERR_UNSUPPORTED, ERR_ARG = 0, 1, 2, 3


class OracleError(RuntimeError):
    def __init__(self, code, what):
        super().__init__(f"{what}: oracle error {code}")
        self.code = code


def build(force=False):
    """Compile oracle/liboracle.so with the committed Makefile."""
    if force and os.path.exists(LIB_PATH):
        os.remove(LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])
    return LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        L.orc_fast_sum.restype = ctypes.c_float
        L.orc_fast_sum_squares.restype = ctypes.c_float
        _lib = L
    return _lib


def _dims(d):
    d = [int(x) for x in d]
    return (ctypes.c_int64 * max(len(d), 1))(*d), len(d)


def _fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _f32(a):
    a = np.asarray(a, dtype=np.float32, order="C")
    return a


def is_scalar(dims):
    d, r = _dims(dims)
    return bool(lib().orc_is_scalar(r, d))


def broadcast(*shapes):
    """Returns the broadcast shape as a list, or None if incompatible."""
    n = len(shapes)
    ranks = (ctypes.c_int * n)(*[len(s) for s in shapes])
    arrs = [_dims(s)[0] for s in shapes]
    ptrs = (ctypes.POINTER(ctypes.c_int64) * n)(
        *[ctypes.cast(a, ctypes.POINTER(ctypes.c_int64)) for a in arrs]
    )
    max_rank = max([len(s) for s in shapes] + [1])
    out = (ctypes.c_int64 * max_rank)()
    out_rank = ctypes.c_int(0)
    rc = lib().orc_broadcast(n, ranks, ptrs, ctypes.byref(out_rank), out)
    if rc != OK:
        return None
    return [int(out[i]) for i in range(out_rank.value)]


def strides_for_broadcasting(from_dims, to_dims):
    fd, fr = _dims(from_dims)
    td, tr = _dims(to_dims)
    out = (ctypes.c_int64 * max(tr, 1))()
    rc = lib().orc_strides_for_broadcasting(fr, fd, tr, td, out)
    if rc != OK:
        return None
    return [int(out[i]) for i in range(tr)]


def compute_strides(dims):
    d, r = _dims(dims)
    out = (ctypes.c_int64 * max(r, 1))()
    lib().orc_compute_strides(r, d, out)
    return [int(out[i]) for i in range(r)]


def reduce_shape(kind, dims, axes, keep_dims):
    d, r = _dims(dims)
    ax, na = _dims(axes)
    out = (ctypes.c_int64 * max(r, 1))()
    out_rank = ctypes.c_int(0)
    rc = lib().orc_reduce_shape(kind, r, d, na, ax, int(bool(keep_dims)), ctypes.byref(out_rank), out)
    if rc != OK:
        raise OracleError(rc, "reduce_shape")
    return [int(out[i]) for i in range(out_rank.value)]


def binary(op, a, b, threads=1, strict=False, info=None):
    a = _f32(a)
    b = _f32(b)
    shape = broadcast(a.shape, b.shape)
    if shape is None:
        raise OracleError(ERR_BROADCAST, "binary")
    out = np.empty(shape, dtype=np.float32)
    ad, ar = _dims(a.shape)
    bd, br = _dims(b.shape)
    noref = ctypes.c_int(0)
    rc = lib().orc_binary(op, _fptr(a), ar, ad, _fptr(b), br, bd, _fptr(out), int(threads),
                          int(bool(strict)), ctypes.byref(noref))
    if rc != OK:
        raise OracleError(rc, "binary")
    if info is not None:
        info["no_reference_kernel"] = bool(noref.value)
    return out


def unary(op, x, alpha=0.0, beta=0.0, threads=1, out=None):
    x = _f32(x)
    if out is None:
        out = np.empty_like(x)
    rc = lib().orc_unary(op, _fptr(x), _fptr(out), ctypes.c_size_t(x.size), ctypes.c_float(alpha),
                         ctypes.c_float(beta), int(threads))
    if rc != OK:
        raise OracleError(rc, "unary")
    return out


def softmax(x, threads=1, out=None):
    x = _f32(x)
    length = x.shape[-1] if x.ndim else 1
    rows = x.size // length if length else 0
    if out is None:
        out = np.empty_like(x)
    rc = lib().orc_softmax(_fptr(x), _fptr(out), ctypes.c_size_t(rows), ctypes.c_size_t(length),
                           int(threads))
    if rc != OK:
        raise OracleError(rc, "softmax")
    return out


def layer_norm(x, scale, bias, eps=1e-5, threads=1, out=None):
    x = _f32(x)
    scale = _f32(scale)
    bias = _f32(bias)
    length = x.shape[-1]
    assert scale.size == length and bias.size == length
    rows = x.size // length if length else 0
    if out is None:
        out = np.empty_like(x)
    rc = lib().orc_layer_norm(_fptr(x), _fptr(scale), _fptr(bias), _fptr(out), ctypes.c_size_t(rows),
                              ctypes.c_size_t(length), ctypes.c_float(eps), int(threads))
    if rc != OK:
        raise OracleError(rc, "layer_norm")
    return out


def reduce(kind, x, axes, keep_dims, strict=False, info=None):
    x = _f32(x)
    shape = reduce_shape(kind, x.shape, axes, keep_dims)
    out = np.empty(shape, dtype=np.float32)
    d, r = _dims(x.shape)
    ax, na = _dims(axes)
    noref = ctypes.c_int(0)
    nan = ctypes.c_int(0)
    rc = lib().orc_reduce(kind, _fptr(x), r, d, na, ax, int(bool(keep_dims)), _fptr(out),
                          int(bool(strict)), ctypes.byref(noref), ctypes.byref(nan))
    if rc != OK:
        raise OracleError(rc, "reduce")
    if info is not None:
        info["no_reference_kernel"] = bool(noref.value)
        info["saw_nan"] = bool(nan.value)
    return out


def fast_sum(x):
    x = _f32(x)
    return np.float32(lib().orc_fast_sum(_fptr(x), ctypes.c_size_t(x.size)))


def fast_sum_squares(x):
    x = _f32(x)
    return np.float32(lib().orc_fast_sum_squares(_fptr(x), ctypes.c_size_t(x.size)))
