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


def binary(op, a, b, threads=1, strict=False, info=None, out=None):
    """out: a float32 array of the broadcast shape to write into (the reference's run_node allocates a fresh
    one per call, which is what out=None does)."""
    a = _f32(a)
    b = _f32(b)
    shape = broadcast(a.shape, b.shape)
    if shape is None:
        raise OracleError(ERR_BROADCAST, "binary")
    if out is None:
        out = np.empty(shape, dtype=np.float32)
    assert out.dtype == np.float32 and list(out.shape) == list(shape) and out.flags.c_contiguous
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


def reduce(kind, x, axes, keep_dims, strict=False, info=None, out=None):
    x = _f32(x)
    shape = reduce_shape(kind, x.shape, axes, keep_dims)
    if out is None:
        out = np.empty(shape, dtype=np.float32)
    assert out.dtype == np.float32 and list(out.shape) == list(shape) and out.flags.c_contiguous
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


def faster_pow2(p):
    """fastapprox::faster::pow2 element by element (the helper inside Erf)."""
    p = _f32(p)
    out = np.empty_like(p)
    lib().orc_faster_pow2(_fptr(p), _fptr(out), ctypes.c_size_t(p.size))
    return out


# ---- data movement and the remaining element-wise kernels ---------------------------------------

_TYPE_OF = {np.dtype(np.bool_): 0, np.dtype(np.float32): 1, np.dtype(np.int32): 2, np.dtype(np.int64): 3}
_NP_OF = {0: np.bool_, 1: np.float32, 2: np.int32, 3: np.int64}


def _c(a):
    return np.asarray(a, order="C")


def _vp(a):
    return ctypes.c_void_p(a.ctypes.data)


def _note(info, noref):
    if info is not None:
        info["no_reference_kernel"] = bool(noref.value)


def transpose(x, perm):
    x = _c(x)
    out = np.empty([x.shape[p] for p in perm], dtype=x.dtype)
    d, r = _dims(x.shape)
    pm, _ = _dims(perm)
    rc = lib().orc_transpose(_vp(x), _vp(out), x.dtype.itemsize, r, d, pm)
    if rc != OK:
        raise OracleError(rc, "transpose")
    return out


def gather(data, indices, axis=0, strict=False, info=None):
    data = _c(data)
    idx = np.asarray(indices, dtype=np.int64, order="C")
    ax = axis + data.ndim if axis < 0 else axis
    out = np.empty(data.shape[:ax] + idx.shape + data.shape[ax + 1:], dtype=data.dtype)
    d, r = _dims(data.shape)
    i_d, i_r = _dims(idx.shape)
    noref = ctypes.c_int(0)
    rc = lib().orc_gather(_vp(data), data.dtype.itemsize, r, d, axis, idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)),
                          i_r, i_d, _vp(out), int(bool(strict)), ctypes.byref(noref))
    _note(info, noref)
    if rc != OK:
        raise OracleError(rc, "gather")
    return out


def split(x, parts, axis, strict=False, info=None):
    x = _c(x)
    ax = axis + x.ndim if axis < 0 else axis
    outs = []
    for p in parts:
        shape = list(x.shape)
        shape[ax] = int(p)
        outs.append(np.empty(shape, dtype=x.dtype))
    ptrs = (ctypes.c_void_p * len(outs))(*[o.ctypes.data for o in outs])
    d, r = _dims(x.shape)
    ps, n = _dims(parts)
    noref = ctypes.c_int(0)
    rc = lib().orc_split(_vp(x), x.dtype.itemsize, r, d, axis, n, ps, ptrs, int(bool(strict)), ctypes.byref(noref))
    _note(info, noref)
    if rc != OK:
        raise OracleError(rc, "split")
    return outs


def where(cond, x, y, strict=False, info=None):
    cond = np.asarray(cond, dtype=np.bool_, order="C")
    x, y = _f32(x), _f32(y)
    out = np.empty(np.broadcast_shapes(cond.shape, x.shape, y.shape), dtype=np.float32)
    cd, cr = _dims(cond.shape)
    xd, xr = _dims(x.shape)
    yd, yr = _dims(y.shape)
    noref = ctypes.c_int(0)
    rc = lib().orc_where(cond.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), cr, cd, _fptr(x), xr, xd, _fptr(y), yr, yd,
                         _fptr(out), int(bool(strict)), ctypes.byref(noref))
    _note(info, noref)
    if rc != OK:
        raise OracleError(rc, "where")
    return out


def greater(a, b, strict=False, info=None):
    a, b = _f32(a), _f32(b)
    out = np.empty(np.broadcast_shapes(a.shape, b.shape), dtype=np.bool_)
    ad, ar = _dims(a.shape)
    bd, br = _dims(b.shape)
    noref = ctypes.c_int(0)
    rc = lib().orc_greater(_fptr(a), ar, ad, _fptr(b), br, bd, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)),
                           int(bool(strict)), ctypes.byref(noref))
    _note(info, noref)
    if rc != OK:
        raise OracleError(rc, "greater")
    return out


def cast(x, to_dtype, strict=False, info=None):
    x = _c(x)
    to_dtype = np.dtype(to_dtype)
    out = np.empty(x.shape, dtype=to_dtype)
    noref = ctypes.c_int(0)
    rc = lib().orc_cast(_vp(x), _TYPE_OF[x.dtype], _vp(out), _TYPE_OF[to_dtype], ctypes.c_size_t(x.size), int(bool(strict)),
                        ctypes.byref(noref))
    _note(info, noref)
    if rc != OK:
        raise OracleError(rc, "cast")
    return out


def batchnorm(x, scale, bias, mean, var, eps=1e-5):
    x, scale, bias, mean, var = (_f32(v) for v in (x, scale, bias, mean, var))
    n, c, h, w = x.shape
    out = np.empty_like(x)
    sz = ctypes.c_size_t
    rc = lib().orc_batchnorm(_fptr(x), _fptr(scale), _fptr(bias), _fptr(mean), _fptr(var), _fptr(out), sz(n), sz(c), sz(h),
                             sz(w), ctypes.c_float(eps))
    if rc != OK:
        raise OracleError(rc, "batchnorm")
    return out


def global_average_pool(x):
    x = _f32(x)
    n, c, h, w = x.shape
    out = np.empty((n, c, 1, 1), dtype=np.float32)
    sz = ctypes.c_size_t
    rc = lib().orc_global_average_pool(_fptr(x), _fptr(out), sz(n), sz(c), sz(h), sz(w))
    if rc != OK:
        raise OracleError(rc, "global_average_pool")
    return out


def leaky_relu(x, alpha=0.01):
    x = _f32(x)
    out = np.empty_like(x)
    rc = lib().orc_leaky_relu(_fptr(x), _fptr(out), ctypes.c_size_t(x.size), ctypes.c_float(alpha))
    if rc != OK:
        raise OracleError(rc, "leaky_relu")
    return out


def matmul(a, b):
    """compute_mat_mul (session.rs:621-684): numpy.matmul shapes, one sgemm per batch item."""
    a, b = _f32(a), _f32(b)
    m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
    batch_shape = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    af = np.ascontiguousarray(np.broadcast_to(a, batch_shape + (m, k))).reshape(-1, m, k)
    bf = np.ascontiguousarray(np.broadcast_to(b, batch_shape + (k, n))).reshape(-1, k, n)
    out = np.zeros((af.shape[0], m, n), dtype=np.float32)
    sz = ctypes.c_size_t
    for i in range(af.shape[0]):
        rc = lib().orc_sgemm(0, 0, sz(m), sz(k), sz(n), ctypes.c_float(1.0), _fptr(af[i]), sz(k), _fptr(bf[i]), sz(n),
                             ctypes.c_float(0.0), _fptr(out[i]), sz(n))
        if rc != OK:
            raise OracleError(rc, "matmul")
    return out.reshape(batch_shape + (m, n))


def gemm(a, b, c=None, alpha=1.0, beta=1.0, trans_a=False, trans_b=False):
    """compute_gemm (session.rs:686-794): C is copied (bias rows repeated) into the output, then sgemm."""
    a, b = _f32(a), _f32(b)
    m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
    n = b.shape[0] if trans_b else b.shape[1]
    out = np.zeros((m, n), dtype=np.float32)
    if c is not None:
        out[:] = np.broadcast_to(_f32(c), (m, n))
    sz = ctypes.c_size_t
    rc = lib().orc_sgemm(int(trans_a), int(trans_b), sz(m), sz(k), sz(n), ctypes.c_float(alpha), _fptr(a), sz(a.shape[1]),
                         _fptr(b), sz(b.shape[1]), ctypes.c_float(beta if c is not None else 0.0), _fptr(out), sz(n))
    if rc != OK:
        raise OracleError(rc, "gemm")
    return out


def _conv_out(n, k, s, p0, p1, d=1):
    return (n + p0 + p1 - d * (k - 1) - 1) // s + 1


def conv2d(x, w, bias=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1):
    x, w = _f32(x), _f32(w)
    b, c, ih, iw = x.shape
    oc, _, kh, kw = w.shape
    oh = _conv_out(ih, kh, strides[0], pads[0], pads[2], dilations[0])
    ow = _conv_out(iw, kw, strides[1], pads[1], pads[3], dilations[1])
    out = np.empty((b, oc, oh, ow), dtype=np.float32)
    bias_arr = _f32(bias) if bias is not None else None
    sz = ctypes.c_size_t
    rc = lib().orc_conv2d(_fptr(x), _fptr(w), _fptr(bias_arr) if bias_arr is not None else None, _fptr(out), sz(b), sz(c), sz(ih),
                          sz(iw), sz(oc), sz(oh), sz(ow), sz(kh), sz(kw), sz(strides[0]), sz(strides[1]), sz(dilations[0]),
                          sz(dilations[1]), sz(pads[0]), sz(pads[1]), sz(group))
    if rc != OK:
        raise OracleError(rc, "conv2d")
    return out


def max_pool(x, kernel, strides, pads=(0, 0, 0, 0)):
    x = _f32(x)
    b, c, ih, iw = x.shape
    oh = _conv_out(ih, kernel[0], strides[0], pads[0], pads[2])
    ow = _conv_out(iw, kernel[1], strides[1], pads[1], pads[3])
    out = np.empty((b, c, oh, ow), dtype=np.float32)
    sz = ctypes.c_size_t
    rc = lib().orc_max_pool(_fptr(x), _fptr(out), sz(b * c), sz(ih), sz(iw), sz(oh), sz(ow), sz(kernel[0]), sz(kernel[1]),
                            sz(strides[0]), sz(strides[1]), sz(pads[0]), sz(pads[1]))
    if rc != OK:
        raise OracleError(rc, "max_pool")
    return out


def resize(x, out_hw, nearest=True):
    x = _f32(x)
    b, c, ih, iw = x.shape
    out = np.empty((b, c, out_hw[0], out_hw[1]), dtype=np.float32)
    sz = ctypes.c_size_t
    rc = lib().orc_resize(_fptr(x), _fptr(out), sz(b * c), sz(ih), sz(iw), sz(out_hw[0]), sz(out_hw[1]), int(bool(nearest)))
    if rc != OK:
        raise OracleError(rc, "resize")
    return out
