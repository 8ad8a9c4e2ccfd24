"""Python handles over the device part of the C ABI: a context (device + stream),
device buffers, events, and the operator kernels on device-resident tensors.

Everything here is a thin call into libaltius_hip.so; no arithmetic happens in
Python.
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import check, i64_array

ADD, SUB, MUL, DIV, POW = 0, 1, 2, 3, 4
SQRT, ERF, GELU, SIGMOID, HARDSIGMOID, RELU, TANH, LEAKYRELU, EXP, ROUND, CLIP = range(11)
REDUCE_MEAN, REDUCE_MAX, REDUCE_SUM = 0, 1, 2
BOOL, F32, I32, I64 = 0, 1, 2, 3
GEMM_AUTO, GEMM_FP32, GEMM_BF16X3 = 0, 1, 2
GEMM_DEFAULT = GEMM_FP32  # what a new context or session uses: the reference's results for every operand value
_ELEM_OF = {np.dtype(np.bool_): BOOL, np.dtype(np.float32): F32, np.dtype(np.int32): I32, np.dtype(np.int64): I64}


def xcd_round_robin_holds(cu_count, xcc_of_block):
    """The decision a context takes from its placement probe (host only): block i ran on XCD i % 8 for every i."""
    ids = np.ascontiguousarray(xcc_of_block, dtype=np.uint32)
    return bool(_lib.lib().ahip_xcd_round_robin_holds(int(cu_count), ids.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)), ids.size))


def broadcast_shape(a_dims, b_dims):
    """fixed_dim::broadcast through the C ABI; raises AltiusHipError(Shape) if incompatible."""
    L = _lib.lib()
    rank = ctypes.c_int(0)
    out = (ctypes.c_int64 * max(len(a_dims), len(b_dims), 1))()
    check(L.ahip_broadcast_shape(len(a_dims), i64_array(a_dims), len(b_dims), i64_array(b_dims),
                                 ctypes.byref(rank), out))
    return [int(out[i]) for i in range(rank.value)]


def strides_for_broadcasting(from_dims, to_dims):
    """Tensor::strides_for_broadcasting through the C ABI."""
    L = _lib.lib()
    out = (ctypes.c_int64 * max(len(to_dims), 1))()
    check(L.ahip_strides_for_broadcasting(len(from_dims), i64_array(from_dims), len(to_dims),
                                          i64_array(to_dims), out))
    return [int(out[i]) for i in range(len(to_dims))]


class DeviceBuffer:
    """A device allocation owned by a Context."""

    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        check(ctx.L.ahip_malloc(ctx.handle, self.nbytes, ctypes.byref(p)), ctx.handle)
        self.ptr = p.value or 0

    def free(self):
        if self.ptr and self.ctx.handle:
            check(self.ctx.L.ahip_free(self.ctx.handle, self.ptr), self.ctx.handle)
        self.ptr = 0

    def offset(self, nbytes):
        return self.ptr + int(nbytes)


class Context:
    """One device + one stream.  Not thread-safe; create one per thread."""

    def __init__(self, device=0):
        self.L = _lib.lib()
        h = ctypes.c_void_p()
        check(self.L.ahip_init(int(device), ctypes.byref(h)))
        self.handle = h
        self._buffers = []

    def close(self):
        if self.handle:
            for b in self._buffers:
                b.free()
            self._buffers = []
            self.L.ahip_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # --- memory ---------------------------------------------------------
    def alloc(self, nbytes):
        b = DeviceBuffer(self, nbytes)
        self._buffers.append(b)
        return b

    def free(self, buf):
        buf.free()
        self._buffers = [b for b in self._buffers if b is not buf]

    def upload(self, array):
        """Copies a numpy array to a new device buffer."""
        a = np.asarray(array, order="C")
        buf = self.alloc(max(a.nbytes, 4))
        if a.nbytes:
            check(self.L.ahip_h2d_async(self.handle, buf.ptr, a.ctypes.data, a.nbytes), self.handle)
            self.sync()
        return buf

    def download(self, buf, shape, dtype=np.float32, offset_bytes=0):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes:
            check(self.L.ahip_d2h_async(self.handle, out.ctypes.data, buf.ptr + offset_bytes, out.nbytes),
                  self.handle)
        self.sync()
        return out

    def memset(self, buf, byte_value):
        check(self.L.ahip_memset_async(self.handle, buf.ptr, byte_value, buf.nbytes), self.handle)

    def sync(self):
        check(self.L.ahip_sync(self.handle), self.handle)

    # --- events -----------------------------------------------------------
    def event(self):
        e = ctypes.c_void_p()
        check(self.L.ahip_event_create(self.handle, ctypes.byref(e)), self.handle)
        return e

    def record(self, event):
        check(self.L.ahip_event_record(self.handle, event), self.handle)

    def elapsed_ms(self, start, stop):
        check(self.L.ahip_event_synchronize(self.handle, stop), self.handle)
        ms = ctypes.c_float(0)
        check(self.L.ahip_event_elapsed_ms(self.handle, start, stop, ctypes.byref(ms)), self.handle)
        return ms.value

    def destroy_event(self, event):
        check(self.L.ahip_event_destroy(self.handle, event), self.handle)

    # --- code objects loaded at run time ----------------------------------
    def load_module(self, image):
        """Loads a gfx950 code object (bytes) and returns its handle."""
        buf = ctypes.create_string_buffer(bytes(image), max(1, len(image)))
        m = ctypes.c_void_p()
        check(self.L.ahip_module_load(self.handle, ctypes.cast(buf, ctypes.c_void_p), len(image), ctypes.byref(m)),
              self.handle)
        return m

    def unload_module(self, module):
        check(self.L.ahip_module_unload(self.handle, module), self.handle)

    def launch(self, module, kernel, grid, block, args, shared_bytes=0):
        """Launches `kernel` of `module`; args are ctypes values (c_void_p, c_float, c_uint64 ...)."""
        u3 = ctypes.c_uint32 * 3
        ptrs = (ctypes.c_void_p * max(1, len(args)))(*[ctypes.cast(ctypes.pointer(a), ctypes.c_void_p) for a in args])
        check(self.L.ahip_launch(self.handle, module, kernel.encode(), u3(*grid), u3(*block), shared_bytes, ptrs),
              self.handle)

    # --- kernels on raw device pointers -----------------------------------
    def binary_raw(self, op, out_ptr, a_ptr, b_ptr, out_dims, a_strides, b_strides):
        check(self.L.ahip_binary(self.handle, op, out_ptr, a_ptr, b_ptr, len(out_dims), i64_array(out_dims),
                                 i64_array(a_strides), i64_array(b_strides)), self.handle)

    def unary_raw(self, op, out_ptr, in_ptr, n, alpha=0.0, beta=0.0):
        check(self.L.ahip_unary(self.handle, op, out_ptr, in_ptr, n, alpha, beta), self.handle)

    def softmax_raw(self, out_ptr, in_ptr, rows, length):
        check(self.L.ahip_softmax_lastaxis(self.handle, out_ptr, in_ptr, rows, length), self.handle)

    def layernorm_raw(self, out_ptr, in_ptr, gamma_ptr, beta_ptr, rows, length, eps):
        check(self.L.ahip_layernorm_lastaxis(self.handle, out_ptr, in_ptr, gamma_ptr, beta_ptr, rows, length,
                                             eps), self.handle)

    def reduce_raw(self, kind, out_ptr, in_ptr, outer, red, inner):
        check(self.L.ahip_reduce(self.handle, kind, out_ptr, in_ptr, outer, red, inner), self.handle)

    def reduce_static_raw(self, kind, out_ptr, in_ptr, outer, red, inner):
        """ahip_reduce_static: the reduction that allocates nothing (partial results in a fixed array)."""
        check(self.L.ahip_reduce_static(self.handle, kind, out_ptr, in_ptr, outer, red, inner), self.handle)

    # --- convenience: numpy in, numpy out (upload, one kernel, download) ----
    def binary(self, op, a, b):
        a = np.asarray(a, dtype=np.float32, order="C")
        b = np.asarray(b, dtype=np.float32, order="C")
        out_dims = broadcast_shape(a.shape, b.shape)
        a_str = strides_for_broadcasting(a.shape, out_dims)
        b_str = strides_for_broadcasting(b.shape, out_dims)
        n = int(np.prod(out_dims, dtype=np.int64)) if out_dims else 1
        da, db = self.upload(a), self.upload(b)
        do = self.alloc(max(n * 4, 4))
        try:
            self.binary_raw(op, do.ptr, da.ptr, db.ptr, out_dims, a_str, b_str)
            return self.download(do, out_dims)
        finally:
            for x in (da, db, do):
                self.free(x)

    def unary(self, op, x, alpha=0.0, beta=0.0):
        x = np.asarray(x, dtype=np.float32, order="C")
        dx = self.upload(x)
        do = self.alloc(max(x.nbytes, 4))
        try:
            self.unary_raw(op, do.ptr, dx.ptr, x.size, alpha, beta)
            return self.download(do, x.shape)
        finally:
            self.free(dx)
            self.free(do)

    def fused_use_compiled_chains(self, enable):
        """False: every chain takes the interpreting kernel, also those the library has compiled code for."""
        check(self.L.ahip_fused_use_compiled_chains(self.handle, int(bool(enable))), self.handle)

    def fused_elemwise(self, inputs, steps):
        """A chain of element-wise steps in one kernel.  inputs: f32 arrays that broadcast to a common shape;
        steps: (kind, op, lhs, rhs[, alpha, beta, pow_scalar_exponent]) with kind "b" (binary, op = ADD..POW) or
        "u" (unary, op = SQRT..), lhs / rhs an index into inputs or _lib.FUSED_ACC.  Returns the last step's
        result at the broadcast shape."""
        arrays = [np.asarray(a, dtype=np.float32, order="C") for a in inputs]
        shape = np.broadcast_shapes(*[a.shape for a in arrays])
        bufs = [self.upload(a) for a in arrays]
        n = int(np.prod(shape, dtype=np.int64))
        out = self.alloc(max(n * 4, 4))
        stride_arrays = [i64_array(strides_for_broadcasting(a.shape, shape)) if len(shape) else i64_array([0]) for a in arrays]
        strides = (ctypes.POINTER(ctypes.c_int64) * len(arrays))(
            *[ctypes.cast(s, ctypes.POINTER(ctypes.c_int64)) for s in stride_arrays])
        ptrs = (ctypes.c_void_p * len(arrays))(*[b.ptr for b in bufs])
        c_steps = (_lib.FusedStep * len(steps))()
        for i, st in enumerate(steps):
            kind, op, lhs, rhs = st[:4]
            extra = list(st[4:]) + [0.0, 0.0, 0][len(st) - 4:]
            c_steps[i] = _lib.FusedStep(1 if kind == "u" else 0, op, lhs, rhs, extra[0], extra[1], int(extra[2]))
        try:
            check(self.L.ahip_fused_elemwise(self.handle, out.ptr, len(shape), i64_array(shape) if len(shape) else None,
                                             len(arrays), ptrs, strides, len(steps), c_steps), self.handle)
            return self.download(out, shape)
        finally:
            for b in bufs + [out]:
                self.free(b)

    def softmax(self, x):
        x = np.asarray(x, dtype=np.float32, order="C")
        length = x.shape[-1]
        rows = x.size // length if length else 0
        dx = self.upload(x)
        do = self.alloc(max(x.nbytes, 4))
        try:
            self.softmax_raw(do.ptr, dx.ptr, rows, length)
            return self.download(do, x.shape)
        finally:
            self.free(dx)
            self.free(do)

    def softmax_prologue(self, x, scale_op=0, scale=1.0, mask=None):
        """softmax((x [*|/] scale) + mask) in one kernel; scale_op 0 none, 1 multiply, 2 divide; mask holds
        x.size / (mask rows * length) consecutive rows of x per mask row."""
        x = np.asarray(x, dtype=np.float32, order="C")
        length = x.shape[-1]
        rows = x.size // length if length else 0
        dx = self.upload(x)
        do = self.alloc(max(x.nbytes, 4))
        dm, rpm = None, 0
        if mask is not None:
            mask = np.asarray(mask, dtype=np.float32, order="C")
            assert mask.shape[-1] == length and rows % (mask.size // length) == 0
            rpm = rows // (mask.size // length)
            dm = self.upload(mask)
        try:
            check(self.L.ahip_softmax_lastaxis_prologue(self.handle, do.ptr, dx.ptr, rows, length, scale_op, float(scale),
                                                        dm.ptr if dm else None, rpm), self.handle)
            return self.download(do, x.shape)
        finally:
            for b in (dx, do, dm):
                if b is not None:
                    self.free(b)

    def layer_norm(self, x, gamma, beta, eps=1e-5):
        x = np.asarray(x, dtype=np.float32, order="C")
        gamma = np.asarray(gamma, dtype=np.float32, order="C")
        beta = np.asarray(beta, dtype=np.float32, order="C")
        length = x.shape[-1]
        assert gamma.size == length and beta.size == length
        rows = x.size // length if length else 0
        dx, dg, db = self.upload(x), self.upload(gamma), self.upload(beta)
        do = self.alloc(max(x.nbytes, 4))
        try:
            self.layernorm_raw(do.ptr, dx.ptr, dg.ptr, db.ptr, rows, length, eps)
            return self.download(do, x.shape)
        finally:
            for t in (dx, dg, db, do):
                self.free(t)

    def reduce(self, kind, x, outer, red, inner):
        """Reduces the middle axis of x viewed as [outer, red, inner]; returns [outer, inner]."""
        x = np.asarray(x, dtype=np.float32, order="C")
        assert x.size == outer * red * inner
        dx = self.upload(x)
        do = self.alloc(max(outer * inner * 4, 4))
        try:
            self.reduce_raw(kind, do.ptr, dx.ptr, outer, red, inner)
            return self.download(do, (outer, inner))
        finally:
            self.free(dx)
            self.free(do)


    # --- data movement: numpy in, numpy out -------------------------------------------------------
    def _upload_any(self, a):
        a = np.asarray(a, order="C")
        if a.dtype not in _ELEM_OF:
            raise TypeError(f"unsupported dtype {a.dtype}")
        return a, self.upload(a)

    def copy_strided(self, x, dims, out_strides, in_strides, out_shape, in_offset=0, out_offset=0, out_init=None):
        """One ahip_copy_strided over a fresh (or given) output array; offsets are in elements."""
        x, dx = self._upload_any(x)
        out = np.zeros(out_shape, x.dtype) if out_init is None else np.asarray(out_init, dtype=x.dtype, order="C")
        do = self.upload(out) if out.size else self.alloc(4)
        try:
            isz = x.dtype.itemsize
            check(self.L.ahip_copy_strided(self.handle, do.ptr + out_offset * isz, dx.ptr + in_offset * isz, isz, len(dims),
                                           i64_array(dims), i64_array(out_strides), i64_array(in_strides)), self.handle)
            return self.download(do, out.shape, x.dtype)
        finally:
            self.free(dx)
            self.free(do)

    def transpose(self, x, perm):
        x, dx = self._upload_any(x)
        shape = [x.shape[p] for p in perm]
        do = self.alloc(max(x.nbytes, 4))
        try:
            check(self.L.ahip_transpose(self.handle, do.ptr, dx.ptr, x.dtype.itemsize, x.ndim, i64_array(x.shape),
                                        i64_array(perm)), self.handle)
            return self.download(do, shape, x.dtype)
        finally:
            self.free(dx)
            self.free(do)

    def gather(self, data, indices, axis=0):
        data, dd = self._upload_any(data)
        idx = np.asarray(indices, order="C")
        if idx.dtype not in (np.int32, np.int64):
            idx = idx.astype(np.int64)
        di = self.upload(idx)
        ax = axis + data.ndim if axis < 0 else axis
        shape = data.shape[:ax] + idx.shape + data.shape[ax + 1:]
        outer = int(np.prod(data.shape[:ax], dtype=np.int64))
        inner = int(np.prod(data.shape[ax + 1:], dtype=np.int64))
        do = self.alloc(max(int(np.prod(shape, dtype=np.int64)) * data.dtype.itemsize, 4))
        try:
            check(self.L.ahip_gather(self.handle, do.ptr, dd.ptr, di.ptr, idx.dtype.itemsize, data.dtype.itemsize, outer,
                                     data.shape[ax], idx.size, inner), self.handle)
            return self.download(do, shape, data.dtype)      # download synchronises: a bad index raises here
        finally:
            for b in (dd, di, do):
                self.free(b)

    def where(self, cond, x, y):
        cond = np.asarray(cond, dtype=np.bool_, order="C")
        x, dx = self._upload_any(x)
        y = np.asarray(y, dtype=x.dtype, order="C")
        dc, dy = self.upload(cond), self.upload(y)
        dims = list(np.broadcast_shapes(cond.shape, x.shape, y.shape))
        st = [strides_for_broadcasting(a.shape, dims) for a in (cond, x, y)]
        n = int(np.prod(dims, dtype=np.int64))
        do = self.alloc(max(n * x.dtype.itemsize, 4))
        try:
            check(self.L.ahip_where(self.handle, do.ptr, dc.ptr, dx.ptr, dy.ptr, x.dtype.itemsize, len(dims), i64_array(dims),
                                    i64_array(st[0]), i64_array(st[1]), i64_array(st[2])), self.handle)
            return self.download(do, dims, x.dtype)
        finally:
            for b in (dc, dx, dy, do):
                self.free(b)

    def greater(self, a, b):
        a = np.asarray(a, dtype=np.float32, order="C")
        b = np.asarray(b, dtype=np.float32, order="C")
        dims = list(np.broadcast_shapes(a.shape, b.shape))
        da, db = self.upload(a), self.upload(b)
        n = int(np.prod(dims, dtype=np.int64))
        do = self.alloc(max(n, 4))
        try:
            check(self.L.ahip_greater(self.handle, do.ptr, da.ptr, db.ptr, len(dims), i64_array(dims),
                                      i64_array(strides_for_broadcasting(a.shape, dims)),
                                      i64_array(strides_for_broadcasting(b.shape, dims))), self.handle)
            return self.download(do, dims, np.bool_)
        finally:
            for x in (da, db, do):
                self.free(x)

    def cast(self, x, to_dtype):
        x, dx = self._upload_any(x)
        to_dtype = np.dtype(to_dtype)
        do = self.alloc(max(x.size * to_dtype.itemsize, 4))
        try:
            check(self.L.ahip_cast(self.handle, do.ptr, dx.ptr, _ELEM_OF[x.dtype], _ELEM_OF[to_dtype], x.size), self.handle)
            return self.download(do, x.shape, to_dtype)
        finally:
            self.free(dx)
            self.free(do)

    def batchnorm(self, x, scale, bias, mean, var, eps=1e-5):
        arrs = [np.asarray(a, dtype=np.float32, order="C") for a in (x, scale, bias, mean, var)]
        n, c, h, w = arrs[0].shape
        bufs = [self.upload(a) for a in arrs]
        do = self.alloc(max(arrs[0].nbytes, 4))
        try:
            check(self.L.ahip_batchnorm(self.handle, do.ptr, *[b.ptr for b in bufs], n, c, h * w, eps), self.handle)
            return self.download(do, arrs[0].shape)
        finally:
            for b in bufs + [do]:
                self.free(b)

    # --- matrix multiplication -------------------------------------------------------------------
    def gemm_raw(self, c_ptr, a_ptr, b_ptr, c0_ptr, batch, m, n, k, trans_a=False, trans_b=False, lda=None, ldb=None,
                 ldc=None, a_bs=0, b_bs=0, c_bs=0, c0_rs=0, c0_cs=0, alpha=1.0, beta=0.0):
        lda = lda if lda is not None else (m if trans_a else k)
        ldb = ldb if ldb is not None else (k if trans_b else n)
        ldc = ldc if ldc is not None else n
        check(self.L.ahip_gemm(self.handle, c_ptr, a_ptr, b_ptr, c0_ptr, batch, m, n, k, int(trans_a), int(trans_b), lda,
                               ldb, ldc, a_bs, b_bs, c_bs, c0_rs, c0_cs, alpha, beta), self.handle)

    def attention(self, q, k, v, scale_op=0, scale=1.0, mask=None):
        """Softmax(scale(Q K^T) + mask) V for q [..., tq, 64], k / v [..., tk, 64] (same leading shape), in one kernel;
        mask: [tk] (shared) or [q.shape[0], tk] (one row per leading batch)."""
        q, k, v = (np.asarray(x, dtype=np.float32, order="C") for x in (q, k, v))
        tq, d = q.shape[-2:]
        tk = k.shape[-2]
        batch = int(np.prod(q.shape[:-2], dtype=np.int64))
        dq, dk, dv = self.upload(q), self.upload(k), self.upload(v)
        do = self.alloc(max(q.nbytes, 4))
        S = ctypes.c_size_t * 2
        dm, outer, inner, mstride = None, batch, 1, 0
        if mask is not None:
            mask = np.asarray(mask, dtype=np.float32, order="C")
            dm = self.upload(mask)
            if mask.ndim == 2:
                outer, inner, mstride = q.shape[0], batch // q.shape[0], tk
        try:
            check(self.L.ahip_attention(self.handle, do.ptr, dq.ptr, dk.ptr, dv.ptr, outer, inner, tq, tk, d, d, d, d, d,
                                        S(inner * tq * d, tq * d), S(inner * tk * d, tk * d), S(inner * tk * d, tk * d),
                                        S(inner * tq * d, tq * d), scale_op, scale, dm.ptr if dm else None, mstride), self.handle)
            return self.download(do, q.shape)
        finally:
            for x in (dq, dk, dv, do) + ((dm,) if dm else ()):
                self.free(x)

    def gemm_set_algorithm(self, algorithm):
        """GEMM_AUTO / GEMM_FP32 / GEMM_BF16X3: the kernel single-batch products take."""
        check(self.L.ahip_gemm_set_algorithm(self.handle, int(algorithm)), self.handle)

    def set_streaming_threshold(self, nbytes):
        """Tensors of at least this many bytes are streamed with non-temporal accesses."""
        check(self.L.ahip_set_streaming_threshold(self.handle, int(nbytes)), self.handle)

    def set_load_streaming_threshold(self, nbytes):
        """Element-wise operators read dense operands of at least this many bytes with non-temporal loads."""
        check(self.L.ahip_set_load_streaming_threshold(self.handle, int(nbytes)), self.handle)

    def gemm_in_kernel_k_cut(self):
        """(placement shown, cut enabled): whether the probe at context creation found block i on XCD i % 8, and
        whether the bf16 GEMM's in-kernel k cut is switched on.  The cut runs only when both hold."""
        shown, enabled = ctypes.c_int(), ctypes.c_int()
        check(self.L.ahip_gemm_in_kernel_k_cut(self.handle, ctypes.byref(shown), ctypes.byref(enabled)), self.handle)
        return bool(shown.value), bool(enabled.value)

    def gemm_set_in_kernel_k_cut(self, enable):
        check(self.L.ahip_gemm_set_in_kernel_k_cut(self.handle, int(bool(enable))), self.handle)

    def gemm_register_constant(self, buf):
        """Declares a device buffer immutable: the split GEMM keeps the planes of operands inside it."""
        check(self.L.ahip_gemm_register_constant(self.handle, buf.ptr, buf.nbytes), self.handle)

    def gemm_unregister_constant(self, buf):
        check(self.L.ahip_gemm_unregister_constant(self.handle, buf.ptr), self.handle)

    def matmul(self, a, b):
        """numpy.matmul semantics for operands of rank >= 2 (batch axes broadcast)."""
        a = np.asarray(a, dtype=np.float32, order="C")
        b = np.asarray(b, dtype=np.float32, order="C")
        m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
        batch_shape = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
        batch = int(np.prod(batch_shape, dtype=np.int64))
        # batched operands are made dense over the broadcast batch unless they are a single shared matrix
        def prep(x):
            if x.ndim == 2 or int(np.prod(x.shape[:-2], dtype=np.int64)) == 1:
                return np.ascontiguousarray(x.reshape(x.shape[-2:])), 0
            full = np.ascontiguousarray(np.broadcast_to(x, batch_shape + x.shape[-2:]))
            return full, x.shape[-2] * x.shape[-1]
        a2, a_bs = prep(a)
        b2, b_bs = prep(b)
        da, db = self.upload(a2), self.upload(b2)
        dc = self.alloc(max(batch * m * n * 4, 4))
        try:
            self.gemm_raw(dc.ptr, da.ptr, db.ptr, None, batch, m, n, k, a_bs=a_bs, b_bs=b_bs, c_bs=m * n)
            return self.download(dc, batch_shape + (m, n))
        finally:
            for x in (da, db, dc):
                self.free(x)

    def gemm(self, a, b, c=None, alpha=1.0, beta=1.0, trans_a=False, trans_b=False):
        a = np.asarray(a, dtype=np.float32, order="C")
        b = np.asarray(b, dtype=np.float32, order="C")
        m, k = (a.shape[1], a.shape[0]) if trans_a else a.shape
        n = b.shape[0] if trans_b else b.shape[1]
        da, db = self.upload(a), self.upload(b)
        dc0, rs, cs = None, 0, 0
        if c is not None:
            c = np.asarray(c, dtype=np.float32, order="C")
            dc0 = self.upload(c)
            if c.ndim == 2:
                rs, cs = (c.shape[1] if c.shape[0] != 1 else 0), (1 if c.shape[1] != 1 else 0)
            elif c.ndim == 1:
                rs, cs = 0, (1 if c.shape[0] != 1 else 0)
        dout = self.alloc(max(m * n * 4, 4))
        try:
            self.gemm_raw(dout.ptr, da.ptr, db.ptr, dc0.ptr if dc0 else None, 1, m, n, k, trans_a, trans_b, c0_rs=rs,
                          c0_cs=cs, alpha=alpha, beta=beta)
            return self.download(dout, (m, n))
        finally:
            for x in (da, db, dout) + ((dc0,) if dc0 else ()):
                self.free(x)

    def conv2d(self, x, w, bias=None, strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1):
        x = np.asarray(x, dtype=np.float32, order="C")
        w = np.asarray(w, dtype=np.float32, order="C")
        b, c, ih, iw = x.shape
        oc, _, kh, kw = w.shape
        oh = (ih + pads[0] + pads[2] - dilations[0] * (kh - 1) - 1) // strides[0] + 1
        ow = (iw + pads[1] + pads[3] - dilations[1] * (kw - 1) - 1) // strides[1] + 1
        dx, dw = self.upload(x), self.upload(w)
        db = self.upload(np.asarray(bias, dtype=np.float32)) if bias is not None else None
        dcol = self.alloc(max(b * c * kh * kw * oh * ow * 4, 4))
        do = self.alloc(max(b * oc * oh * ow * 4, 4))
        try:
            check(self.L.ahip_conv2d(self.handle, do.ptr, dx.ptr, dw.ptr, db.ptr if db else None, dcol.ptr, b, c, ih, iw, oc, oh, ow,
                                     kh, kw, strides[0], strides[1], dilations[0], dilations[1], pads[0], pads[1], group), self.handle)
            return self.download(do, (b, oc, oh, ow))
        finally:
            for t in (dx, dw, dcol, do) + ((db,) if db else ()):
                self.free(t)

    def max_pool(self, x, kernel, strides, pads=(0, 0, 0, 0)):
        x = np.asarray(x, dtype=np.float32, order="C")
        b, c, ih, iw = x.shape
        oh = (ih + pads[0] + pads[2] - kernel[0]) // strides[0] + 1
        ow = (iw + pads[1] + pads[3] - kernel[1]) // strides[1] + 1
        dx = self.upload(x)
        do = self.alloc(max(b * c * oh * ow * 4, 4))
        try:
            check(self.L.ahip_maxpool(self.handle, do.ptr, dx.ptr, b * c, ih, iw, oh, ow, kernel[0], kernel[1], strides[0], strides[1],
                                      pads[0], pads[1]), self.handle)
            return self.download(do, (b, c, oh, ow))
        finally:
            self.free(dx)
            self.free(do)

    def resize(self, x, out_hw, nearest=True):
        x = np.asarray(x, dtype=np.float32, order="C")
        b, c, ih, iw = x.shape
        dx = self.upload(x)
        do = self.alloc(max(b * c * out_hw[0] * out_hw[1] * 4, 4))
        try:
            check(self.L.ahip_resize(self.handle, do.ptr, dx.ptr, b * c, ih, iw, out_hw[0], out_hw[1], int(nearest)), self.handle)
            return self.download(do, (b, c, out_hw[0], out_hw[1]))
        finally:
            self.free(dx)
            self.free(do)
