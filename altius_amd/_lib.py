"""Loads libaltius_hip.so and declares the C ABI (include/altius_hip.h) for ctypes.

There is no fallback: if the library is missing the import of any compute path
raises, so a GPU run can never silently use something else.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libaltius_hip.so")

OK, ERR_HIP, ERR_ARG, ERR_SHAPE, ERR_UNSUPPORTED, ERR_OOM = 0, 1, 2, 3, 4, 5
MAX_RANK = 8

c_int = ctypes.c_int
c_size_t = ctypes.c_size_t
c_float = ctypes.c_float
c_void_p = ctypes.c_void_p
c_char_p = ctypes.c_char_p
c_int64 = ctypes.c_int64
P = ctypes.POINTER

_lib = None


class AltiusHipError(RuntimeError):
    """A non-zero status from the C ABI (SessionError on the reference side)."""

    def __init__(self, code, message):
        super().__init__(f"[{_CODE_NAMES.get(code, code)}] {message}")
        self.code = code
        self.message = message


_CODE_NAMES = {
    ERR_HIP: "HIP",
    ERR_ARG: "ARG",
    ERR_SHAPE: "Shape",
    ERR_UNSUPPORTED: "Message",
    ERR_OOM: "OOM",
}


def _declare(L):
    def f(name, argtypes, restype=c_int):
        fn = getattr(L, name)
        fn.argtypes = argtypes
        fn.restype = restype

    f("ahip_init", [c_int, P(c_void_p)])
    f("ahip_init_on_stream", [c_int, c_void_p, P(c_void_p)])
    f("ahip_destroy", [c_void_p])
    f("ahip_last_error", [c_void_p], c_char_p)
    f("ahip_device_count", [])
    f("ahip_malloc", [c_void_p, c_size_t, P(c_void_p)])
    f("ahip_free", [c_void_p, c_void_p])
    f("ahip_h2d_async", [c_void_p, c_void_p, c_void_p, c_size_t])
    f("ahip_d2h_async", [c_void_p, c_void_p, c_void_p, c_size_t])
    f("ahip_d2d_async", [c_void_p, c_void_p, c_void_p, c_size_t])
    f("ahip_memset_async", [c_void_p, c_void_p, c_int, c_size_t])
    f("ahip_sync", [c_void_p])
    f("ahip_host_alloc", [c_void_p, c_size_t, P(c_void_p)])
    f("ahip_host_free", [c_void_p, c_void_p])
    f("ahip_event_create", [c_void_p, P(c_void_p)])
    f("ahip_event_record", [c_void_p, c_void_p])
    f("ahip_event_synchronize", [c_void_p, c_void_p])
    f("ahip_event_elapsed_ms", [c_void_p, c_void_p, c_void_p, P(c_float)])
    f("ahip_event_destroy", [c_void_p, c_void_p])
    f("ahip_broadcast_shape", [c_int, P(c_int64), c_int, P(c_int64), P(c_int), P(c_int64)])
    f("ahip_strides_for_broadcasting", [c_int, P(c_int64), c_int, P(c_int64), P(c_int64)])
    f("ahip_binary", [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, P(c_int64), P(c_int64), P(c_int64)])
    f("ahip_unary", [c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_float, c_float])
    f("ahip_softmax_lastaxis", [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t])
    f("ahip_layernorm_lastaxis", [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_float])
    f("ahip_reduce", [c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t])


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m altius_amd.build` "
                "(there is no CPU fallback)"
            )
        L = ctypes.CDLL(LIB_PATH)
        _declare(L)
        _lib = L
    return _lib


def i64_array(values):
    values = [int(v) for v in values]
    return (c_int64 * max(len(values), 1))(*values)


def check(rc, ctx=None):
    if rc != OK:
        msg = lib().ahip_last_error(ctx)
        raise AltiusHipError(rc, msg.decode("utf-8", "replace") if msg else "")
