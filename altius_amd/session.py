"""HipSessionBuilder / HipSession: the MI355X stand-in for altius's
InterpreterSessionBuilder / InterpreterSession, over the C ABI."""
import ctypes

import numpy as np

from . import _lib
from ._lib import check
from .graph import _ELEM_OF, _NP_OF, Model, Tensor


class DeviceTensor:
    """An output of HipSession.run_device: memory on the session's GPU, released by free() (or when
    the object is dropped)."""

    def __init__(self, handle):
        self.L = _lib.lib()
        self.handle = handle

    def __del__(self):
        self.free()

    def free(self):
        if getattr(self, "handle", None):
            self.L.ahip_device_tensor_free(self.handle)
            self.handle = None

    @property
    def ptr(self):
        return self.L.ahip_device_tensor_ptr(self.handle) or 0

    @property
    def shape(self):
        rank = self.L.ahip_device_tensor_rank(self.handle)
        dims = (ctypes.c_int64 * max(rank, 1))()
        check(self.L.ahip_device_tensor_dims(self.handle, dims, rank))
        return tuple(dims[i] for i in range(rank))

    @property
    def dtype(self):
        return np.dtype(_NP_OF[self.L.ahip_device_tensor_elem_type(self.handle)])

    @property
    def nbytes(self):
        return self.L.ahip_device_tensor_nbytes(self.handle)


class HipSession:
    def __init__(self, handle):
        self.L = _lib.lib()
        self.handle = handle

    def __del__(self):
        self.close()

    def close(self):
        if getattr(self, "handle", None):
            self.L.ahip_session_free(self.handle)
            self.handle = None

    def model(self):
        """A borrowed view of the session's model (valid while the session lives)."""
        return Model(_handle=ctypes.c_void_p(self.L.ahip_session_model(self.handle)), _borrowed=True)

    def run(self, inputs, copy=True):
        """inputs: numpy arrays or Tensors, positional in graph.inputs order.  Returns numpy arrays
        in graph.outputs order; with copy=False they are views of the output tensors' own memory."""
        tensors = [t if isinstance(t, Tensor) else Tensor.from_numpy(t) for t in inputs]
        arr = (ctypes.c_void_p * max(len(tensors), 1))(*[t.handle for t in tensors])
        cap = 16
        outs = (ctypes.c_void_p * cap)()
        n = ctypes.c_int()
        check(self.L.ahip_session_run(self.handle, len(tensors), arr, cap, outs, ctypes.byref(n)))
        tensors_out = [Tensor(ctypes.c_void_p(outs[i])) for i in range(n.value)]
        return [t.numpy() if copy else t.view() for t in tensors_out]

    def prepare_device_inputs(self, inputs):
        """The C arguments of run_device for these (device pointer, shape, numpy dtype) triples, built once: a loop that
        calls the same graph on the same buffers passes them to run_device_prepared and pays for the call alone."""
        n_in = len(inputs)
        ptrs = (ctypes.c_void_p * max(n_in, 1))(*[int(p) for p, _, _ in inputs])
        elem = (ctypes.c_int * max(n_in, 1))(*[_ELEM_OF[np.dtype(dt)] for _, _, dt in inputs])
        ranks = (ctypes.c_int * max(n_in, 1))(*[len(shape) for _, shape, _ in inputs])
        dim_arrays = [(ctypes.c_int64 * max(len(shape), 1))(*[int(d) for d in shape]) for _, shape, _ in inputs]
        dims = (ctypes.POINTER(ctypes.c_int64) * max(n_in, 1))(*[ctypes.cast(a, ctypes.POINTER(ctypes.c_int64)) for a in dim_arrays])
        cap = 16
        return (n_in, ptrs, elem, ranks, dims, cap, (ctypes.c_void_p * cap)(), ctypes.c_int(), dim_arrays)

    def run_device_prepared(self, prepared):
        n_in, ptrs, elem, ranks, dims, cap, outs, n, _ = prepared
        check(self.L.ahip_session_run_device(self.handle, n_in, ptrs, elem, ranks, dims, cap, outs, ctypes.byref(n)))
        return [DeviceTensor(ctypes.c_void_p(outs[i])) for i in range(n.value)]

    def run_device(self, inputs):
        """inputs: (device pointer, shape, numpy dtype) triples, positional in graph.inputs order, on the
        session's GPU.  Enqueues the plan and returns DeviceTensors without waiting for the GPU; call
        synchronize() before reading them from another stream or copying them out."""
        return self.run_device_prepared(self.prepare_device_inputs(inputs))

    def synchronize(self):
        check(self.L.ahip_session_synchronize(self.handle))

    def profile(self):
        """{op name: device milliseconds} of the last run (profiling enabled)."""
        count = ctypes.c_int()
        check(self.L.ahip_session_profile(self.handle, -1, None, None, ctypes.byref(count)))
        out = {}
        for i in range(count.value):
            name, ms = ctypes.c_char_p(), ctypes.c_double()
            check(self.L.ahip_session_profile(self.handle, i, ctypes.byref(name), ctypes.byref(ms), None))
            out[name.value.decode()] = ms.value
        return out

    def last_run_ms(self):
        ms = ctypes.c_double()
        check(self.L.ahip_session_last_run_ms(self.handle, ctypes.byref(ms)))
        return ms.value

    def last_device_ms(self):
        """Device time of the last run's kernels alone (uploads and downloads excluded)."""
        ms = ctypes.c_double()
        check(self.L.ahip_session_last_device_ms(self.handle, ctypes.byref(ms)))
        return ms.value

    def graph_replays(self):
        c = ctypes.c_size_t()
        check(self.L.ahip_session_graph_replays(self.handle, ctypes.byref(c)))
        return c.value

    def copies_avoided(self):
        """Nodes of the last node-by-node run served without their copy (views taken, layouts written in place)."""
        c = ctypes.c_size_t()
        check(self.L.ahip_session_copies_avoided(self.handle, ctypes.byref(c)))
        return c.value

    def lanes(self):
        """Streams (each with a buffer pool and a copy of the initializers) the session holds so far: 1 until two
        run() calls have overlapped."""
        c = ctypes.c_size_t()
        check(self.L.ahip_session_lanes(self.handle, ctypes.byref(c)))
        return c.value

    def device_allocations(self):
        c = ctypes.c_size_t()
        check(self.L.ahip_session_device_allocations(self.handle, ctypes.byref(c)))
        return c.value


class HipSessionBuilder:
    """HipSessionBuilder(model).with_intra_op_num_threads(n).with_profiling_enabled(b).build()"""

    def __init__(self, model):
        self.L = _lib.lib()
        h = ctypes.c_void_p()
        check(self.L.ahip_session_builder_new(model.handle, ctypes.byref(h)))
        self.handle = h

    def __del__(self):
        if getattr(self, "handle", None):
            self.L.ahip_session_builder_free(self.handle)
            self.handle = None

    def with_intra_op_num_threads(self, n):
        check(self.L.ahip_session_builder_with_intra_op_num_threads(self.handle, n))
        return self

    def with_profiling_enabled(self, enable):
        check(self.L.ahip_session_builder_with_profiling_enabled(self.handle, int(bool(enable))))
        return self

    def with_device_timing(self, enable=True):
        """Bracket every run by two events so that last_device_ms() can report the kernels' time (default on)."""
        check(self.L.ahip_session_builder_with_device_timing(self.handle, int(bool(enable))))
        return self

    def with_graph_replay(self, enable=True):
        """Record each input-shape signature as a HIP graph on its second run and replay it afterwards."""
        check(self.L.ahip_session_builder_with_graph_replay(self.handle, int(bool(enable))))
        return self

    def with_gemm_algorithm(self, algorithm):
        """device.GEMM_FP32 (default: the reference's results for every operand value) / GEMM_AUTO / GEMM_BF16X3
        for the large single-batch products."""
        check(self.L.ahip_session_builder_with_gemm_algorithm(self.handle, int(algorithm)))
        return self

    def with_fused_attention(self, enable=True):
        """MatMul -> Softmax -> MatMul as one attention kernel (default off: differs from the three operators by
        up to 2e-4 relative)."""
        check(self.L.ahip_session_builder_with_fused_attention(self.handle, int(bool(enable))))
        return self

    def with_strided_views(self, enable=True):
        """Split / Transpose results that only MatMuls read become views instead of copies (default on)."""
        check(self.L.ahip_session_builder_with_strided_views(self.handle, int(bool(enable))))
        return self

    def with_device(self, device):
        check(self.L.ahip_session_builder_with_device(self.handle, device))
        return self

    def build(self):
        s = ctypes.c_void_p()
        check(self.L.ahip_session_builder_build(self.handle, ctypes.byref(s)))
        return HipSession(s)
