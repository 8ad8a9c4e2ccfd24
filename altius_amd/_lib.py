"""Loads libaltius_hip.so and declares the C ABI (include/altius_hip.h) for ctypes.

There is no fallback: if the library is missing the import of any compute path
raises, so a GPU run can never silently use something else.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libaltius_hip.so")

OK, ERR_HIP, ERR_ARG, ERR_SHAPE, ERR_UNSUPPORTED, ERR_OOM, ERR_IO = 0, 1, 2, 3, 4, 5, 6
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
    ERR_IO: "Io",
}


class FusedStep(ctypes.Structure):
    """ahip_fused_step"""
    _fields_ = [("is_unary", c_int), ("op", c_int), ("lhs", c_int), ("rhs", c_int), ("alpha", c_float), ("beta", c_float),
                ("pow_scalar_exponent", c_int)]


FUSED_ACC = -1
FUSED_MAX_INPUTS = 6
FUSED_MAX_STEPS = 16


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
    f("ahip_copy_strided", [c_void_p, c_void_p, c_void_p, c_int, c_int, P(c_int64), P(c_int64), P(c_int64)])
    f("ahip_transpose", [c_void_p, c_void_p, c_void_p, c_int, c_int, P(c_int64), P(c_int64)])
    f("ahip_gather", [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_size_t, c_size_t, c_size_t, c_size_t])
    f("ahip_where", [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, P(c_int64), P(c_int64), P(c_int64),
                     P(c_int64)])
    f("ahip_greater", [c_void_p, c_void_p, c_void_p, c_void_p, c_int, P(c_int64), P(c_int64), P(c_int64)])
    f("ahip_cast", [c_void_p, c_void_p, c_void_p, c_int, c_int, c_size_t])
    f("ahip_batchnorm", [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t,
                         c_float])
    f("ahip_gemm", [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p] + [c_size_t] * 4 + [c_int, c_int] + [c_size_t] * 8
      + [c_float, c_float])
    f("ahip_gemm_batch2", [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p] + [c_size_t] * 5 + [c_int, c_int] + [c_size_t] * 3
      + [P(c_size_t)] * 3 + [c_size_t, c_size_t, c_float, c_float])
    f("ahip_gemm_activated", [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p] + [c_size_t] * 3 + [c_int, c_int]
      + [c_size_t] * 5 + [c_float, c_float])
    f("ahip_gemm_post", [c_void_p] * 5 + [c_size_t] * 3 + [c_int, c_int] + [c_size_t] * 5 + [c_float, c_float, c_int, c_void_p])
    f("ahip_attention", [c_void_p] * 5 + [c_size_t] * 9 + [P(c_size_t)] * 4 + [c_int, c_float, c_void_p, c_size_t])
    f("ahip_gemm_set_algorithm", [c_void_p, c_int])
    f("ahip_set_streaming_threshold", [c_void_p, c_size_t])
    f("ahip_set_load_streaming_threshold", [c_void_p, c_size_t])
    f("ahip_gemm_in_kernel_k_cut", [c_void_p, P(c_int), P(c_int)])
    f("ahip_gemm_set_in_kernel_k_cut", [c_void_p, c_int])
    f("ahip_xcd_round_robin_holds", [c_int, P(ctypes.c_uint32), c_size_t])
    f("ahip_gemm_register_constant", [c_void_p, c_void_p, c_size_t])
    f("ahip_gemm_unregister_constant", [c_void_p, c_void_p])
    f("ahip_conv2d", [c_void_p] * 6 + [c_size_t] * 16)
    f("ahip_maxpool", [c_void_p] * 3 + [c_size_t] * 11)
    f("ahip_resize", [c_void_p] * 3 + [c_size_t] * 5 + [c_int])
    f("ahip_module_load", [c_void_p, c_void_p, c_size_t, P(c_void_p)])
    f("ahip_module_unload", [c_void_p, c_void_p])
    f("ahip_launch", [c_void_p, c_void_p, c_char_p, P(ctypes.c_uint32), P(ctypes.c_uint32), ctypes.c_uint32,
                      P(c_void_p)])
    f("ahip_broadcast_shape", [c_int, P(c_int64), c_int, P(c_int64), P(c_int), P(c_int64)])
    f("ahip_strides_for_broadcasting", [c_int, P(c_int64), c_int, P(c_int64), P(c_int64)])
    f("ahip_binary", [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, P(c_int64), P(c_int64), P(c_int64)])
    f("ahip_unary", [c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_float, c_float])
    f("ahip_fused_use_compiled_chains", [c_void_p, c_int])
    f("ahip_fused_elemwise", [c_void_p, c_void_p, c_int, P(c_int64), c_int, P(c_void_p), P(P(c_int64)), c_int, P(FusedStep)])
    f("ahip_softmax_lastaxis", [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t])
    f("ahip_softmax_lastaxis_prologue", [c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_int, c_float, c_void_p, c_size_t])
    f("ahip_layernorm_lastaxis", [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_size_t, c_float])
    f("ahip_reduce", [c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t])
    f("ahip_reduce_static", [c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_size_t, c_size_t])
    f("ahip_reduce_static_capacity", [], c_size_t)


class OpAttrs(ctypes.Structure):
    """ahip_op_attrs"""

    _fields_ = [
        ("axis", c_int64),
        ("axes", c_int64 * MAX_RANK),
        ("n_axes", ctypes.c_int32),
        ("keep_dims", ctypes.c_int32),
        ("alpha", c_float),
        ("beta", c_float),
        ("epsilon", c_float),
        ("stash_type", c_int64),
    ]


def _declare_graph(L):
    def f(name, argtypes, restype=c_int):
        fn = getattr(L, name)
        fn.argtypes = argtypes
        fn.restype = restype

    c_double = ctypes.c_double
    f("ahip_op_attrs_default", [P(OpAttrs)], None)
    f("ahip_op_name", [c_int], c_char_p)
    f("ahip_model_new", [c_int64, P(c_void_p)])
    f("ahip_model_clone", [c_void_p, P(c_void_p)])
    f("ahip_model_free", [c_void_p], None)
    f("ahip_model_new_value", [c_void_p, c_char_p, P(c_int64)])
    f("ahip_model_new_value_shaped", [c_void_p, c_char_p, c_int, c_int, P(c_int64), P(c_int64)])
    f("ahip_model_add_initializer", [c_void_p, c_int64, c_int, c_int, P(c_int64), c_void_p, c_size_t])
    f("ahip_model_add_node", [c_void_p, c_int, P(OpAttrs), c_char_p, c_int, P(c_int64), c_int, P(c_int64), P(c_int64)])
    f("ahip_model_add_input", [c_void_p, c_int64])
    f("ahip_model_add_output", [c_void_p, c_int64])
    f("ahip_model_lookup_named_value", [c_void_p, c_char_p, P(c_int64)])
    f("ahip_model_graph_io", [c_void_p, c_int, P(c_int64), c_int, P(c_int)])
    f("ahip_model_topo_sort", [c_void_p, P(c_int64), c_int, P(c_int)])
    f("ahip_model_node_info", [c_void_p, c_int64, P(c_int), P(OpAttrs), P(c_int), P(c_int64), P(c_int), P(c_int64), c_int])
    f("ahip_model_load_onnx", [c_char_p, P(c_void_p)])
    f("ahip_model_load_onnx_buffer", [c_void_p, c_size_t, P(c_void_p)])
    f("ahip_model_opset_version", [c_void_p], c_int64)
    f("ahip_model_num_values", [c_void_p], c_int64)
    f("ahip_model_num_nodes", [c_void_p], c_int64)
    f("ahip_model_value_info", [c_void_p, c_int64, P(c_char_p), P(c_int), P(c_int), P(c_int64), c_int])
    f("ahip_model_initializer", [c_void_p, c_int64, P(c_void_p)])
    f("ahip_model_node_name", [c_void_p, c_int64], c_char_p)
    f("ahip_node_set_attr_int", [c_void_p, c_int64, c_char_p, c_int64])
    f("ahip_node_set_attr_float", [c_void_p, c_int64, c_char_p, c_float])
    f("ahip_node_set_attr_ints", [c_void_p, c_int64, c_char_p, P(c_int64), c_int])
    f("ahip_node_set_attr_string", [c_void_p, c_int64, c_char_p, c_char_p])
    f("ahip_node_set_attr_tensor", [c_void_p, c_int64, c_char_p, c_void_p])
    f("ahip_node_get_attr_int", [c_void_p, c_int64, c_char_p, P(c_int64)])
    f("ahip_node_get_attr_float", [c_void_p, c_int64, c_char_p, P(c_float)])
    f("ahip_node_get_attr_ints", [c_void_p, c_int64, c_char_p, P(c_int64), c_int, P(c_int)])
    f("ahip_node_get_attr_string", [c_void_p, c_int64, c_char_p, c_char_p, c_int, P(c_int)])
    f("ahip_node_get_attr_tensor", [c_void_p, c_int64, c_char_p, P(c_void_p)])
    f("ahip_model_infer_value_shape", [c_void_p, c_int64, P(c_int), P(c_int), P(c_int64)])
    f("ahip_model_execution_plan", [c_void_p, P(c_int64), P(c_int), c_int, P(c_int64), c_int, P(c_int), P(c_int)])
    for name in ("ahip_fuse_layer_norm", "ahip_fuse_gelu", "ahip_fuse_fast_gelu", "ahip_eliminate_identity", "ahip_fuse_softmax_prologue",
                 "ahip_fuse_matmul_bias", "ahip_fuse_transpose_matmul"):
        f(name, [c_void_p, P(c_int)])
    f("ahip_fuse_elemwise_ops", [c_void_p, c_int, P(c_int)])
    f("ahip_tensor_new", [c_int, c_int, P(c_int64), c_void_p, c_size_t, P(c_void_p)])
    f("ahip_tensor_free", [c_void_p], None)
    f("ahip_tensor_elem_type", [c_void_p])
    f("ahip_tensor_rank", [c_void_p])
    f("ahip_tensor_dims", [c_void_p, P(c_int64), c_int])
    f("ahip_tensor_nbytes", [c_void_p], c_size_t)
    f("ahip_tensor_data", [c_void_p], c_void_p)
    f("ahip_tensor_data_mut", [c_void_p], c_void_p)
    f("ahip_host_pool_stats", [P(c_size_t), P(c_size_t), P(c_size_t), P(c_size_t)])
    f("ahip_host_pool_trim", [], c_size_t)
    f("ahip_session_builder_new", [c_void_p, P(c_void_p)])
    f("ahip_session_builder_free", [c_void_p], None)
    f("ahip_session_builder_with_intra_op_num_threads", [c_void_p, c_size_t])
    f("ahip_session_builder_with_profiling_enabled", [c_void_p, c_int])
    f("ahip_session_builder_with_device", [c_void_p, c_int])
    f("ahip_session_builder_with_graph_replay", [c_void_p, c_int])
    f("ahip_session_builder_with_device_timing", [c_void_p, c_int])
    f("ahip_session_builder_with_gemm_algorithm", [c_void_p, c_int])
    f("ahip_session_builder_with_fused_attention", [c_void_p, c_int])
    f("ahip_session_builder_with_strided_views", [c_void_p, c_int])
    f("ahip_session_copies_avoided", [c_void_p, P(c_size_t)])
    f("ahip_session_lanes", [c_void_p, P(c_size_t)])
    f("ahip_session_graph_replays", [c_void_p, P(c_size_t)])
    f("ahip_session_builder_build", [c_void_p, P(c_void_p)])
    f("ahip_session_free", [c_void_p], None)
    f("ahip_session_run", [c_void_p, c_int, P(c_void_p), c_int, P(c_void_p), P(c_int)])
    f("ahip_session_run_device", [c_void_p, c_int, P(c_void_p), P(c_int), P(c_int), P(P(c_int64)), c_int, P(c_void_p), P(c_int)])
    f("ahip_session_synchronize", [c_void_p])
    f("ahip_device_tensor_free", [c_void_p], None)
    f("ahip_device_tensor_ptr", [c_void_p], c_void_p)
    f("ahip_device_tensor_elem_type", [c_void_p])
    f("ahip_device_tensor_rank", [c_void_p])
    f("ahip_device_tensor_dims", [c_void_p, P(c_int64), c_int])
    f("ahip_device_tensor_nbytes", [c_void_p], c_size_t)
    f("ahip_session_model", [c_void_p], c_void_p)
    f("ahip_session_profile", [c_void_p, c_int, P(c_char_p), P(c_double), P(c_int)])
    f("ahip_session_last_run_ms", [c_void_p, P(c_double)])
    f("ahip_session_last_device_ms", [c_void_p, P(c_double)])
    f("ahip_session_device_allocations", [c_void_p, P(c_size_t)])


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
        _declare_graph(L)
        _lib = L
    return _lib


def i64_array(values):
    values = [int(v) for v in values]
    return (c_int64 * max(len(values), 1))(*values)


def check(rc, ctx=None):
    if rc != OK:
        msg = lib().ahip_last_error(ctx)
        raise AltiusHipError(rc, msg.decode("utf-8", "replace") if msg else "")
