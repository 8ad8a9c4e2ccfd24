"""Graph IR handles over the C ABI: Model, Op, Tensor and the fusion passes.

The structure is altius_core's (Model -> Graph -> nodes / values / initializers /
inputs / outputs), so a test written against the reference reads the same here:

    model = Model()
    x = model.new_val_named("x"); y = model.new_val_named("y"); z = model.new_val_named("z")
    model.add_node(Op.Add, [x, y], [z])
    model.inputs.append(x) ... (add_input / add_output)
"""
import ctypes

import numpy as np

from . import _lib
from ._lib import OpAttrs, check, i64_array

BOOL, F32, I32, I64 = 0, 1, 2, 3
_NP_OF = {BOOL: np.bool_, F32: np.float32, I32: np.int32, I64: np.int64}
_ELEM_OF = {np.dtype(np.bool_): BOOL, np.dtype(np.float32): F32, np.dtype(np.int32): I32, np.dtype(np.int64): I64}


class Op:
    """Operator kinds, in the order of altius_core::op::Op."""

    _NAMES = [
        "Identity", "Conv2d", "Add", "Sub", "Mul", "Div", "Pow", "Greater", "Sqrt", "ReLU", "Gelu", "LeakyReLU",
        "Sigmoid", "Erf", "Tanh", "Clip", "Where", "Softmax", "Cast", "MaxPool", "GlobalAveragePool", "Reshape",
        "Flatten", "Resize", "Concat", "Transpose", "Squeeze", "Unsqueeze", "ReduceMin", "ReduceMax",
        "ReduceMean", "Round", "Exp", "Expand", "Range", "Loop", "Tile", "Split", "Slice", "Gather", "Shape",
        "NonMaxSuppression", "MatMul", "Gemm", "BatchNormalization", "LayerNormalization", "HardSigmoid",
        "Constant", "FusedElemwise",
    ]


for _i, _n in enumerate(Op._NAMES):
    setattr(Op, _n, _i)


def op_name(kind):
    return _lib.lib().ahip_op_name(kind).decode()


def make_attrs(axis=None, axes=None, keep_dims=None, alpha=None, beta=None, epsilon=None, stash_type=None):
    a = OpAttrs()
    _lib.lib().ahip_op_attrs_default(ctypes.byref(a))
    if axis is not None:
        a.axis = axis
    if axes is not None:
        a.n_axes = len(axes)
        for i, v in enumerate(axes):
            a.axes[i] = v
    if keep_dims is not None:
        a.keep_dims = int(bool(keep_dims))
    if alpha is not None:
        a.alpha = alpha
    if beta is not None:
        a.beta = beta
    if epsilon is not None:
        a.epsilon = epsilon
    if stash_type is not None:
        a.stash_type = stash_type
    return a


class Tensor:
    """A host tensor owned by the library (altius_core::tensor::Tensor)."""

    def __init__(self, handle):
        self.handle = handle

    @classmethod
    def from_numpy(cls, array):
        a = np.asarray(array, order="C")
        if a.dtype not in _ELEM_OF:
            raise TypeError(f"unsupported dtype {a.dtype}")
        h = ctypes.c_void_p()
        check(_lib.lib().ahip_tensor_new(_ELEM_OF[a.dtype], a.ndim, i64_array(a.shape), a.ctypes.data, a.nbytes,
                                         ctypes.byref(h)))
        return cls(h)

    @property
    def dims(self):
        L = _lib.lib()
        r = L.ahip_tensor_rank(self.handle)
        d = (ctypes.c_int64 * max(r, 1))()
        check(L.ahip_tensor_dims(self.handle, d, r))
        return [int(d[i]) for i in range(r)]

    @property
    def elem_ty(self):
        return _lib.lib().ahip_tensor_elem_type(self.handle)

    def numpy(self):
        L = _lib.lib()
        n = L.ahip_tensor_nbytes(self.handle)
        out = np.empty(self.dims, dtype=_NP_OF[self.elem_ty])
        assert out.nbytes == n
        if n:
            ctypes.memmove(out.ctypes.data, L.ahip_tensor_data(self.handle), n)
        return out

    def view(self):
        """The tensor's own bytes as a numpy array, without a copy.  The array keeps this Tensor
        alive; writing through it fills the tensor in place (Tensor::data_mut)."""
        L = _lib.lib()
        n = L.ahip_tensor_nbytes(self.handle)
        dtype = _NP_OF[self.elem_ty]
        if n == 0:
            return np.empty(self.dims, dtype=dtype)
        raw = (ctypes.c_ubyte * n).from_address(L.ahip_tensor_data_mut(self.handle))
        raw._tensor = self  # the buffer object owns a reference to the tensor
        return np.frombuffer(raw, dtype=dtype).reshape(self.dims)

    @classmethod
    def zeros(cls, dims, elem_ty=1):
        """A zero-filled tensor of the given shape (fill it through view())."""
        h = ctypes.c_void_p()
        check(_lib.lib().ahip_tensor_new(elem_ty, len(dims), i64_array(dims), None, 0, ctypes.byref(h)))
        return cls(h)

    def __del__(self):
        if getattr(self, "handle", None):
            _lib.lib().ahip_tensor_free(self.handle)
            self.handle = None


def host_pool_stats():
    """(live_bytes, cached_bytes, pinned_allocations, reuses) of the pinned pool behind host tensors."""
    v = [ctypes.c_size_t() for _ in range(4)]
    check(_lib.lib().ahip_host_pool_stats(*[ctypes.byref(x) for x in v]))
    return tuple(x.value for x in v)


def host_pool_trim():
    return _lib.lib().ahip_host_pool_trim()


class Model:
    """altius_core::model::Model."""

    def __init__(self, opset_version=13, _handle=None, _borrowed=False):
        self.L = _lib.lib()
        self._borrowed = _borrowed
        if _handle is None:
            h = ctypes.c_void_p()
            check(self.L.ahip_model_new(opset_version, ctypes.byref(h)))
            _handle = h
        self.handle = _handle

    def __del__(self):
        if getattr(self, "handle", None) and not self._borrowed:
            self.L.ahip_model_free(self.handle)
        self.handle = None

    def clone(self):
        h = ctypes.c_void_p()
        check(self.L.ahip_model_clone(self.handle, ctypes.byref(h)))
        return Model(_handle=h)

    # --- values -----------------------------------------------------------------
    def new_val(self):
        v = ctypes.c_int64()
        check(self.L.ahip_model_new_value(self.handle, None, ctypes.byref(v)))
        return v.value

    def new_val_named(self, name):
        v = ctypes.c_int64()
        check(self.L.ahip_model_new_value(self.handle, name.encode(), ctypes.byref(v)))
        return v.value

    def new_val_named_and_shaped(self, name, dims, elem_ty=F32):
        """A negative (or None) dimension is dynamic."""
        d = [-1 if x is None else int(x) for x in dims]
        v = ctypes.c_int64()
        check(self.L.ahip_model_new_value_shaped(self.handle, name.encode(), elem_ty, len(d), i64_array(d),
                                                 ctypes.byref(v)))
        return v.value

    def add_initializer(self, value_id, array):
        a = np.asarray(array, order="C")
        check(self.L.ahip_model_add_initializer(self.handle, value_id, _ELEM_OF[a.dtype], a.ndim, i64_array(a.shape),
                                                a.ctypes.data, a.nbytes))

    def new_initializer(self, array, name=None):
        v = self.new_val_named(name) if name else self.new_val()
        self.add_initializer(v, array)
        return v

    def lookup_named_value(self, name):
        v = ctypes.c_int64()
        rc = self.L.ahip_model_lookup_named_value(self.handle, name.encode(), ctypes.byref(v))
        return v.value if rc == 0 else None

    # --- nodes --------------------------------------------------------------------
    _ATTR_ALIASES = {"keep_dims": "keepdims", "trans_a": "transA", "trans_b": "transB", "padding": "pads"}

    def add_node(self, op_kind, inputs, outputs, name=None, **attrs):
        """Attributes go by their ONNX names (axis, axes, keepdims, perm, kernel_shape, transB, to, ...;
        keep_dims / trans_a / trans_b / padding are accepted spellings of the reference's field names).
        Absent ones keep the defaults the ONNX loader applies."""
        nid = ctypes.c_int64()
        check(self.L.ahip_model_add_node(self.handle, op_kind, None, name.encode() if name else None,
                                         len(inputs), i64_array(inputs), len(outputs), i64_array(outputs),
                                         ctypes.byref(nid)))
        for key, value in attrs.items():
            self.set_attr(nid.value, self._ATTR_ALIASES.get(key, key), value)
        return nid.value

    def set_attr(self, node_id, name, value):
        n = name.encode()
        if isinstance(value, Tensor):
            check(self.L.ahip_node_set_attr_tensor(self.handle, node_id, n, value.handle))
        elif isinstance(value, np.ndarray):
            t = Tensor.from_numpy(value)
            check(self.L.ahip_node_set_attr_tensor(self.handle, node_id, n, t.handle))
        elif isinstance(value, str):
            check(self.L.ahip_node_set_attr_string(self.handle, node_id, n, value.encode()))
        elif isinstance(value, (list, tuple)):
            check(self.L.ahip_node_set_attr_ints(self.handle, node_id, n, i64_array(value), len(value)))
        elif isinstance(value, (bool, int, np.integer)):
            check(self.L.ahip_node_set_attr_int(self.handle, node_id, n, int(value)))
        elif isinstance(value, (float, np.floating)):
            check(self.L.ahip_node_set_attr_float(self.handle, node_id, n, float(value)))
        else:
            raise TypeError(f"attribute {name}: unsupported value {value!r}")

    def get_attr(self, node_id, name, kind):
        """kind: 'int', 'float', 'ints', 'string' or 'tensor'."""
        n = name.encode()
        if kind == "int":
            v = ctypes.c_int64()
            check(self.L.ahip_node_get_attr_int(self.handle, node_id, n, ctypes.byref(v)))
            return v.value
        if kind == "float":
            v = ctypes.c_float()
            check(self.L.ahip_node_get_attr_float(self.handle, node_id, n, ctypes.byref(v)))
            return v.value
        if kind == "ints":
            c = ctypes.c_int()
            check(self.L.ahip_node_get_attr_ints(self.handle, node_id, n, None, 0, ctypes.byref(c)))
            buf = (ctypes.c_int64 * max(c.value, 1))()
            check(self.L.ahip_node_get_attr_ints(self.handle, node_id, n, buf, c.value, ctypes.byref(c)))
            return [int(buf[i]) for i in range(c.value)]
        if kind == "string":
            c = ctypes.c_int()
            check(self.L.ahip_node_get_attr_string(self.handle, node_id, n, None, 0, ctypes.byref(c)))
            buf = ctypes.create_string_buffer(c.value + 1)
            check(self.L.ahip_node_get_attr_string(self.handle, node_id, n, buf, c.value + 1, ctypes.byref(c)))
            return buf.value.decode()
        if kind == "tensor":
            h = ctypes.c_void_p()
            check(self.L.ahip_node_get_attr_tensor(self.handle, node_id, n, ctypes.byref(h)))
            return Tensor(h).numpy()
        raise ValueError(kind)

    # --- ONNX files (altius_core::onnx::load_onnx) ----------------------------------------------
    @classmethod
    def load_onnx(cls, path):
        h = ctypes.c_void_p()
        check(_lib.lib().ahip_model_load_onnx(str(path).encode(), ctypes.byref(h)))
        return cls(_handle=h)

    @classmethod
    def load_onnx_from_buffer(cls, data):
        data = bytes(data)
        buf = ctypes.create_string_buffer(data, max(1, len(data)))
        h = ctypes.c_void_p()
        check(_lib.lib().ahip_model_load_onnx_buffer(ctypes.cast(buf, ctypes.c_void_p), len(data), ctypes.byref(h)))
        return cls(_handle=h)

    @property
    def opset_version(self):
        return self.L.ahip_model_opset_version(self.handle)

    def num_values(self):
        return self.L.ahip_model_num_values(self.handle)

    def value_info(self, value_id):
        """(name or None, elem type or None, dims or None); dynamic dimensions read -1."""
        name, ty, rank = ctypes.c_char_p(), ctypes.c_int(), ctypes.c_int()
        dims = (ctypes.c_int64 * 16)()
        check(self.L.ahip_model_value_info(self.handle, value_id, ctypes.byref(name), ctypes.byref(ty),
                                           ctypes.byref(rank), dims, 16))
        nm = name.value.decode() if name.value is not None else None
        if rank.value < 0:
            return nm, None, None
        return nm, ty.value, [int(dims[i]) for i in range(rank.value)]

    def initializer(self, value_id):
        h = ctypes.c_void_p()
        check(self.L.ahip_model_initializer(self.handle, value_id, ctypes.byref(h)))
        return Tensor(h).numpy()

    def node_name(self, node_id):
        n = self.L.ahip_model_node_name(self.handle, node_id)
        return n.decode() if n is not None else None

    def add_input(self, value_id):
        check(self.L.ahip_model_add_input(self.handle, value_id))

    def add_output(self, value_id):
        check(self.L.ahip_model_add_output(self.handle, value_id))

    def _io(self, which):
        n = ctypes.c_int()
        check(self.L.ahip_model_graph_io(self.handle, which, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_int64 * max(n.value, 1))()
        check(self.L.ahip_model_graph_io(self.handle, which, buf, n.value, ctypes.byref(n)))
        return [int(buf[i]) for i in range(n.value)]

    @property
    def inputs(self):
        return self._io(0)

    @property
    def outputs(self):
        return self._io(1)

    def topo_sort_nodes(self):
        n = ctypes.c_int()
        check(self.L.ahip_model_topo_sort(self.handle, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_int64 * max(n.value, 1))()
        check(self.L.ahip_model_topo_sort(self.handle, buf, n.value, ctypes.byref(n)))
        return [int(buf[i]) for i in range(n.value)]

    def node(self, node_id, io_capacity=16):
        kind, nin, nout = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        a = OpAttrs()
        ins = (ctypes.c_int64 * io_capacity)()
        outs = (ctypes.c_int64 * io_capacity)()
        check(self.L.ahip_model_node_info(self.handle, node_id, ctypes.byref(kind), ctypes.byref(a),
                                          ctypes.byref(nin), ins, ctypes.byref(nout), outs, io_capacity))
        return {
            "id": node_id,
            "op": kind.value,
            "op_name": op_name(kind.value),
            "inputs": [int(ins[i]) for i in range(min(nin.value, io_capacity))],
            "outputs": [int(outs[i]) for i in range(min(nout.value, io_capacity))],
            "axis": a.axis,
            "axes": [int(a.axes[i]) for i in range(a.n_axes)],
            "keep_dims": bool(a.keep_dims),
            "alpha": a.alpha,
            "beta": a.beta,
            "epsilon": a.epsilon,
            "stash_type": a.stash_type,
        }

    def nodes(self):
        """Live nodes in topological order."""
        return [self.node(i) for i in self.topo_sort_nodes()]

    # --- analysis --------------------------------------------------------------------
    def infer_value_shape(self, value_id):
        ty, rank = ctypes.c_int(), ctypes.c_int()
        dims = (ctypes.c_int64 * _lib.MAX_RANK)()
        check(self.L.ahip_model_infer_value_shape(self.handle, value_id, ctypes.byref(ty), ctypes.byref(rank), dims))
        return [int(dims[i]) for i in range(rank.value)], ty.value

    def execution_plan(self):
        """[(node_id, [value ids freed after it]), ...] in execution order."""
        nn, nf = ctypes.c_int(), ctypes.c_int()
        check(self.L.ahip_model_execution_plan(self.handle, None, None, 0, None, 0, ctypes.byref(nn), ctypes.byref(nf)))
        ids = (ctypes.c_int64 * max(nn.value, 1))()
        offs = (ctypes.c_int * (nn.value + 1))()
        vals = (ctypes.c_int64 * max(nf.value, 1))()
        check(self.L.ahip_model_execution_plan(self.handle, ids, offs, nn.value, vals, nf.value, ctypes.byref(nn),
                                               ctypes.byref(nf)))
        return [(int(ids[i]), [int(vals[j]) for j in range(offs[i], offs[i + 1])]) for i in range(nn.value)]

    # --- optimize::* -------------------------------------------------------------------
    def _pass(self, fn):
        c = ctypes.c_int()
        check(fn(self.handle, ctypes.byref(c)))
        return c.value

    def fuse_layer_norm(self):
        return self._pass(self.L.ahip_fuse_layer_norm)

    def fuse_gelu(self):
        return self._pass(self.L.ahip_fuse_gelu)

    def fuse_fast_gelu(self):
        return self._pass(self.L.ahip_fuse_fast_gelu)

    def eliminate_identity(self):
        return self._pass(self.L.ahip_eliminate_identity)

    def fuse_transpose_matmul(self):
        """A Transpose of the last two axes feeding a MatMul operand becomes a flag of the product."""
        return self._pass(self.L.ahip_fuse_transpose_matmul)

    def fuse_matmul_bias(self):
        """MatMul -> Add(bias row) becomes a MatMul node with the bias as third input."""
        return self._pass(self.L.ahip_fuse_matmul_bias)

    def fuse_softmax_prologue(self):
        """[Mul | Div by a constant] -> [Add mask] -> Softmax becomes one Softmax node with inputs (x, scale?, mask?)."""
        return self._pass(self.L.ahip_fuse_softmax_prologue)

    def fuse_elemwise_ops(self, extended=False):
        """Chains of element-wise operators -> FusedElemwise nodes; the reference's rule, or this backend's
        wider one with extended=True.  Returns the number of chains fused."""
        c = ctypes.c_int()
        check(self.L.ahip_fuse_elemwise_ops(self.handle, 1 if extended else 0, ctypes.byref(c)))
        return c.value

    def fused_chain(self, node_id):
        """Operator names of a FusedElemwise node, in order."""
        n = ctypes.c_int()
        check(self.L.ahip_node_get_attr_string(self.handle, node_id, b"chain", None, 0, ctypes.byref(n)))
        buf = ctypes.create_string_buffer(n.value + 1)
        check(self.L.ahip_node_get_attr_string(self.handle, node_id, b"chain", buf, n.value + 1, None))
        return buf.value.decode().split(",")
