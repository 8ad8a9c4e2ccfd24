"""The reference's Python entry points over this backend: `load`, `session` and `InferenceSession`
(crates/altius_py/src/lib.rs:31-88, crates/altius_py/altius_py/__init__.py:4-30), so a script written for
`altius_py` runs on the GPU by importing this module instead."""
import numpy as np

from .graph import Model
from .session import HipSessionBuilder


def load(path):
    """altius_py.load: an ONNX file -> Model (lib.rs:31-42)."""
    return Model.load_onnx(path)


class _NamedSession:
    """What altius_py.session returns: run({input name: array}) -> [outputs] (lib.rs:95-180)."""

    def __init__(self, sess):
        self._sess = sess
        self._model = sess.model()

    def run(self, inputs):
        by_id = {}
        for name, value in inputs.items():
            vid = self._model.lookup_named_value(name)
            if vid is None:
                raise RuntimeError(f"Input '{name}' not found")
            a = np.asarray(value)
            if a.dtype not in (np.float32, np.int64, np.int32, np.bool_):
                raise RuntimeError(f"Input {name} unsupported type")
            by_id[vid] = np.ascontiguousarray(a) if a.ndim else a
        try:
            ordered = [by_id[v] for v in self._model.inputs]
        except KeyError as e:
            raise RuntimeError(f"Inference failed: graph input {e.args[0]} was not given") from None
        return self._sess.run(ordered)

    def profile(self):
        return self._sess.profile()


def session(model, enable_profiling=False, intra_op_num_threads=1, backend="hip", device=0, gemm_algorithm=1,
            fused_attention=False):
    """altius_py.session (lib.rs:44-88): the same rewrite pipeline -- fuse_layer_norm, fuse_gelu, fuse_fast_gelu,
    element-wise fusion for the backend that has a kernel for it (the reference: "cpu"; here: "hip", with the wider
    rule, after the scale and mask in front of each Softmax and the bias row behind each MatMul have been folded into them), eliminate_identity -- then the session builder.  The model object is left untouched, as in the
    reference (it takes a clone).  gemm_algorithm (default device.GEMM_FP32) and fused_attention (default off) are the
    two switches that trade the reference's exact semantics for speed; a caller opts in."""
    if backend != "hip":
        raise RuntimeError(f"Unknown backend: {backend}")
    m = model.clone()
    m.fuse_layer_norm()
    m.fuse_gelu()
    m.fuse_fast_gelu()
    m.fuse_softmax_prologue()
    m.fuse_matmul_bias()
    m.fuse_transpose_matmul()
    m.fuse_elemwise_ops(extended=True)
    m.eliminate_identity()
    builder = HipSessionBuilder(m).with_profiling_enabled(enable_profiling).with_intra_op_num_threads(intra_op_num_threads)
    return _NamedSession(builder.with_device(device).with_gemm_algorithm(gemm_algorithm).with_fused_attention(fused_attention).build())


class InferenceSession:
    """altius_py.InferenceSession (__init__.py:4-30): InferenceSession(path).run(None, {name: array})."""

    def __init__(self, model_path, enable_profile=False, intra_op_num_threads=1, backend="hip"):
        self.model_path = model_path
        self.model = load(model_path)
        self.session = session(self.model, enable_profile, intra_op_num_threads, backend)

    def run(self, output, input):
        assert output is None
        return self.session.run(input)
