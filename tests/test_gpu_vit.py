"""A whole (small) vision transformer as ONNX bytes: patch-embedding Conv, class token Concat,
position Add, two encoder blocks written the way exporters write them (9-node LayerNorm chains,
5-node erf-GELU chains, reshape / transpose head handling), final LayerNorm, class-token Gather
and Gemm head.  Loaded, fused, run on the GPU, and compared with the same computation carried out
step by step with the CPU oracle; then again without the fusion passes."""
import numpy as np
import pytest

import onnx_writer as W
import oracle as O
from altius_amd.graph import Model
from altius_amd.session import HipSessionBuilder

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(51)
B, IMG, P, H, NH, MLP, LAYERS, CLASSES = 2, 32, 8, 64, 4, 128, 2, 10
T = (IMG // P) ** 2 + 1
D = H // NH


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


class Builder:
    def __init__(self):
        self.nodes, self.inits, self.count = [], [], 0

    def init(self, array, name=None):
        name = name or f"c{len(self.inits)}"
        self.inits.append(W.tensor(name, np.asarray(array)))
        return name

    def node(self, op, inputs, n_out=1, **attrs):
        outs = [f"v{self.count + i}" for i in range(n_out)]
        self.count += n_out
        self.nodes.append(W.node(op, inputs, outs, **attrs))
        return outs[0] if n_out == 1 else outs

    def layer_norm(self, x, gamma, beta):
        mean = self.node("ReduceMean", [x], axes=[-1])
        d = self.node("Sub", [x, mean])
        sq = self.node("Pow", [d, self.init(np.array(2.0, np.float32))])
        var = self.node("ReduceMean", [sq], axes=[-1])
        sd = self.node("Sqrt", [self.node("Add", [var, self.init(np.array(1e-6, np.float32))])])
        return self.node("Add", [self.node("Mul", [self.node("Div", [d, sd]), self.init(gamma)]), self.init(beta)])

    def gelu(self, x):
        e = self.node("Erf", [self.node("Div", [x, self.init(np.array(1.4142135, np.float32))])])
        return self.node("Mul", [self.node("Mul", [x, self.node("Add", [e, self.init(np.array(1.0, np.float32))])]),
                                 self.init(np.array(0.5, np.float32))])

    def linear(self, x, w, b):
        return self.node("Add", [self.node("MatMul", [x, self.init(w)]), self.init(b)])


def make_vit():
    p = {"patch_w": rnd(H, 3, P, P, scale=0.05), "patch_b": rnd(H, scale=0.1), "cls": rnd(1, 1, H), "pos": rnd(1, T, H, scale=0.1),
         "lnf": (1 + rnd(H, scale=0.1), rnd(H, scale=0.1)), "head_w": rnd(CLASSES, H, scale=0.1), "head_b": rnd(CLASSES), "blocks": []}
    g = Builder()
    x = g.node("Conv", ["image", g.init(p["patch_w"]), g.init(p["patch_b"])], kernel_shape=[P, P], strides=[P, P])
    x = g.node("Reshape", [x, g.init(np.array([B, H, T - 1], np.int64))])
    x = g.node("Transpose", [x], perm=[0, 2, 1])
    x = g.node("Concat", [g.init(np.broadcast_to(p["cls"], (B, 1, H)).copy()), x], axis=1)
    x = g.node("Add", [x, g.init(p["pos"])])
    for _ in range(LAYERS):
        blk = {"ln1": (1 + rnd(H, scale=0.1), rnd(H, scale=0.1)), "wqkv": rnd(H, 3 * H, scale=0.1), "bqkv": rnd(3 * H, scale=0.1),
               "wo": rnd(H, H, scale=0.1), "bo": rnd(H, scale=0.1), "ln2": (1 + rnd(H, scale=0.1), rnd(H, scale=0.1)),
               "w1": rnd(H, MLP, scale=0.1), "b1": rnd(MLP, scale=0.1), "w2": rnd(MLP, H, scale=0.1), "b2": rnd(H, scale=0.1)}
        p["blocks"].append(blk)
        y = g.layer_norm(x, *blk["ln1"])
        qkv = g.linear(y, blk["wqkv"], blk["bqkv"])
        q, k, v = g.node("Split", [qkv, g.init(np.array([H, H, H], np.int64))], n_out=3, axis=2)
        heads = [g.node("Transpose", [g.node("Reshape", [t, g.init(np.array([B, T, NH, D], np.int64))])], perm=[0, 2, 1, 3]) for t in (q, k, v)]
        s = g.node("MatMul", [heads[0], g.node("Transpose", [heads[1]], perm=[0, 1, 3, 2])])
        s = g.node("Softmax", [g.node("Mul", [s, g.init(np.array(D ** -0.5, np.float32))])], axis=-1)
        a = g.node("Transpose", [g.node("MatMul", [s, heads[2]])], perm=[0, 2, 1, 3])
        a = g.node("Reshape", [a, g.init(np.array([B, T, H], np.int64))])
        x = g.node("Add", [x, g.linear(a, blk["wo"], blk["bo"])])
        y = g.layer_norm(x, *blk["ln2"])
        x = g.node("Add", [x, g.linear(g.gelu(g.linear(y, blk["w1"], blk["b1"])), blk["w2"], blk["b2"])])
    x = g.layer_norm(x, *p["lnf"])
    cls = g.node("Gather", [x, g.init(np.array(0, np.int64))], axis=1)
    logits = g.node("Gemm", [cls, g.init(p["head_w"]), g.init(p["head_b"])], transB=1)
    g.nodes.append(W.node("Identity", [logits], ["logits"]))
    data = W.model(W.graph(g.nodes, g.inits, [W.value_info("image", W.FLOAT, [B, 3, IMG, IMG])],
                           [W.value_info("logits", W.FLOAT, [B, CLASSES])]), opsets=(("", 13),))
    return data, p


def oracle_vit(image, p, fused):
    """The same network with the oracle's kernels: LayerNormalization / Gelu when `fused`, the node chains otherwise."""
    s = lambda v: np.array(v, np.float32)

    def ln(x, gamma, beta):
        if fused:
            return O.layer_norm(x, gamma, beta, 1e-6)
        mean = O.reduce(O.REDUCE_MEAN, x, [-1], True)
        d = O.binary(O.SUB, x, mean)
        var = O.reduce(O.REDUCE_MEAN, O.binary(O.POW, d, s(2.0)), [-1], True)
        n = O.binary(O.DIV, d, O.unary(O.SQRT, O.binary(O.ADD, var, s(1e-6))))
        return O.binary(O.ADD, O.binary(O.MUL, n, gamma), beta)

    def gelu(x):
        if fused:
            return O.unary(O.GELU, x)
        e = O.unary(O.ERF, O.binary(O.DIV, x, s(1.4142135)))
        return O.binary(O.MUL, O.binary(O.MUL, x, O.binary(O.ADD, e, s(1.0))), s(0.5))

    lin = lambda x, w, b: O.binary(O.ADD, O.matmul(x, w), b)
    x = O.conv2d(image, p["patch_w"], p["patch_b"], strides=(P, P)).reshape(B, H, T - 1)
    x = np.concatenate([np.broadcast_to(p["cls"], (B, 1, H)), O.transpose(x, (0, 2, 1))], axis=1)
    x = O.binary(O.ADD, x, p["pos"])
    for blk in p["blocks"]:
        qkv = lin(ln(x, *blk["ln1"]), blk["wqkv"], blk["bqkv"])
        q, k, v = (O.transpose(t.reshape(B, T, NH, D), (0, 2, 1, 3)) for t in O.split(qkv, [H, H, H], 2, strict=True))
        sc = O.softmax(O.binary(O.MUL, O.matmul(q, O.transpose(k, (0, 1, 3, 2))), s(D ** -0.5)))
        a = O.transpose(O.matmul(sc, v), (0, 2, 1, 3)).reshape(B, T, H)
        x = O.binary(O.ADD, x, lin(a, blk["wo"], blk["bo"]))
        x = O.binary(O.ADD, x, lin(gelu(lin(ln(x, *blk["ln2"]), blk["w1"], blk["b1"])), blk["w2"], blk["b2"]))
    x = ln(x, *p["lnf"])
    return O.gemm(np.ascontiguousarray(x[:, 0]), p["head_w"], p["head_b"], trans_b=True)


def test_vit_from_onnx_bytes(case):
    case("ViT from ONNX bytes")
    data, params = make_vit()
    image = rnd(B, 3, IMG, IMG)
    model = Model.load_onnx_from_buffer(data)
    n_nodes = len(model.nodes())
    unfused = model.clone()
    assert model.fuse_layer_norm() == 2 * LAYERS + 1 and model.fuse_gelu() == LAYERS and model.eliminate_identity() >= 0
    assert len(model.nodes()) < n_nodes - 8 * (2 * LAYERS + 1)
    ops = [n["op_name"] for n in model.nodes()]
    assert ops.count("LayerNormalization") == 2 * LAYERS + 1 and ops.count("Gelu") == LAYERS and "Erf" not in ops

    sess = HipSessionBuilder(model).with_profiling_enabled(True).build()
    (logits,) = sess.run([image])
    assert logits.shape == (B, CLASSES)
    np.testing.assert_allclose(logits, oracle_vit(image, params, fused=True), rtol=2e-4, atol=2e-4)
    assert {"Conv2d", "MatMul", "Softmax", "LayerNormalization", "Gelu", "Gemm", "Transpose"} <= set(sess.profile())
    allocs = sess.device_allocations()
    (again,) = sess.run([image])
    assert np.array_equal(again, logits) and sess.device_allocations() == allocs      # deterministic, pool in steady state

    (plain,) = HipSessionBuilder(unfused).build().run([image])
    np.testing.assert_allclose(plain, oracle_vit(image, params, fused=False), rtol=2e-4, atol=2e-4)
    # the two reference paths differ only by their GELU approximations
    assert np.max(np.abs(plain - logits)) < 0.2


def test_inference_session_like_altius_py(case, tmp_path):
    """altius_py.InferenceSession(path).run(None, {name: array}) (crates/altius_py/altius_py/__init__.py:4-30) with
    the rewrite pipeline of altius_py.session (crates/altius_py/src/lib.rs:52-62) on this backend."""
    case("InferenceSession on a ViT file")
    from altius_amd.inference import InferenceSession, load, session

    data, params = make_vit()
    path = tmp_path / "vit.onnx"
    path.write_bytes(data)
    image = rnd(B, 3, IMG, IMG)
    sess = InferenceSession(str(path), enable_profile=True)
    (logits,) = sess.run(None, {"image": image})
    np.testing.assert_allclose(logits, oracle_vit(image, params, fused=True), rtol=2e-4, atol=2e-4)
    assert "LayerNormalization" in sess.session.profile()
    with pytest.raises(RuntimeError, match="not found"):
        sess.run(None, {"picture": image})
    with pytest.raises(RuntimeError, match="Unknown backend"):
        session(load(str(path)), backend="cuda")


def test_elementwise_fusion_keeps_the_bits_of_the_plain_graph(case):
    """The exporter's graph with only fuse_elemwise_ops applied: fewer nodes, the same logits bit for bit."""
    case("ViT with element-wise chains fused")
    data, _ = make_vit()
    image = rnd(B, 3, IMG, IMG)
    plain = Model.load_onnx_from_buffer(data)
    fused = plain.clone()
    n = fused.fuse_elemwise_ops(extended=True)
    ops = [k["op_name"] for k in fused.nodes()]
    assert n >= 3 * LAYERS + 1 and ops.count("FusedElemwise") == n and "Erf" not in ops
    (want,) = HipSessionBuilder(plain).build().run([image])
    (got,) = HipSessionBuilder(fused).build().run([image])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
