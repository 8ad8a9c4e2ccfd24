"""Two more whole graphs as ONNX bytes, of the families the reference's scripts run
(crates/altius_py/mobilenet.py, bert.py): a MobileNetV3-style CNN (stem Conv + BatchNorm + hard-swish,
inverted-residual blocks with depthwise Conv and squeeze-excite, GlobalAveragePool, classifier Gemm)
and a BERT-style encoder layer (embedding Gather, the exporter's mask arithmetic
(1 - mask) * -10000 through Unsqueeze / Cast / Sub / Mul, scaled and masked attention, LayerNorm
chains, erf-GELU).  Each is loaded, rewritten by the session pipeline of altius_py
(crates/altius_py/src/lib.rs:52-62) and compared with the same computation carried out node by node
with the CPU oracle, whose Gelu / LayerNormalization are the fused operators' formulas."""
import os

import numpy as np
import pytest

import onnx_writer as W
import oracle as O
from altius_amd.graph import Model
from altius_amd.inference import InferenceSession, session
from altius_amd.session import HipSessionBuilder

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(77)


def rnd(*shape, scale=1.0, shift=0.0):
    return (RNG.standard_normal(shape) * scale + shift).astype(np.float32)


class G:
    def __init__(self):
        self.nodes, self.inits, self.n = [], [], 0

    def c(self, array):
        name = f"c{len(self.inits)}"
        self.inits.append(W.tensor(name, np.asarray(array)))
        return name

    def op(self, op_type, inputs, **attrs):
        out = f"v{self.n}"
        self.n += 1
        self.nodes.append(W.node(op_type, inputs, [out], **attrs))
        return out


# ---- MobileNetV3-style ---------------------------------------------------------------------------------
def hard_swish_nodes(g, x):
    return g.op("Mul", [x, g.op("HardSigmoid", [x], alpha=1.0 / 6.0, beta=0.5)])


def hard_swish_oracle(x):
    return O.binary(O.MUL, x, O.unary(O.HARDSIGMOID, x, np.float32(1.0 / 6.0), 0.5))


def make_mobilenet(batch=2, classes=10):
    p = {"stem_w": rnd(16, 3, 3, 3, scale=0.2), "stem_bn": [rnd(16, shift=1.0, scale=0.1), rnd(16, scale=0.1), rnd(16, scale=0.1),
                                                            np.abs(rnd(16)) + np.float32(0.5)],
         "blocks": [], "head_w": rnd(classes, 24, scale=0.2), "head_b": rnd(classes, scale=0.1)}
    g = G()
    x = g.op("Conv", ["image", g.c(p["stem_w"])], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1])
    x = g.op("BatchNormalization", [x] + [g.c(t) for t in p["stem_bn"]], epsilon=1e-5)
    x = hard_swish_nodes(g, x)
    cin = 16
    for cexp, cout, stride, k in ((32, 16, 1, 3), (48, 24, 2, 5)):
        blk = {"exp_w": rnd(cexp, cin, 1, 1, scale=0.2), "exp_b": rnd(cexp, scale=0.1),
               "dw_w": rnd(cexp, 1, k, k, scale=0.2), "dw_b": rnd(cexp, scale=0.1),
               "se1_w": rnd(cexp // 4, cexp, 1, 1, scale=0.2), "se1_b": rnd(cexp // 4, scale=0.1),
               "se2_w": rnd(cexp, cexp // 4, 1, 1, scale=0.2), "se2_b": rnd(cexp, scale=0.1),
               "proj_w": rnd(cout, cexp, 1, 1, scale=0.2), "proj_b": rnd(cout, scale=0.1), "stride": stride, "k": k,
               "residual": stride == 1 and cin == cout}
        p["blocks"].append(blk)
        y = hard_swish_nodes(g, g.op("Conv", [x, g.c(blk["exp_w"]), g.c(blk["exp_b"])], kernel_shape=[1, 1]))
        y = g.op("Conv", [y, g.c(blk["dw_w"]), g.c(blk["dw_b"])], kernel_shape=[k, k], strides=[stride, stride],
                 pads=[k // 2] * 4, group=cexp)
        y = g.op("Relu", [y])
        s = g.op("GlobalAveragePool", [y])
        s = g.op("Relu", [g.op("Conv", [s, g.c(blk["se1_w"]), g.c(blk["se1_b"])], kernel_shape=[1, 1])])
        s = g.op("HardSigmoid", [g.op("Conv", [s, g.c(blk["se2_w"]), g.c(blk["se2_b"])], kernel_shape=[1, 1])], alpha=1.0 / 6.0, beta=0.5)
        y = g.op("Mul", [y, s])
        y = g.op("Conv", [y, g.c(blk["proj_w"]), g.c(blk["proj_b"])], kernel_shape=[1, 1])
        x = g.op("Add", [x, y]) if blk["residual"] else y
        cin = cout
    x = g.op("Flatten", [g.op("GlobalAveragePool", [x])], axis=1)
    logits = g.op("Gemm", [x, g.c(p["head_w"]), g.c(p["head_b"])], transB=1)
    g.nodes.append(W.node("Identity", [logits], ["logits"]))
    data = W.model(W.graph(g.nodes, g.inits, [W.value_info("image", W.FLOAT, [batch, 3, 32, 32])],
                           [W.value_info("logits", W.FLOAT, [batch, classes])]), opsets=(("", 13),))
    return data, p


def oracle_mobilenet(image, p):
    x = O.conv2d(image, p["stem_w"], None, strides=(2, 2), pads=(1, 1, 1, 1))
    x = hard_swish_oracle(O.batchnorm(x, *p["stem_bn"], eps=1e-5))
    for b in p["blocks"]:
        y = hard_swish_oracle(O.conv2d(x, b["exp_w"], b["exp_b"]))
        k = b["k"]
        y = O.unary(O.RELU, O.conv2d(y, b["dw_w"], b["dw_b"], strides=(b["stride"],) * 2, pads=(k // 2,) * 4, group=y.shape[1]))
        s = O.global_average_pool(y)
        s = O.unary(O.RELU, O.conv2d(s, b["se1_w"], b["se1_b"]))
        s = O.unary(O.HARDSIGMOID, O.conv2d(s, b["se2_w"], b["se2_b"]), np.float32(1.0 / 6.0), 0.5)
        y = O.conv2d(O.binary(O.MUL, y, s), b["proj_w"], b["proj_b"])
        x = O.binary(O.ADD, x, y) if b["residual"] else y
    pooled = O.global_average_pool(x).reshape(x.shape[0], -1)
    return O.gemm(pooled, p["head_w"], p["head_b"], trans_b=True)


def test_mobilenet_style_cnn(case, tmp_path):
    case("MobileNetV3-style CNN from ONNX bytes")
    data, p = make_mobilenet()
    image = rnd(2, 3, 32, 32)
    want = oracle_mobilenet(image, p)
    model = Model.load_onnx_from_buffer(data)
    (plain,) = HipSessionBuilder(model).build().run([image])
    np.testing.assert_allclose(plain, want, rtol=2e-4, atol=2e-4)
    # the session pipeline: hard-swish and squeeze-excite pairs become FusedElemwise nodes, same bits
    sess = session(model, enable_profiling=True)
    (logits,) = sess.run({"image": image})
    assert "FusedElemwise" in sess.profile()
    assert np.array_equal(logits.view(np.uint32), plain.view(np.uint32))
    path = os.path.join(tmp_path, "mobilenet.onnx")
    with open(path, "wb") as f:
        f.write(data)
    (again,) = InferenceSession(path).run(None, {"image": image})
    assert np.array_equal(again, logits)


# ---- BERT-style --------------------------------------------------------------------------------------
B, T, H, NH, FF, VOCAB = 2, 24, 64, 4, 128, 50
DH = H // NH


def make_bert():
    p = {"tok": rnd(VOCAB, H, scale=0.5), "pos": rnd(T, H, scale=0.1), "ln0": (rnd(H, shift=1.0, scale=0.1), rnd(H, scale=0.1)),
         "wq": rnd(H, H, scale=0.1), "bq": rnd(H, scale=0.1), "wk": rnd(H, H, scale=0.1), "bk": rnd(H, scale=0.1),
         "wv": rnd(H, H, scale=0.1), "bv": rnd(H, scale=0.1), "wo": rnd(H, H, scale=0.1), "bo": rnd(H, scale=0.1),
         "ln1": (rnd(H, shift=1.0, scale=0.1), rnd(H, scale=0.1)), "w1": rnd(H, FF, scale=0.1), "b1": rnd(FF, scale=0.1),
         "w2": rnd(FF, H, scale=0.1), "b2": rnd(H, scale=0.1), "ln2": (rnd(H, shift=1.0, scale=0.1), rnd(H, scale=0.1))}
    g = G()
    f = lambda v: g.c(np.array(v, np.float32))

    def layer_norm(x, gamma, beta):
        mean = g.op("ReduceMean", [x], axes=[-1])
        d = g.op("Sub", [x, mean])
        var = g.op("ReduceMean", [g.op("Pow", [d, f(2.0)])], axes=[-1])
        return g.op("Add", [g.op("Mul", [g.op("Div", [d, g.op("Sqrt", [g.op("Add", [var, f(1e-12)])])]), g.c(gamma)]), g.c(beta)])

    def linear(x, w, b):
        return g.op("Add", [g.op("MatMul", [x, g.c(w)]), g.c(b)])

    def heads(x):
        return g.op("Transpose", [g.op("Reshape", [x, g.c(np.array([B, T, NH, DH], np.int64))])], perm=[0, 2, 1, 3])

    x = g.op("Add", [g.op("Gather", [g.c(p["tok"]), "input_ids"], axis=0), g.c(p["pos"])])
    x = layer_norm(x, *p["ln0"])
    # (1 - mask[:, None, None, :]) * -10000, the way exporters write it
    m = g.op("Cast", [g.op("Unsqueeze", ["attention_mask"], axes=[1, 2])], to=W.FLOAT)
    m = g.op("Mul", [g.op("Sub", [f(1.0), m]), f(-10000.0)])
    q, k, v = heads(linear(x, p["wq"], p["bq"])), heads(linear(x, p["wk"], p["bk"])), heads(linear(x, p["wv"], p["bv"]))
    s = g.op("MatMul", [q, g.op("Transpose", [k], perm=[0, 1, 3, 2])])
    s = g.op("Softmax", [g.op("Add", [g.op("Div", [s, f(np.sqrt(DH))]), m])], axis=-1)
    a = g.op("Reshape", [g.op("Transpose", [g.op("MatMul", [s, v])], perm=[0, 2, 1, 3]), g.c(np.array([B, T, H], np.int64))])
    x = layer_norm(g.op("Add", [x, linear(a, p["wo"], p["bo"])]), *p["ln1"])
    h = linear(x, p["w1"], p["b1"])
    h = g.op("Mul", [g.op("Mul", [h, g.op("Add", [g.op("Erf", [g.op("Div", [h, f(1.4142135)])]), f(1.0)])]), f(0.5)])
    x = layer_norm(g.op("Add", [x, linear(h, p["w2"], p["b2"])]), *p["ln2"])
    g.nodes.append(W.node("Identity", [x], ["hidden"]))
    data = W.model(W.graph(g.nodes, g.inits, [W.value_info("input_ids", W.INT64, [B, T]), W.value_info("attention_mask", W.INT64, [B, T])],
                           [W.value_info("hidden", W.FLOAT, [B, T, H])]), opsets=(("", 11),))
    return data, p


def oracle_bert(ids, mask, p):
    s = lambda v: np.array(v, np.float32)
    ln = lambda x, gb: O.layer_norm(x, gb[0], gb[1], 1e-12)
    lin = lambda x, w, b: O.binary(O.ADD, O.matmul(x, w), b)
    heads = lambda x: O.transpose(x.reshape(B, T, NH, DH), (0, 2, 1, 3))
    x = ln(O.binary(O.ADD, p["tok"][ids], p["pos"]), p["ln0"])
    m = O.binary(O.MUL, O.binary(O.SUB, s(1.0), mask[:, None, None, :].astype(np.float32)), s(-10000.0))
    q, k, v = heads(lin(x, p["wq"], p["bq"])), heads(lin(x, p["wk"], p["bk"])), heads(lin(x, p["wv"], p["bv"]))
    sc = O.binary(O.ADD, O.binary(O.DIV, O.matmul(q, O.transpose(k, (0, 1, 3, 2))), s(np.sqrt(DH))), m)
    a = O.transpose(O.matmul(O.softmax(sc), v), (0, 2, 1, 3)).reshape(B, T, H)
    x = ln(O.binary(O.ADD, x, lin(a, p["wo"], p["bo"])), p["ln1"])
    h = lin(x, p["w1"], p["b1"])
    x = ln(O.binary(O.ADD, x, lin(O.unary(O.GELU, h), p["w2"], p["b2"])), p["ln2"])
    return x


@pytest.mark.parametrize("fused_attention", [False, True])
def test_bert_style_encoder_layer(case, fused_attention):
    case(f"BERT-style encoder layer from ONNX bytes, one-kernel attention {fused_attention}")
    data, p = make_bert()
    ids = RNG.integers(0, VOCAB, size=(B, T)).astype(np.int64)
    mask = np.ones((B, T), np.int64)
    mask[0, 17:] = 0
    mask[1, 9:] = 0
    model = Model.load_onnx_from_buffer(data)
    sess = session(model, enable_profiling=True, fused_attention=fused_attention)
    (hidden,) = sess.run({"input_ids": ids, "attention_mask": mask})
    np.testing.assert_allclose(hidden, oracle_bert(ids, mask, p), rtol=3e-4, atol=3e-4)
    ops = set(sess.profile())
    assert {"LayerNormalization", "FusedElemwise", "Softmax", "Gather", "MatMul"} <= ops
    # the scale and the mask went into the Softmax, the erf chain became Gelu, the LayerNorm chains one node each,
    # the bias rows went into their products
    assert not ops & {"Div", "Erf", "Pow", "Sqrt", "ReduceMean"}


# ---- GPT-2-style -------------------------------------------------------------------------------------
# The graph `python -m transformers.onnx --model=gpt2` writes (crates/altius_py/gpt2.py:1), one block of it:
# token and position Gathers, LayerNorm chains, every linear layer as Reshape -> Gemm -> Reshape, one Split of the
# fused qkv projection, keys transposed straight to [b, h, d, t], Div by sqrt(d), the causal mask as Where over a
# Slice of a lower-triangular bool buffer, the padding mask added, tanh-GELU written out, the output projection
# on the transposed token table.
GB, GT, GH, GNH, GFF, GV, GCTX = 2, 20, 128, 2, 256, 60, 32
GDH = GH // GNH


def make_gpt2():
    p = {"wte": rnd(GV, GH, scale=0.3), "wpe": rnd(GCTX, GH, scale=0.1), "ln1": (rnd(GH, shift=1.0, scale=0.1), rnd(GH, scale=0.1)),
         "w_qkv": rnd(GH, 3 * GH, scale=0.08), "b_qkv": rnd(3 * GH, scale=0.05), "w_o": rnd(GH, GH, scale=0.08), "b_o": rnd(GH, scale=0.05),
         "ln2": (rnd(GH, shift=1.0, scale=0.1), rnd(GH, scale=0.1)), "w_fc": rnd(GH, GFF, scale=0.08), "b_fc": rnd(GFF, scale=0.05),
         "w_pr": rnd(GFF, GH, scale=0.08), "b_pr": rnd(GH, scale=0.05), "lnf": (rnd(GH, shift=1.0, scale=0.1), rnd(GH, scale=0.1))}
    g = G()
    f = lambda v: g.c(np.array(v, np.float32))
    i64 = lambda *v: g.c(np.array(v, np.int64))

    def layer_norm(x, gamma, beta):
        mean = g.op("ReduceMean", [x], axes=[-1])
        d = g.op("Sub", [x, mean])
        var = g.op("ReduceMean", [g.op("Pow", [d, f(2.0)])], axes=[-1])
        return g.op("Add", [g.op("Mul", [g.op("Div", [d, g.op("Sqrt", [g.op("Add", [var, f(1e-5)])])]), g.c(gamma)]), g.c(beta)])

    def conv1d(x, w, b, n_in, n_out):  # HF's Conv1D: x.view(-1, n_in) @ w + b, viewed back
        y = g.op("Gemm", [g.op("Reshape", [x, i64(-1, n_in)]), g.c(w), g.c(b)])
        return g.op("Reshape", [y, i64(GB, GT, n_out)])

    x = g.op("Add", [g.op("Gather", [g.c(p["wte"]), "input_ids"], axis=0), g.op("Gather", [g.c(p["wpe"]), "position_ids"], axis=0)])
    h = layer_norm(x, *p["ln1"])
    qkv = conv1d(h, p["w_qkv"], p["b_qkv"], GH, 3 * GH)
    parts = [f"qkv{i}" for i in range(3)]
    g.nodes.append(W.node("Split", [qkv, i64(GH, GH, GH)], parts, axis=2))
    heads = lambda t, perm: g.op("Transpose", [g.op("Reshape", [t, i64(GB, GT, GNH, GDH)])], perm=perm)
    q, k, v = heads(parts[0], [0, 2, 1, 3]), heads(parts[1], [0, 2, 3, 1]), heads(parts[2], [0, 2, 1, 3])
    s = g.op("Div", [g.op("MatMul", [q, k]), f(np.sqrt(GDH))])
    tril = np.tril(np.ones((1, 1, GCTX, GCTX), np.bool_))
    causal = g.op("Slice", [g.c(tril), i64(0, 0), i64(GT, GT), i64(2, 3)])
    s = g.op("Where", [causal, s, f(-1e4)])
    pad = g.op("Mul", [g.op("Sub", [f(1.0), g.op("Cast", [g.op("Unsqueeze", ["attention_mask", i64(1, 2)])], to=W.FLOAT)]), f(-10000.0)])
    s = g.op("Softmax", [g.op("Add", [s, pad])], axis=-1)
    a = g.op("Reshape", [g.op("Transpose", [g.op("MatMul", [s, v])], perm=[0, 2, 1, 3]), i64(GB, GT, GH)])
    x = g.op("Add", [x, conv1d(a, p["w_o"], p["b_o"], GH, GH)])
    h = conv1d(layer_norm(x, *p["ln2"]), p["w_fc"], p["b_fc"], GH, GFF)
    # 0.5 h (1 + tanh(0.79788456 (h + 0.044715 h^3))) as the exporter writes it (fast_gelu_fusion.rs:5-190)
    inner = g.op("Mul", [g.op("Add", [h, g.op("Mul", [g.op("Pow", [h, f(3.0)]), f(0.044715)])]), f(0.7978845608)])
    h = g.op("Mul", [g.op("Mul", [h, f(0.5)]), g.op("Add", [g.op("Tanh", [inner]), f(1.0)])])
    x = g.op("Add", [x, conv1d(h, p["w_pr"], p["b_pr"], GFF, GH)])
    x = layer_norm(x, *p["lnf"])
    logits = g.op("MatMul", [x, g.op("Transpose", [g.c(p["wte"])], perm=[1, 0])])
    g.nodes.append(W.node("Identity", [logits], ["logits"]))
    data = W.model(W.graph(g.nodes, g.inits,
                           [W.value_info(nm, W.INT64, [GB, GT]) for nm in ("input_ids", "attention_mask", "position_ids")],
                           [W.value_info("logits", W.FLOAT, [GB, GT, GV])]), opsets=(("", 13),))
    return data, p


def oracle_gpt2(ids, mask, pos, p):
    s = lambda v: np.array(v, np.float32)
    ln = lambda x, gb: O.layer_norm(x, gb[0], gb[1], 1e-5)
    lin = lambda x, w, b: O.gemm(x.reshape(-1, x.shape[-1]), w, b).reshape(x.shape[:-1] + (w.shape[1],))
    x = O.binary(O.ADD, p["wte"][ids], p["wpe"][pos])
    qkv = lin(ln(x, p["ln1"]), p["w_qkv"], p["b_qkv"])
    q, k, v = (np.ascontiguousarray(t.reshape(GB, GT, GNH, GDH).transpose(0, 2, 1, 3)) for t in np.split(qkv, 3, axis=2))
    sc = O.binary(O.DIV, O.matmul(q, np.ascontiguousarray(k.transpose(0, 1, 3, 2))), s(np.sqrt(GDH)))
    sc = np.where(np.tril(np.ones((GT, GT), np.bool_))[None, None], sc, s(-1e4)).astype(np.float32)
    pad = O.binary(O.MUL, O.binary(O.SUB, s(1.0), mask[:, None, None, :].astype(np.float32)), s(-10000.0))
    a = O.matmul(O.softmax(O.binary(O.ADD, sc, pad)), v).transpose(0, 2, 1, 3).reshape(GB, GT, GH)
    x = O.binary(O.ADD, x, lin(np.ascontiguousarray(a), p["w_o"], p["b_o"]))
    h = O.unary(O.GELU, lin(ln(x, p["ln2"]), p["w_fc"], p["b_fc"]))
    x = ln(O.binary(O.ADD, x, lin(h, p["w_pr"], p["b_pr"])), p["lnf"])
    return O.matmul(x, np.ascontiguousarray(p["wte"].T))


def test_gpt2_style_decoder_block(case):
    case("GPT-2-style decoder block from ONNX bytes")
    data, p = make_gpt2()
    ids = RNG.integers(0, GV, size=(GB, GT)).astype(np.int64)
    mask = np.ones((GB, GT), np.int64)
    mask[1, 13:] = 0
    pos = np.tile(np.arange(GT, dtype=np.int64), (GB, 1))
    model = Model.load_onnx_from_buffer(data)
    sess = session(model, enable_profiling=True)
    (logits,) = sess.run({"input_ids": ids, "attention_mask": mask, "position_ids": pos})
    np.testing.assert_allclose(logits, oracle_gpt2(ids, mask, pos, p), rtol=5e-4, atol=5e-4)
    ops = set(sess.profile())
    assert {"LayerNormalization", "Gemm", "Where", "Softmax", "Gather", "MatMul", "Gelu"} <= ops
    assert not ops & {"Tanh", "Pow", "Sqrt", "ReduceMean"}      # the tanh chain became Gelu, the LayerNorm chains one node each


@pytest.mark.parametrize("batch", [1, 8, 24])
def test_full_width_vit_encoder_every_fast_path_agrees_with_the_plain_one(case, batch):
    """A ViT-B/16-shaped encoder at full width (12 layers, 768 wide, 12 heads of 64, 197 tokens) after the reference's own
    rewrites, run the plain way (fp32 kernels only, every operator its own kernel, no views) and with everything this
    backend adds (softmax prologue, MatMul bias, element-wise chains, views, one-kernel attention, the activation and
    the residual Add done by the products, the k cut at batch 1, the bf16 route from batch 8 on, graph replay): the
    logits agree to 2e-4 of their range, and replaying gives the eager run's bits."""
    from altius_amd import device as D
    from altius_amd import graphs
    from altius_amd.graph import Tensor

    case(f"full-width ViT-B/16-shaped encoder, batch {batch}")
    base = graphs.vit_encoder(batch, layers=12)
    assert base.fuse_layer_norm() == 25 and base.fuse_gelu() == 12
    base.eliminate_identity()
    x = Tensor.from_numpy(np.random.default_rng(5).standard_normal((batch, 197, 768)).astype(np.float32))

    plain = HipSessionBuilder(base.clone()).with_gemm_algorithm(D.GEMM_FP32).with_strided_views(False).build()
    want = np.array(plain.run([x])[0])
    assert plain.copies_avoided() == 0
    plain.close()

    fast = base.clone()
    fast.fuse_softmax_prologue(), fast.fuse_matmul_bias(), fast.fuse_transpose_matmul(), fast.fuse_elemwise_ops(extended=True)
    sess = HipSessionBuilder(fast).with_gemm_algorithm(D.GEMM_AUTO).with_fused_attention().with_graph_replay().build()
    got = np.array(sess.run([x])[0])
    assert sess.copies_avoided() > 0
    scale = float(np.abs(want).max())
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-4 * scale)
    for _ in range(3):  # the second run records, later ones replay
        again = np.array(sess.run([x])[0])
        assert np.array_equal(again, got)
    assert sess.graph_replays() >= 1
    sess.close()
