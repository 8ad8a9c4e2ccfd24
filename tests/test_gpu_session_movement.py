"""Graphs with data-movement operators through the session: head split / merge, qkv split, cls-token
concat, embedding gather, masks, shape arithmetic (Shape -> Gather -> Concat -> Reshape) evaluated on
the host, aliasing reshapes, multiple outputs.  Expectations are numpy's routines and the CPU oracle."""
import numpy as np
import pytest

import oracle as O
import onnx_writer as W
from altius_amd._lib import ERR_ARG, AltiusHipError
from altius_amd.graph import BOOL, F32, I64, Model, Op
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(21)


def f32(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def run(model, *inputs):
    return HipSessionBuilder(model).build().run(list(inputs))


def test_head_split_and_merge(case):
    case("session: reshape + transpose round trip")
    x = f32(2, 197, 768)
    m = Model()
    v = m.new_val_named_and_shaped("x", x.shape)
    s1, t1, kt, t2, s2 = (m.new_val() for _ in range(5))
    m.add_node(Op.Reshape, [v, m.new_initializer(np.array([2, 197, 12, 64], np.int64))], [s1])
    m.add_node(Op.Transpose, [s1], [t1], perm=[0, 2, 1, 3])          # [2,12,197,64]
    m.add_node(Op.Transpose, [t1], [kt], perm=[0, 1, 3, 2])          # K^T [2,12,64,197]
    m.add_node(Op.Transpose, [t1], [t2], perm=[0, 2, 1, 3])          # back to [2,197,12,64]
    m.add_node(Op.Reshape, [t2, m.new_initializer(np.array([0, 0, -1], np.int64))], [s2])
    m.add_input(v)
    for o in (t1, kt, s2):
        m.add_output(o)
    heads, k_t, back = run(m, x)
    want = x.reshape(2, 197, 12, 64).transpose(0, 2, 1, 3)
    assert_bits_equal(heads, want, "split heads")
    assert_bits_equal(k_t, want.transpose(0, 1, 3, 2), "K^T")
    assert_bits_equal(back, x, "merge heads")


def test_qkv_split_and_cls_concat(case):
    case("session: Split (3 outputs), Concat, Slice, Gather")
    qkv = f32(2, 197, 2304)
    cls = f32(1, 1, 768)
    m = Model(opset_version=13)
    v = m.new_val_named_and_shaped("qkv", qkv.shape)
    q, k, vv, cat, sl, first = (m.new_val() for _ in range(6))
    m.add_node(Op.Split, [v, m.new_initializer(np.array([768, 768, 768], np.int64))], [q, k, vv], axis=2)
    c = m.new_initializer(np.broadcast_to(cls, (2, 1, 768)).copy())
    m.add_node(Op.Concat, [c, q], [cat], axis=1)                                                  # [2,198,768]
    i64 = lambda *a: m.new_initializer(np.array(a, np.int64))
    m.add_node(Op.Slice, [cat, i64(1), i64(198), i64(1), i64(1)], [sl])                         # drop the token again
    m.add_node(Op.Gather, [cat, m.new_initializer(np.array(0, np.int64))], [first], axis=1)       # class token [2,768]
    m.add_input(v)
    for o in (q, k, vv, cat, sl, first):
        m.add_output(o)
    gq, gk, gv, gcat, gsl, gfirst = run(m, qkv)
    for got, want in zip((gq, gk, gv), np.split(qkv, 3, axis=2)):
        assert_bits_equal(got, want, "split")
    assert_bits_equal(gq, O.split(qkv, [768, 768, 768], 2, strict=True)[0], "split vs oracle")
    want_cat = np.concatenate([np.broadcast_to(cls, (2, 1, 768)), gq], axis=1)
    assert_bits_equal(gcat, want_cat, "concat")
    assert_bits_equal(gsl, want_cat[:, 1:198], "slice")
    assert_bits_equal(gfirst, want_cat[:, 0], "gather")


def test_shape_arithmetic_runs_on_the_host(case):
    """x -> Shape -> Gather(0) -> Unsqueeze -> Concat with [-1] -> Reshape(x, .): the exporter's idiom for
    flatten-keeping-batch.  Shapes are unknown until run time; no integer kernel is launched."""
    case("session: dynamic reshape")
    x = f32(3, 5, 7)
    m = Model(opset_version=13)
    v = m.new_val_named("x")
    sh, b, bu, target, y, n_el = (m.new_val() for _ in range(6))
    m.add_node(Op.Shape, [v], [sh])
    m.add_node(Op.Gather, [sh, m.new_initializer(np.array(0, np.int64))], [b], axis=0)
    m.add_node(Op.Unsqueeze, [b, m.new_initializer(np.array([0], np.int64))], [bu])
    m.add_node(Op.Concat, [bu, m.new_initializer(np.array([-1], np.int64))], [target], axis=0)
    m.add_node(Op.Reshape, [v, target], [y])
    # sqrt(d_k)-style scalar: Shape -> Gather(-1) -> Cast(f32) -> Sqrt -> Div
    d, df, ds, z = (m.new_val() for _ in range(4))
    m.add_node(Op.Gather, [sh, m.new_initializer(np.array(-1, np.int64))], [d], axis=0)
    m.add_node(Op.Cast, [d], [df], to=1)
    m.add_node(Op.Sqrt, [df], [ds])
    m.add_node(Op.Div, [v, ds], [z])
    m.add_input(v)
    for o in (y, target, z):
        m.add_output(o)
    sess = HipSessionBuilder(m).build()
    for batch in (3, 6):                                   # the same session serves another batch size
        xb = f32(batch, 5, 7)
        gy, gt, gz = sess.run([xb])
        assert gt.dtype == np.int64 and gt.tolist() == [batch, -1]
        assert_bits_equal(gy, xb.reshape(batch, -1), "reshape")
        assert_bits_equal(gz, xb / np.sqrt(np.float32(7)), "scaled")


def test_where_mask_cast_greater_expand_tile(case):
    case("session: Greater -> Where, Cast, Expand, Tile")
    x = f32(2, 3, 8, 8)
    m = Model(opset_version=13)
    v = m.new_val_named_and_shaped("x", x.shape)
    g, w, ci, cf, ex, tl = (m.new_val() for _ in range(6))
    zero = m.new_initializer(np.array(0.0, np.float32))
    m.add_node(Op.Greater, [v, zero], [g])
    m.add_node(Op.Where, [g, v, m.new_initializer(np.array(-1.0, np.float32))], [w])
    m.add_node(Op.Cast, [v], [ci], to=7)
    m.add_node(Op.Cast, [ci], [cf], to=1)
    row = m.new_initializer(f32(1, 1, 1, 8))
    m.add_node(Op.Expand, [row, m.new_initializer(np.array([2, 3, 8, 8], np.int64))], [ex])
    m.add_node(Op.Tile, [v, m.new_initializer(np.array([1, 2, 1, 2], np.int64))], [tl])
    m.add_input(v)
    for o in (g, w, ci, cf, ex, tl):
        m.add_output(o)
    gg, gw, gci, gcf, gex, gtl = run(m, x)
    assert_bits_equal(gg, O.greater(x, np.float32(0), strict=True), "greater")
    assert_bits_equal(gw, np.where(x > 0, x, np.float32(-1)), "where")
    assert_bits_equal(gci, O.cast(x, np.int64), "f32 -> i64")
    assert_bits_equal(gcf, O.cast(O.cast(x, np.int64), np.float32, strict=True), "i64 -> f32")
    assert_bits_equal(gex, np.broadcast_to(m.initializer(row), x.shape), "expand")
    assert_bits_equal(gtl, np.tile(x, (1, 2, 1, 2)), "tile")


def test_cnn_tail_batchnorm_leakyrelu_gap_flatten(case):
    case("session: BatchNormalization -> LeakyRelu -> GlobalAveragePool -> Flatten, Squeeze/Unsqueeze, Clip")
    x = f32(4, 16, 7, 7)
    scale, bias, mean = f32(16), f32(16), f32(16)
    var = (RNG.random(16) + 0.1).astype(np.float32)
    m = Model(opset_version=13)
    v = m.new_val_named_and_shaped("x", x.shape)
    bn, lr, gp, fl, sq, us, cl = (m.new_val() for _ in range(7))
    m.add_node(Op.BatchNormalization, [v] + [m.new_initializer(a) for a in (scale, bias, mean, var)], [bn], epsilon=1e-3)
    m.add_node(Op.LeakyReLU, [bn], [lr], alpha=0.1)
    m.add_node(Op.GlobalAveragePool, [lr], [gp])
    m.add_node(Op.Flatten, [gp], [fl])
    m.add_node(Op.Squeeze, [gp, m.new_initializer(np.array([2, 3], np.int64))], [sq])
    m.add_node(Op.Unsqueeze, [sq, m.new_initializer(np.array([0], np.int64))], [us])
    m.add_node(Op.Clip, [lr, m.new_initializer(np.array(-0.05, np.float32)), m.new_initializer(np.array(1.5, np.float32))], [cl])
    m.add_input(v)
    for o in (lr, gp, fl, us, cl):
        m.add_output(o)
    glr, ggp, gfl, gus, gcl = run(m, x)
    want_lr = O.leaky_relu(O.batchnorm(x, scale, bias, mean, var, 1e-3), 0.1)
    assert_bits_equal(glr, want_lr, "bn + leaky relu")
    want_gp = O.global_average_pool(want_lr)
    assert_close(ggp, want_gp, what="global average pool")
    assert_bits_equal(gfl, ggp.reshape(4, 16), "flatten aliases the pooled tensor")
    assert_bits_equal(gus, ggp.reshape(1, 4, 16), "squeeze + unsqueeze")
    assert_bits_equal(gcl, np.clip(want_lr, np.float32(-0.05), np.float32(1.5)), "clip")


def test_embedding_lookup_from_int64_input_and_bad_index(case):
    case("session: Gather with indices from a graph input")
    table = f32(500, 64)
    m = Model()
    ids = m.new_val_named_and_shaped("ids", [1, 12], I64)
    e = m.new_val()
    m.add_node(Op.Gather, [m.new_initializer(table), ids], [e], axis=0)
    m.add_input(ids)
    m.add_output(e)
    sess = HipSessionBuilder(m).build()
    idx = RNG.integers(0, 500, size=(1, 12)).astype(np.int64)
    (got,) = sess.run([idx])
    assert_bits_equal(got, O.gather(table, idx, 0, strict=True), "embedding")
    bad = idx.copy()
    bad[0, 3] = 500
    with pytest.raises(AltiusHipError) as err:
        sess.run([bad])
    assert err.value.code == ERR_ARG and "Gather" in err.value.message
    (again,) = sess.run([idx])
    assert_bits_equal(again, got, "the session recovers")


def test_loaded_onnx_graph_runs(case):
    """The same kind of graph arriving as ONNX bytes: loader -> shape inference -> session."""
    case("session: ONNX bytes")
    x = f32(2, 6, 8)
    nodes = [W.node("Transpose", ["x"], ["t"], perm=[0, 2, 1]), W.node("Softmax", ["t"], ["p"], axis=-1),
             W.node("Reshape", ["p", "shape"], ["r"]), W.node("Relu", ["r"], ["y"])]
    data = W.model(W.graph(nodes, [W.tensor("shape", np.array([2, 48], np.int64))], [W.value_info("x", W.FLOAT, [2, 6, 8])],
                           [W.value_info("y", W.FLOAT, [2, 48])]))
    m = Model.load_onnx_from_buffer(data)
    (got,) = run(m, x)
    want = O.unary(O.RELU, O.softmax(np.ascontiguousarray(x.transpose(0, 2, 1))).reshape(2, 48))
    assert_close(got, want, what="onnx graph")
