"""Split / Transpose results that only MatMuls read are strided views, and a MatMul read only by a Transpose
writes that Transpose's layout: the session with views must give, bit for bit, what the session that copies
gives (same kernels, same values, other addresses), and both must match NumPy's definition of the graph.
Also every way a view has to fall back to a copy."""
import numpy as np
import pytest

from altius_amd.graph import Model, Op, Tensor
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(2025)


def run_both(model, feeds, exact=True, attention=False):
    """Outputs with views and with copies, and how many nodes the first run served without a copy.  attention=True
    opts in to the one-kernel attention, and exact=False goes with it where that kernel replaces three operators
    (other summation orders: 2e-4 relative)."""
    outs = []
    avoided = 0
    for views in (True, False):
        sess = HipSessionBuilder(model.clone()).with_strided_views(views).with_fused_attention(attention and views).build()
        for _ in range(2):  # the second run reuses pooled blocks: a stale view would show
            got = [np.array(t) for t in sess.run([Tensor.from_numpy(x) for x in feeds])]
        if views:
            avoided = sess.copies_avoided()
        else:
            assert sess.copies_avoided() == 0
        sess.close()
        outs.append(got)
    for a, b in zip(*outs):
        if exact:
            assert_bits_equal(a, b, "views vs copies")
        else:
            np.testing.assert_allclose(a, b, rtol=2e-4, atol=2e-5)
    return outs[0], avoided


def i64(m, *v):
    return m.new_initializer(np.array(v, np.int64))


def node(m, op, inputs, n_out=1, **attrs):
    outs = [m.new_val() for _ in range(n_out)]
    m.add_node(op, inputs, outs, **attrs)
    return outs[0] if n_out == 1 else outs


def attention(batch, tokens, heads, d, fold_kt):
    """qkv [b, t, 3 h d] -> Split -> Reshape -> Transpose(0,2,1,3) -> QK^T -> Softmax -> PV -> Transpose -> Reshape -> proj."""
    hd = heads * d
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("qkv", [batch, tokens, 3 * hd])
    m.add_input(x)
    parts = node(m, Op.Split, [x, i64(m, hd, hd, hd)], 3, axis=2)
    q, k, v = (node(m, Op.Transpose, [node(m, Op.Reshape, [p, i64(m, batch, tokens, heads, d)])], perm=[0, 2, 1, 3]) for p in parts)
    s = node(m, Op.MatMul, [q, node(m, Op.Transpose, [k], perm=[0, 1, 3, 2])])
    s = node(m, Op.Softmax, [s], axis=-1)
    a = node(m, Op.Reshape, [node(m, Op.Transpose, [node(m, Op.MatMul, [s, v])], perm=[0, 2, 1, 3]), i64(m, batch, tokens, hd)])
    w = (RNG.standard_normal((hd, hd)) * 0.1).astype(np.float32)
    out = node(m, Op.MatMul, [a, m.new_initializer(w)])
    m.add_output(out)
    if fold_kt:
        m.fuse_transpose_matmul()
    return m, w


def attention_numpy(x, heads, d, w):
    b, t, _ = x.shape
    hd = heads * d
    q, k, v = (x[:, :, i * hd:(i + 1) * hd].reshape(b, t, heads, d).transpose(0, 2, 1, 3).astype(np.float64) for i in range(3))
    s = q @ k.transpose(0, 1, 3, 2)
    s = np.exp(s - s.max(-1, keepdims=True))
    s /= s.sum(-1, keepdims=True)
    return (s @ v).transpose(0, 2, 1, 3).reshape(b, t, hd) @ w.astype(np.float64)


@pytest.mark.parametrize("fold_kt", [False, True])
@pytest.mark.parametrize("batch,tokens,heads,d", [(2, 197, 12, 64), (3, 50, 4, 32), (1, 7, 1, 8), (4, 33, 3, 20)])
def test_attention_reads_and_writes_heads_in_place(case, batch, tokens, heads, d, fold_kt):
    case(f"attention views b={batch} t={tokens} h={heads} d={d} fold_kt={fold_kt}")
    m, w = attention(batch, tokens, heads, d, fold_kt)
    x = (RNG.standard_normal((batch, tokens, 3 * heads * d)) * 0.3).astype(np.float32)
    # A default session: views, three operators.  Split, three head transposes, (the K^T transpose unless folded,)
    # and the merge transpose behind P V are not copied, and not a bit changes.
    (got,), avoided = run_both(m, [x], exact=True)
    assert avoided == (5 if fold_kt else 6), avoided
    np.testing.assert_allclose(got, attention_numpy(x, heads, d, w), rtol=2e-4, atol=2e-5)
    # Opted in to the one-kernel attention (it takes 64-wide heads): also the first product and the Softmax.
    fused = d == 64
    (got,), avoided = run_both(m, [x], exact=not fused, attention=True)
    assert avoided == (5 if fold_kt else 6) + (2 if fused else 0), avoided
    np.testing.assert_allclose(got, attention_numpy(x, heads, d, w), rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("batch,tokens,planes", [(24, 45, True), (22, 197, True), (4, 45, False)])
def test_attention_writes_the_operand_planes_of_the_projection_behind_it(case, batch, tokens, planes):
    """On the bf16 route, with the one-kernel attention and heads enough for full blocks, the attention's output is
    read by nothing but the Transpose it is written ahead of, the Reshape and the projection: it leaves the kernel as
    that product's three bf16 planes and the separate split is not launched (one more copy avoided than the first
    product's and the Softmax's).  Checked against the definition and against the same session with the three
    operators apart, to the bars of the attention kernel.  With too few heads for the bf16 kernel's blocks the fp32
    kernel runs and the projection splits its operand itself."""
    case(f"attention -> planes -> projection, b={batch} t={tokens}")
    from altius_amd import device as D

    heads, d = 12, 64
    m, w = attention(batch, tokens, heads, d, True)
    x = (RNG.standard_normal((batch, tokens, 3 * heads * d)) * 0.3).astype(np.float32)
    outs, avoided = [], []
    for fused in (True, False):
        sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(D.GEMM_BF16X3).with_fused_attention(fused).build()
        for _ in range(2):
            (got,) = [np.array(t) for t in sess.run([Tensor.from_numpy(x)])]
        avoided.append(sess.copies_avoided())
        sess.close()
        outs.append(got)
    assert avoided[0] == avoided[1] + (3 if planes else 2), avoided  # the first product's, the Softmax's, the operand split
    want = attention_numpy(x, heads, d, w)
    np.testing.assert_allclose(outs[0], want, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(outs[0], outs[1], rtol=2e-4, atol=2e-5)


def test_attention_planes_are_not_planned_for_a_reshape_that_keeps_the_heads_apart(case):
    """The same chain with the Reshape behind the merge Transpose giving [b, t * h, 64] and weights of 64 rows: a
    valid graph whose last product has another geometry than the planes would be written for.  The plan must leave
    it to the ordinary route (one copy avoided fewer than with the merging Reshape) and the result must be right."""
    case("attention -> Transpose -> Reshape [b, t*h, 64] -> MatMul [64, n]")
    from altius_amd import device as D

    batch, tokens, heads, d = 24, 45, 12, 64
    hd = heads * d
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("qkv", [batch, tokens, 3 * hd])
    m.add_input(x)
    parts = node(m, Op.Split, [x, i64(m, hd, hd, hd)], 3, axis=2)
    q, k, v = (node(m, Op.Transpose, [node(m, Op.Reshape, [p, i64(m, batch, tokens, heads, d)])], perm=[0, 2, 1, 3]) for p in parts)
    s = node(m, Op.Softmax, [node(m, Op.MatMul, [q, node(m, Op.Transpose, [k], perm=[0, 1, 3, 2])])], axis=-1)
    a = node(m, Op.Reshape, [node(m, Op.Transpose, [node(m, Op.MatMul, [s, v])], perm=[0, 2, 1, 3]), i64(m, batch, tokens * heads, d)])
    w = (RNG.standard_normal((d, 96)) * 0.1).astype(np.float32)
    m.add_output(node(m, Op.MatMul, [a, m.new_initializer(w)]))
    m.fuse_transpose_matmul()
    feed = (RNG.standard_normal((batch, tokens, 3 * hd)) * 0.3).astype(np.float32)
    sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(D.GEMM_BF16X3).with_fused_attention(True).build()
    for _ in range(2):
        (got,) = [np.array(t) for t in sess.run([Tensor.from_numpy(feed)])]
    sess.close()
    qn, kn, vn = (feed[:, :, i * hd:(i + 1) * hd].reshape(batch, tokens, heads, d).transpose(0, 2, 1, 3).astype(np.float64) for i in range(3))
    p = qn @ kn.transpose(0, 1, 3, 2)
    p = np.exp(p - p.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = (p @ vn).transpose(0, 2, 1, 3).reshape(batch, tokens * heads, d) @ w.astype(np.float64)
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-5)


def test_view_with_another_reader_is_copied(case):
    """A part that an element-wise operator also reads is not made a view; its siblings' fate follows (one Split node)."""
    case("split part read by Add as well")
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [2, 9, 24])
    m.add_input(x)
    a, b = node(m, Op.Split, [x, i64(m, 12, 12)], 2, axis=2)
    w = RNG.standard_normal((12, 5)).astype(np.float32)
    y = node(m, Op.MatMul, [a, m.new_initializer(w)])
    z = node(m, Op.Add, [node(m, Op.MatMul, [b, m.new_initializer(w)]), node(m, Op.ReduceMean, [b], axes=[-1], keep_dims=True)])
    m.add_output(y)
    m.add_output(z)
    xv = RNG.standard_normal((2, 9, 24)).astype(np.float32)
    (gy, gz), avoided = run_both(m, [xv])
    assert avoided == 0
    np.testing.assert_allclose(gy, xv[:, :, :12] @ w, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gz, xv[:, :, 12:] @ w + xv[:, :, 12:].mean(-1, keepdims=True), rtol=1e-5, atol=1e-5)


def test_split_part_that_is_a_graph_output_is_copied(case):
    case("split part as graph output")
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [6, 10])
    m.add_input(x)
    a, b = node(m, Op.Split, [x, i64(m, 4, 6)], 2, axis=1)
    w = RNG.standard_normal((4, 3)).astype(np.float32)
    m.add_output(node(m, Op.MatMul, [a, m.new_initializer(w)]))
    m.add_output(b)
    xv = RNG.standard_normal((6, 10)).astype(np.float32)
    (gy, gb), avoided = run_both(m, [xv])
    assert avoided == 0
    np.testing.assert_allclose(gy, xv[:, :4] @ w, rtol=1e-5, atol=1e-5)
    assert_bits_equal(gb, xv[:, 4:], "second part")


@pytest.mark.parametrize("axis", [0, 1, 2])
def test_split_on_any_axis_feeds_matmul_in_place(case, axis):
    case(f"split axis {axis} -> matmul")
    shape = [4, 6, 8]
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", shape)
    m.add_input(x)
    half = shape[axis] // 2
    a, b = node(m, Op.Split, [x, i64(m, half, half)], 2, axis=axis)
    k = a_shape_last = shape[2] if axis != 2 else half
    w = RNG.standard_normal((k, 5)).astype(np.float32)
    m.add_output(node(m, Op.MatMul, [a, m.new_initializer(w)]))
    m.add_output(node(m, Op.MatMul, [b, m.new_initializer(w)]))
    xv = RNG.standard_normal(shape).astype(np.float32)
    (ga, gb), avoided = run_both(m, [xv])
    assert avoided == 1
    pa, pb = np.split(xv, 2, axis=axis)
    np.testing.assert_allclose(ga, pa @ w, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(gb, pb @ w, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("perm,side", [([1, 0], 0), ([1, 0], 1), ([0, 2, 1], 0), ([0, 2, 1], 1), ([1, 0, 2], 0), ([2, 0, 1], 0), ([2, 1, 0], 1)])
def test_transposed_operand_of_any_permutation(case, perm, side):
    """A lazy Transpose in front of either operand: unit row stride flips the product's transpose flag, other
    permutations are read through batch strides or, when no unit stride is left, copied."""
    case(f"transpose {perm} as operand {side}")
    shape = [5, 6, 7][:len(perm)]
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", shape)
    m.add_input(x)
    t = node(m, Op.Transpose, [x], perm=perm)
    tshape = [shape[p] for p in perm]
    if side == 0:
        other = RNG.standard_normal((tshape[-1], 4)).astype(np.float32)
        out = node(m, Op.MatMul, [t, m.new_initializer(other)])
    else:
        other = RNG.standard_normal((3, tshape[-2])).astype(np.float32)
        out = node(m, Op.MatMul, [m.new_initializer(other), t])
    m.add_output(out)
    xv = RNG.standard_normal(shape).astype(np.float32)
    (got,), avoided = run_both(m, [xv])
    assert avoided == 1
    want = (xv.transpose(perm) @ other) if side == 0 else (other @ xv.transpose(perm))
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_reshape_that_a_view_cannot_express_copies(case):
    """Transpose(0,2,1,3) then Reshape that merges the two middle axes: no strides describe it, so the Reshape copies."""
    case("reshape of a view that needs a copy")
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [2, 3, 4, 5])
    m.add_input(x)
    t = node(m, Op.Transpose, [x], perm=[0, 2, 1, 3])
    r = node(m, Op.Reshape, [t, i64(m, 2, 12, 5)])
    w = RNG.standard_normal((5, 6)).astype(np.float32)
    m.add_output(node(m, Op.MatMul, [r, m.new_initializer(w)]))
    xv = RNG.standard_normal((2, 3, 4, 5)).astype(np.float32)
    (got,), _ = run_both(m, [xv])
    np.testing.assert_allclose(got, xv.transpose(0, 2, 1, 3).reshape(2, 12, 5) @ w, rtol=1e-5, atol=1e-5)


def test_three_independent_batch_axes_fall_back(case):
    """[a, b, c, t, d] heads taken out of the middle: three batch axes that do not fold; the operands are copied."""
    case("three batch axes")
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [2, 3, 5, 4, 6])
    m.add_input(x)
    t = node(m, Op.Transpose, [x], perm=[2, 1, 0, 3, 4])        # [5, 3, 2, 4, 6]: batch strides 24, 120, 360
    y = m.new_val_named_and_shaped("y", [5, 3, 2, 6, 7])
    m.add_input(y)
    m.add_output(node(m, Op.MatMul, [t, y]))
    xv = RNG.standard_normal((2, 3, 5, 4, 6)).astype(np.float32)
    yv = RNG.standard_normal((5, 3, 2, 6, 7)).astype(np.float32)
    (got,), _ = run_both(m, [xv, yv])
    np.testing.assert_allclose(got, xv.transpose(2, 1, 0, 3, 4) @ yv, rtol=1e-5, atol=1e-5)


def test_matmul_writes_the_layout_of_the_transpose_behind_it(case):
    case("matmul -> transpose written in place")
    for perm in ([0, 2, 1, 3], [1, 0, 2, 3], [2, 0, 1, 3], [1, 2, 0, 3]):
        m = Model(opset_version=13)
        a = m.new_val_named_and_shaped("a", [2, 3, 9, 4])
        b = m.new_val_named_and_shaped("b", [2, 3, 4, 6])
        m.add_input(a)
        m.add_input(b)
        t = node(m, Op.Transpose, [node(m, Op.MatMul, [a, b])], perm=perm)
        m.add_output(node(m, Op.ReLU, [t]))
        av, bv = RNG.standard_normal((2, 3, 9, 4)).astype(np.float32), RNG.standard_normal((2, 3, 4, 6)).astype(np.float32)
        (got,), avoided = run_both(m, [av, bv])
        assert avoided == 1, (perm, avoided)
        np.testing.assert_allclose(got, np.maximum((av @ bv).transpose(perm), 0), rtol=1e-5, atol=1e-5)


# ---- the activation between two products, folded into the second one's operand split ----

from altius_amd import device as D  # noqa: E402
from altius_amd._lib import ERR_ARG, ERR_UNSUPPORTED, AltiusHipError, check  # noqa: E402


def mlp(rows, hidden, inner, act, second_reader=False):
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", list(rows) + [hidden])
    m.add_input(x)
    w1 = (RNG.standard_normal((hidden, inner)) * 0.2).astype(np.float32)
    w2 = (RNG.standard_normal((inner, hidden)) * 0.2).astype(np.float32)
    b1 = RNG.standard_normal(inner).astype(np.float32)
    h = node(m, Op.Add, [node(m, Op.MatMul, [x, m.new_initializer(w1)]), m.new_initializer(b1)])
    a = node(m, act, [h])
    m.add_output(node(m, Op.MatMul, [a, m.new_initializer(w2)]))
    if second_reader:
        m.add_output(node(m, Op.Sqrt, [node(m, Op.Mul, [a, a])]))
    m.fuse_matmul_bias()
    return m, (w1, b1, w2)


@pytest.mark.parametrize("act", ["Gelu", "ReLU"])
@pytest.mark.parametrize("algo", [D.GEMM_BF16X3, D.GEMM_FP32])
def test_activation_between_two_products(case, act, algo):
    """With the bf16 route the activation rides on the second product's operand split (no pass, no tensor); with
    the fp32 route it runs when the product asks for its operand.  Either way the bits are those of the separate
    operators."""
    case(f"{act} between two MatMuls, algorithm {algo}")
    m, (w1, b1, w2) = mlp((3, 50), 40, 72, getattr(Op, act))
    x = RNG.standard_normal((3, 50, 40)).astype(np.float32)
    outs = []
    for views in (True, False):
        sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(algo).with_strided_views(views).build()
        outs.append(np.array(sess.run([Tensor.from_numpy(x)])[0]))
        assert sess.copies_avoided() == (1 if views else 0)
        sess.close()
    assert_bits_equal(outs[0], outs[1], "folded vs separate")
    h = x.astype(np.float64) @ w1 + b1
    import math
    a = np.maximum(h, 0) if act == "ReLU" else 0.5 * h * (1 + np.vectorize(math.erf)(h / np.sqrt(2)))
    np.testing.assert_allclose(outs[0], a @ w2, rtol=2e-3, atol=2e-3)      # the reference's Gelu is the tanh form (fast_gelu)


def test_activation_with_a_second_reader_is_never_left_pending(case):
    """A Gelu that a MatMul and an element-wise operator both read cannot wait for the second product's operand split.
    On the fp32 kernel the product in front of it applies it (one node served per run); on the bf16 route it runs as
    its own kernel."""
    case("Gelu read by a MatMul and by an element-wise operator")
    m, _ = mlp((20,), 16, 24, Op.Gelu, second_reader=True)
    x = RNG.standard_normal((20, 16)).astype(np.float32)
    (y, z), avoided = run_both(m, [x])
    assert avoided == 1
    sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(D.GEMM_BF16X3).build()
    y2, z2 = (np.array(t) for t in sess.run([Tensor.from_numpy(x)]))
    assert sess.copies_avoided() == 0
    sess.close()
    np.testing.assert_allclose(y2, y, rtol=1e-5, atol=1e-5)  # the first product's sums are rounded in another order
    np.testing.assert_allclose(z2, z, rtol=1e-5, atol=1e-5)


def test_gemm_activated_through_the_c_abi(ctx, case):
    case("ahip_gemm_activated vs ahip_unary + ahip_gemm")
    m, k, n = 130, 70, 90
    a = RNG.standard_normal((m, k)).astype(np.float32)
    b = RNG.standard_normal((k, n)).astype(np.float32)
    da, db, dc = ctx.upload(a), ctx.upload(b), ctx.alloc(m * n * 4)
    try:
        ctx.gemm_set_algorithm(D.GEMM_FP32)
        with pytest.raises(AltiusHipError) as e:
            check(ctx.L.ahip_gemm_activated(ctx.handle, D.GELU, dc.ptr, da.ptr, db.ptr, None, m, n, k, 0, 0, k, n, n, 0, 0, 1.0, 0.0), ctx.handle)
        assert e.value.code == ERR_UNSUPPORTED
        ctx.gemm_set_algorithm(D.GEMM_BF16X3)
        for op in (D.GELU, D.RELU):
            check(ctx.L.ahip_gemm_activated(ctx.handle, op, dc.ptr, da.ptr, db.ptr, None, m, n, k, 0, 0, k, n, n, 0, 0, 1.0, 0.0), ctx.handle)
            got = ctx.download(dc, (m, n))
            assert_bits_equal(got, ctx.matmul(ctx.unary(op, a), b), f"op {op}")
    finally:
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)
        for x in (da, db, dc):
            ctx.free(x)


def transformer_mlp(rows, hidden, inner, residual_first):
    """x -> MatMul + bias -> Gelu -> MatMul + bias -> Add(x): the second half of a transformer block."""
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", list(rows) + [hidden])
    m.add_input(x)
    w1 = (RNG.standard_normal((hidden, inner)) * 0.2).astype(np.float32)
    w2 = (RNG.standard_normal((inner, hidden)) * 0.2).astype(np.float32)
    b1 = RNG.standard_normal(inner).astype(np.float32)
    b2 = RNG.standard_normal(hidden).astype(np.float32)
    h = node(m, Op.Add, [node(m, Op.MatMul, [x, m.new_initializer(w1)]), m.new_initializer(b1)])
    y = node(m, Op.Add, [node(m, Op.MatMul, [node(m, Op.Gelu, [h]), m.new_initializer(w2)]), m.new_initializer(b2)])
    m.add_output(node(m, Op.Add, [x, y] if residual_first else [y, x]))
    m.fuse_matmul_bias()
    return m


@pytest.mark.parametrize("rows,hidden,inner", [((197,), 768, 3072), ((3, 50), 40, 72), ((1,), 16, 8)])
@pytest.mark.parametrize("residual_first", [True, False])
def test_gelu_and_residual_add_ride_on_the_fp32_products(case, rows, hidden, inner, residual_first):
    """On the fp32 kernel the Gelu behind the first product and the residual Add behind the second are done while the
    products are written (the first shape through the k cut's finishing kernel): two nodes served without a kernel, and the
    bits of the separate operators."""
    case(f"MatMul -> Gelu -> MatMul -> Add(residual), rows {rows}, {hidden} -> {inner}")
    m = transformer_mlp(rows, hidden, inner, residual_first)
    x = RNG.standard_normal(tuple(rows) + (hidden,)).astype(np.float32)
    outs = []
    for views in (True, False):
        sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(D.GEMM_FP32).with_strided_views(views).build()
        for _ in range(2):
            got = np.array(sess.run([Tensor.from_numpy(x)])[0])
        assert sess.copies_avoided() == (2 if views else 0)  # the Gelu node and the Add node
        sess.close()
        outs.append(got)
    assert_bits_equal(outs[0], outs[1], "done by the products vs separate operators")


def test_residual_that_is_not_the_products_shape_stays_an_add(case):
    """Add(product, row vector) broadcasts: not a residual the product can absorb."""
    case("MatMul -> Add(broadcast operand)")
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [20, 16])
    r = m.new_val_named_and_shaped("r", [1, 24])
    m.add_input(x)
    m.add_input(r)
    w = (RNG.standard_normal((16, 24)) * 0.2).astype(np.float32)
    m.add_output(node(m, Op.Add, [node(m, Op.MatMul, [x, m.new_initializer(w)]), r]))
    xs = RNG.standard_normal((20, 16)).astype(np.float32)
    rs = RNG.standard_normal((1, 24)).astype(np.float32)
    (y,), avoided = run_both(m, [xs, rs])
    assert avoided == 0
    np.testing.assert_allclose(y, xs.astype(np.float64) @ w + rs, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("m,k,n", [(197, 768, 3072), (130, 70, 90), (300, 1024, 96), (1, 16, 5)])
def test_gemm_post_through_the_c_abi(ctx, case, m, k, n):
    case(f"ahip_gemm_post vs ahip_gemm + ahip_unary + ahip_binary, [{m},{k}]x[{k},{n}]")
    a = RNG.standard_normal((m, k)).astype(np.float32)
    b = (RNG.standard_normal((k, n)) * 0.1).astype(np.float32)
    bias = RNG.standard_normal(n).astype(np.float32)
    res = RNG.standard_normal((m, n)).astype(np.float32)
    da, db, dbias, dres, dc = ctx.upload(a), ctx.upload(b), ctx.upload(bias), ctx.upload(res), ctx.alloc(m * n * 4)
    try:
        ctx.gemm_set_algorithm(D.GEMM_FP32)
        plain = ctx.matmul(a, b) + bias     # the kernel's own 1 * acc + 1 * bias rounds like this Add
        for act in (0, D.GELU, D.RELU):
            for with_res in (False, True):
                check(ctx.L.ahip_gemm_post(ctx.handle, dc.ptr, da.ptr, db.ptr, dbias.ptr, m, n, k, 0, 0, k, n, n, 0, 1, 1.0, 1.0, act,
                                           dres.ptr if with_res else None), ctx.handle)
                want = plain if act == 0 else ctx.unary(act, plain)
                if with_res:
                    want = want + res
                assert_bits_equal(ctx.download(dc, (m, n)), want, f"act {act}, residual {with_res}")
        with pytest.raises(AltiusHipError) as e:
            check(ctx.L.ahip_gemm_post(ctx.handle, dc.ptr, da.ptr, db.ptr, None, m, n, k, 0, 0, k, n, n, 0, 0, 1.0, 0.0, D.SIGMOID, None), ctx.handle)
        assert e.value.code == ERR_ARG
    finally:
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)
        for x in (da, db, dbias, dres, dc):
            ctx.free(x)


# ---- MatMul -> Softmax -> MatMul as one kernel ----

def scaled_attention(batch, tq, tk, heads, d, scale_kind, extra_reader=False, mask=False):
    # mask: False, "keys" ([b, 1, 1, tk], one value per key and batch), "shared" ([tk]) or "queries" ([b, 1, tq, tk])
    """q [b, h, tq, d], k [b, h, tk, d], v [b, h, tk, d] as inputs; scores scaled by Mul / Div of a scalar (or not)."""
    m = Model(opset_version=13)
    q = m.new_val_named_and_shaped("q", [batch, heads, tq, d])
    k = m.new_val_named_and_shaped("k", [batch, heads, tk, d])
    v = m.new_val_named_and_shaped("v", [batch, heads, tk, d])
    for x in (q, k, v):
        m.add_input(x)
    s = node(m, Op.MatMul, [q, node(m, Op.Transpose, [k], perm=[0, 1, 3, 2])])
    if scale_kind == "mul":
        s = node(m, Op.Mul, [s, m.new_initializer(np.array(d ** -0.5, np.float32))])
    elif scale_kind == "div":
        s = node(m, Op.Div, [s, m.new_initializer(np.array(d ** 0.5, np.float32))])
    if mask:
        shape = {"keys": (batch, 1, 1, tk), "shared": (tk,), "queries": (batch, 1, tq, tk)}[mask]
        mk = np.where(RNG.random(shape) < 0.2, np.float32(-1e4), np.float32(0)).astype(np.float32)
        s = node(m, Op.Add, [s, m.new_initializer(mk)])
        m.mask_values = mk
    p = node(m, Op.Softmax, [s], axis=-1)
    m.add_output(node(m, Op.MatMul, [p, v]))
    if extra_reader:
        m.add_output(node(m, Op.ReduceMax, [p], axes=[1], keep_dims=False))
    m.fuse_softmax_prologue()
    m.fuse_transpose_matmul()
    return m


@pytest.mark.parametrize("scale_kind", [None, "mul", "div"])
@pytest.mark.parametrize("batch,tq,tk,heads", [(2, 197, 197, 3), (1, 40, 256, 2), (3, 5, 33, 1), (1, 70, 600, 2)])
def test_attention_triple_becomes_one_kernel(case, batch, tq, tk, heads, scale_kind):
    case(f"session attention b={batch} tq={tq} tk={tk} h={heads} scale={scale_kind}")
    m = scaled_attention(batch, tq, tk, heads, 64, scale_kind)
    q, k, v = (RNG.standard_normal((batch, heads, t, 64)).astype(np.float32) for t in (tq, tk, tk))
    (got,), avoided = run_both(m, [q, k, v], exact=False, attention=True)
    assert avoided == 2, avoided            # the first product and the Softmax
    s = q.astype(np.float64) @ k.astype(np.float64).transpose(0, 1, 3, 2)
    s = s * np.float32(64 ** -0.5) if scale_kind == "mul" else s / np.float32(8.0) if scale_kind == "div" else s
    e = np.exp(s - s.max(-1, keepdims=True))
    np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("mask", ["keys", "shared"])
def test_attention_with_a_per_key_mask(case, mask):
    """The padding mask of BERT-style graphs, absorbed by the Softmax and from there by the attention kernel."""
    case(f"session attention with a {mask} mask")
    batch, tq, tk, heads = 3, 37, 50, 2
    m = scaled_attention(batch, tq, tk, heads, 64, "div", mask=mask)
    q, k, v = (RNG.standard_normal((batch, heads, t, 64)).astype(np.float32) for t in (tq, tk, tk))
    (got,), avoided = run_both(m, [q, k, v], exact=False, attention=True)
    assert avoided == 2, avoided
    s = q.astype(np.float64) @ k.astype(np.float64).transpose(0, 1, 3, 2) / np.float32(8.0) + m.mask_values
    e = np.exp(s - s.max(-1, keepdims=True))
    np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("mask", [False, "keys"])
def test_attention_of_a_session_on_the_bf16_route(case, mask):
    """A session whose products may use the bf16 matrix cores (AHIP_GEMM_AUTO) and that has opted in to the one-kernel
    attention: with enough (batch, head) pairs for full blocks the kernel's two products take that route as well.
    Compared with the definition and with a default session (fp32 products, three operators)."""
    case(f"session attention on the bf16 route, mask {mask}")
    from altius_amd import device as D

    batch, tq, tk, heads = 24, 45, 70, 12
    m = scaled_attention(batch, tq, tk, heads, 64, "div", mask=mask)
    q, k, v = (RNG.standard_normal((batch, heads, t, 64)).astype(np.float32) for t in (tq, tk, tk))
    outs = []
    for fast in (True, False):
        b = HipSessionBuilder(m.clone())
        if fast:
            b = b.with_gemm_algorithm(D.GEMM_AUTO).with_fused_attention(True)
        sess = b.build()
        for _ in range(2):
            (got,) = [np.array(t) for t in sess.run([Tensor.from_numpy(x) for x in (q, k, v)])]
        if fast:
            assert sess.copies_avoided() == 2, sess.copies_avoided()
        sess.close()
        outs.append(got)
    s_ = q.astype(np.float64) @ k.astype(np.float64).transpose(0, 1, 3, 2) / np.float32(8.0)
    if mask:
        s_ = s_ + m.mask_values
    e = np.exp(s_ - s_.max(-1, keepdims=True))
    want = (e / e.sum(-1, keepdims=True)) @ v
    np.testing.assert_allclose(outs[0], want, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(outs[0], outs[1], rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("why", ["narrow heads", "second reader of the probabilities", "mask per query"])
def test_attention_triples_that_stay_three_operators(case, why):
    case(f"attention not fused: {why}")
    kw = dict(batch=2, tq=20, tk=40, heads=2, d=64, scale_kind="mul")
    if why == "narrow heads":
        kw["d"] = 32
    elif why == "second reader of the probabilities":
        kw["extra_reader"] = True
    else:
        kw["mask"] = "queries"    # found only when the Softmax runs: the deferred first product is computed after all
    m = scaled_attention(**kw)
    q, k, v = (RNG.standard_normal((kw["batch"], kw["heads"], t, kw["d"])).astype(np.float32) for t in (kw["tq"], kw["tk"], kw["tk"]))
    outs, avoided = run_both(m, [q, k, v], attention=True)          # bit for bit: nothing may have changed
    assert avoided == 0, avoided


# ---- LayerNormalization (with the residual Add in front) writing the next product's operand planes ----

def residual_norm_block(rows, hidden, n_out, with_add, sum_read_again, ln_second_reader=False):
    """x (+ r) -> LayerNormalization -> MatMul(weights) [+ bias]; optionally the sum is read again behind (the next
    residual connection of a transformer block), or the normalised tensor has a second reader."""
    m = Model(opset_version=17)
    shape = list(rows) + [hidden]
    x = m.new_val_named_and_shaped("x", shape)
    m.add_input(x)
    s = x
    if with_add:
        r = m.new_val_named_and_shaped("r", shape)
        m.add_input(r)
        s = node(m, Op.Add, [x, r])
    gamma = (1.0 + 0.1 * RNG.standard_normal(hidden)).astype(np.float32)
    beta = (0.1 * RNG.standard_normal(hidden)).astype(np.float32)
    w = (RNG.standard_normal((hidden, n_out)) * 0.1).astype(np.float32)
    b = RNG.standard_normal(n_out).astype(np.float32)
    y = node(m, Op.LayerNormalization, [s, m.new_initializer(gamma), m.new_initializer(beta)], axis=-1, epsilon=1e-5)
    p = node(m, Op.Add, [node(m, Op.MatMul, [y, m.new_initializer(w)]), m.new_initializer(b)])
    m.add_output(p)
    if sum_read_again:
        m.add_output(node(m, Op.Mul, [s, s]))
    if ln_second_reader:
        m.add_output(node(m, Op.Relu if hasattr(Op, "Relu") else Op.ReLU, [y]))
    m.fuse_matmul_bias()
    return m, (gamma, beta, w, b)


@pytest.mark.parametrize("rows,hidden", [((3, 50), 768), ((300,), 256), ((2, 17), 1024), ((40,), 512), ((5, 7), 128)])
@pytest.mark.parametrize("with_add,sum_read_again", [(False, False), (True, False), (True, True)])
def test_layernorm_writes_the_operand_planes_of_the_product_behind_it(case, rows, hidden, with_add, sum_read_again):
    """On the bf16 route a LayerNormalization whose only reader is a product with a weight matrix writes that
    product's operand planes instead of fp32 values, and the residual Add in front of it leaves its sum to the same
    kernel.  Every bit must be that of the separate operators (views off: Add, LayerNormalization, operand split)."""
    case(f"Add {with_add} -> LayerNormalization -> MatMul, rows {rows}, hidden {hidden}, sum read again {sum_read_again}")
    m, (gamma, beta, w, b) = residual_norm_block(rows, hidden, 96, with_add, sum_read_again)
    feeds = [RNG.standard_normal(list(rows) + [hidden]).astype(np.float32) for _ in range(2 if with_add else 1)]
    outs = []
    for views in (True, False):
        sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(D.GEMM_BF16X3).with_strided_views(views).build()
        for _ in range(2):
            got = [np.array(t) for t in sess.run([Tensor.from_numpy(x) for x in feeds])]
        outs.append(got)
        # rows of 128 have no wavefront-per-row layout: the separate kernels run; otherwise the operand split is
        # saved, and with it the Add's own pass
        fits = hidden != 128
        assert sess.copies_avoided() == ((1 + (1 if with_add else 0)) if views and fits else 0)
        sess.close()
    for a, c in zip(*outs):
        assert_bits_equal(a, c, "planes written by LayerNormalization vs separate operators")
    s = feeds[0].astype(np.float64) + (feeds[1] if with_add else 0)
    mu, var = s.mean(-1, keepdims=True), s.var(-1, keepdims=True)
    want = ((s - mu) / np.sqrt(var + 1e-5) * gamma + beta) @ w.astype(np.float64) + b
    np.testing.assert_allclose(outs[0][0], want, rtol=1e-4, atol=1e-4)
    if sum_read_again:
        np.testing.assert_allclose(outs[0][1], s * s, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("why", ["row length without a wavefront layout", "second reader of the normalised tensor", "fp32 route"])
def test_layernorm_planes_fall_back(case, why):
    case(f"LayerNormalization -> MatMul without planes: {why}")
    hidden = 200 if why.startswith("row length") else 256
    m, _ = residual_norm_block((30,), hidden, 64, True, True, ln_second_reader=why.startswith("second reader"))
    feeds = [RNG.standard_normal((30, hidden)).astype(np.float32) for _ in range(2)]
    algo = D.GEMM_FP32 if why == "fp32 route" else D.GEMM_BF16X3
    outs = []
    for views in (True, False):
        sess = HipSessionBuilder(m.clone()).with_gemm_algorithm(algo).with_strided_views(views).build()
        outs.append([np.array(t) for t in sess.run([Tensor.from_numpy(x) for x in feeds])])
        assert sess.copies_avoided() == 0
        sess.close()
    for a, c in zip(*outs):
        assert_bits_equal(a, c, why)
