"""The session on the GPU: graphs built the way the reference's tests build them
(crates/session_interpreter/tests/op_bin.rs:27-37), run through HipSessionBuilder / HipSession,
and compared with the CPU oracle applied node by node.  Covers every benchmark configuration at
reduced batch, the fused-vs-unfused comparisons, and the error paths."""
import numpy as np
import pytest

import oracle as O
from altius_amd import synth
from altius_amd._lib import ERR_ARG, ERR_OOM, ERR_SHAPE, ERR_UNSUPPORTED, AltiusHipError
from altius_amd.graph import F32, I64, Model, Op, Tensor, host_pool_stats, host_pool_trim
from altius_amd.graphs import erf_gelu_chain, layer_norm_chain
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu


def binary_model(op):
    """x, y -> op -> z with no declared shapes, exactly as op_bin.rs:27-37 builds it."""
    m = Model()
    x, y, z = m.new_val_named("x"), m.new_val_named("y"), m.new_val_named("z")
    m.add_node(op, [x, y], [z])
    m.add_input(x)
    m.add_input(y)
    m.add_output(z)
    return m


@pytest.mark.parametrize("shape", [[1, 2], [3, 1, 10], [16, 3, 224, 224]])
@pytest.mark.parametrize("name,op,fn", [("add", Op.Add, np.add), ("sub", Op.Sub, np.subtract),
                                        ("mul", Op.Mul, np.multiply), ("div", Op.Div, np.divide)])
def test_op_bin(case, name, op, fn, shape):
    """test_op_{add,sub,mul,div}_{1,2,3} (op_bin.rs:62-76); expected = x op y (op_bin.rs:41-46),
    tolerance 1e-5/1e-5 there, bit equality here."""
    case(f"session op_bin {name} {shape}")
    sess = HipSessionBuilder(binary_model(op)).build()
    x = synth.uniform(42, shape)
    y = synth.uniform(43, shape) + np.float32(1e-3)
    (z,) = sess.run([x, y])
    assert_bits_equal(z, fn(x, y), f"{name} {shape}")


def test_run_time_shape_inference_with_broadcast(case):
    """Inputs without declared shapes are inferred at run time (session.rs:149-158)."""
    case("session run-time shapes")
    sess = HipSessionBuilder(binary_model(Op.Mul)).build()
    for sa, sb in (([3, 15, 15], [15]), ([4, 1, 2], [3, 1]), ([2, 3], [])):
        a, b = synth.normal(1, sa), synth.normal(2, sb)
        (z,) = sess.run([a, b])
        assert_bits_equal(z, a * b, f"{sa}*{sb}")


def test_cfg0_bias_add(case):
    case("session cfg0")
    c = synth.cfg0()
    m = Model()
    a = m.new_val_named_and_shaped("a", c["a"].shape)
    b = m.new_initializer(c["b"], "bias")
    z = m.new_val_named("z")
    m.add_node(Op.Add, [a, b], [z])
    m.add_input(a)
    m.add_output(z)
    sess = HipSessionBuilder(m).build()
    (out,) = sess.run([c["a"]])
    assert_bits_equal(out, O.binary(O.ADD, c["a"], c["b"]), "cfg0")


def test_cfg1_softmax_and_layernorm(case):
    case("session cfg1")
    c = synth.cfg1(batch=2)
    m = Model()
    s = m.new_val_named_and_shaped("scores", c["scores"].shape)
    x = m.new_val_named_and_shaped("x", c["x"].shape)
    g = m.new_initializer(c["gamma"])
    b = m.new_initializer(c["beta"])
    p, y = m.new_val_named("p"), m.new_val_named("y")
    m.add_node(Op.Softmax, [s], [p], axis=-1)
    m.add_node(Op.LayerNormalization, [x, g, b], [y], axis=-1, epsilon=c["eps"])
    m.add_input(s)
    m.add_input(x)
    m.add_output(p)
    m.add_output(y)
    sess = HipSessionBuilder(m).with_profiling_enabled(True).build()
    p_out, y_out = sess.run([c["scores"], c["x"]])
    assert_close(p_out, O.softmax(c["scores"]), what="cfg1 softmax")
    assert_close(y_out, O.layer_norm(c["x"], c["gamma"], c["beta"], c["eps"]), what="cfg1 layernorm")
    prof = sess.profile()
    assert set(prof) == {"Softmax", "LayerNormalization"} and all(v > 0 for v in prof.values())
    assert sess.last_run_ms() > 0


def oracle_ln_chain(x, gamma, beta, eps):
    mean = O.reduce(O.REDUCE_MEAN, x, [-1], True)
    d = O.binary(O.SUB, x, mean)
    sq = O.binary(O.POW, d, np.array(2.0, np.float32))
    var = O.reduce(O.REDUCE_MEAN, sq, [-1], True)
    ve = O.binary(O.ADD, var, np.array(eps, np.float32))
    sd = O.unary(O.SQRT, ve)
    n = O.binary(O.DIV, d, sd)
    return O.binary(O.ADD, O.binary(O.MUL, n, gamma), beta)


def test_cfg2_unfused_chain_and_fused_layernorm(case):
    """The 9-node chain against the oracle's 9 steps, then the same model after fuse_layer_norm against
    the oracle's LayerNormalization; the two results agree to fp32 rounding of the two formulas."""
    case("session cfg2")
    c = synth.cfg2(batch=4)
    m = Model()
    x = m.new_val_named_and_shaped("x", c["x"].shape)
    out, _, _ = layer_norm_chain(m, x, c["gamma"], c["beta"], eps=float(c["eps"]))
    m.add_input(x)
    m.add_output(out)
    fused = m.clone()
    assert fused.fuse_layer_norm() == 1 and [n["op_name"] for n in fused.nodes()] == ["LayerNormalization"]

    sess = HipSessionBuilder(m).build()
    (unfused_out,) = sess.run([c["x"]])
    assert_close(unfused_out, oracle_ln_chain(c["x"], c["gamma"], c["beta"], c["eps"]), what="cfg2 chain")
    allocs = sess.device_allocations()
    (again,) = sess.run([c["x"]])
    assert_bits_equal(again, unfused_out, "second run")
    assert sess.device_allocations() == allocs        # steady state: the pool serves every buffer

    fsess = HipSessionBuilder(fused).build()
    (fused_out,) = fsess.run([c["x"]])
    assert_close(fused_out, O.layer_norm(c["x"], c["gamma"], c["beta"], float(c["eps"])), what="cfg2 fused")
    np.testing.assert_allclose(fused_out, unfused_out, rtol=1e-4, atol=1e-5)


def test_cfg3_gelu_unfused_and_fused(case):
    """Div -> Erf -> Add -> Mul -> Mul against the oracle's chain (approximate erf), and after fuse_gelu
    against the oracle's Gelu (tanh form): each path matches its own reference path."""
    case("session cfg3 gelu")
    c = synth.cfg3(batch=2)
    m = Model()
    x = m.new_val_named_and_shaped("x", c["x"].shape)
    out = erf_gelu_chain(m, x, sqrt2=float(c["sqrt2"]))
    m.add_input(x)
    m.add_output(out)
    fused = m.clone()
    assert fused.fuse_gelu() == 1

    (got,) = HipSessionBuilder(m).build().run([c["x"]])
    t = O.binary(O.DIV, c["x"], np.array(c["sqrt2"], np.float32))
    t = O.binary(O.ADD, O.unary(O.ERF, t), np.array(1.0, np.float32))
    want = O.binary(O.MUL, O.binary(O.MUL, c["x"], t), np.array(0.5, np.float32))
    assert_bits_equal(got, want, "cfg3 erf chain")

    (gf,) = HipSessionBuilder(fused).build().run([c["x"]])
    assert_bits_equal(gf, O.unary(O.GELU, c["x"]), "cfg3 fused gelu")
    assert np.max(np.abs(gf - got)) < 5e-2     # the two reference paths differ by the erf approximation


def test_cfg3_squeeze_excite(case):
    """ReduceMean over H,W -> HardSigmoid(1/6, 0.5) -> Mul back onto NCHW.  The reference interpreter
    has no kernel for the two-axis mean; the oracle computes it per the ONNX definition."""
    case("session cfg3 squeeze-excite")
    c = synth.cfg3(batch=4)
    m = Model()
    x = m.new_val_named_and_shaped("se", c["se"].shape)
    s, h, y = m.new_val(), m.new_val(), m.new_val_named("y")
    m.add_node(Op.ReduceMean, [x], [s], axes=[2, 3], keep_dims=True)
    m.add_node(Op.HardSigmoid, [s], [h], alpha=float(c["alpha"]), beta=float(c["beta"]))
    m.add_node(Op.Mul, [x, h], [y])
    m.add_input(x)
    m.add_output(y)
    (got,) = HipSessionBuilder(m).build().run([c["se"]])
    info = {}
    mean = O.reduce(O.REDUCE_MEAN, c["se"], [2, 3], True, info=info)
    assert info["no_reference_kernel"] and mean.shape == (4, 576, 1, 1)
    want = O.binary(O.MUL, c["se"], O.unary(O.HARDSIGMOID, mean, c["alpha"], c["beta"]))
    assert_close(got, want, what="cfg3 squeeze-excite")


def test_cfg4_pipeline(case):
    case("session cfg4")
    c = synth.cfg4(batch=4)
    m = Model()
    s = m.new_val_named_and_shaped("scores", c["scores"].shape)
    mask = m.new_val_named_and_shaped("mask", c["mask"].shape)
    r = m.new_val_named_and_shaped("r", c["rmax_in"].shape)
    d = m.new_val_named_and_shaped("d", c["div_in"].shape)
    k = m.new_initializer(np.array(c["div_scalar"], np.float32))
    z, p, mx, q = (m.new_val() for _ in range(4))
    m.add_node(Op.Add, [s, mask], [z])
    m.add_node(Op.Softmax, [z], [p], axis=-1)
    m.add_node(Op.ReduceMax, [r], [mx], axes=[1], keep_dims=False)
    m.add_node(Op.Div, [d, k], [q])
    for v in (s, mask, r, d):
        m.add_input(v)
    for v in (p, mx, q):
        m.add_output(v)
    p_out, mx_out, q_out = HipSessionBuilder(m).build().run([c["scores"], c["mask"], c["rmax_in"], c["div_in"]])
    assert_close(p_out, O.softmax(O.binary(O.ADD, c["scores"], c["mask"])), what="cfg4 softmax")
    assert mx_out.shape == (4, 197)
    assert_bits_equal(mx_out, O.reduce(O.REDUCE_MAX, c["rmax_in"], [1], False), "cfg4 reducemax")
    assert_bits_equal(q_out, O.binary(O.DIV, c["div_in"], np.array(c["div_scalar"], np.float32)), "cfg4 div")


def test_reference_reduce_kernels(case):
    """The two reductions the reference implements: ReduceMean(axis 2 of rank 3, keepdims) and
    ReduceMax(all axes, keepdims=0) (crates/altius_py/tests/test_ops_reduce.py:10-41)."""
    case("session reference reductions")
    x = synth.uniform(7, [1, 50, 70])
    for op, kind, kw, shape in ((Op.ReduceMean, O.REDUCE_MEAN, dict(axes=[-1], keep_dims=True), [1, 50, 1]),
                                (Op.ReduceMax, O.REDUCE_MAX, dict(axes=[], keep_dims=False), [1])):
        m = Model()
        a = m.new_val_named_and_shaped("x", x.shape)
        y = m.new_val_named("y")
        m.add_node(op, [a], [y], **kw)
        m.add_input(a)
        m.add_output(y)
        (got,) = HipSessionBuilder(m).build().run([x])
        info = {}
        want = O.reduce(kind, x, kw["axes"], kw["keep_dims"], strict=True, info=info)
        assert list(got.shape) == shape and not info["no_reference_kernel"]
        assert_close(got, want, what=f"reduce {op}")


def test_identity_and_sigmoid_sqrt_relu_tanh(case):
    case("session unary chain")
    x = synth.normal(9, [3, 1, 28, 28], std=2.0)
    m = Model()
    a = m.new_val_named_and_shaped("x", x.shape)
    v = [m.new_val() for _ in range(6)]
    m.add_node(Op.Identity, [a], [v[0]])
    m.add_node(Op.Sigmoid, [v[0]], [v[1]])
    m.add_node(Op.Sqrt, [v[1]], [v[2]])
    m.add_node(Op.Tanh, [v[2]], [v[3]])
    m.add_node(Op.ReLU, [a], [v[4]])
    m.add_node(Op.Identity, [v[4]], [v[5]])
    m.add_input(a)
    m.add_output(v[3])
    m.add_output(v[5])
    assert m.eliminate_identity() == 1   # the one feeding a graph output stays
    got1, got2 = HipSessionBuilder(m).build().run([x])
    assert_bits_equal(got1, O.unary(O.TANH, O.unary(O.SQRT, O.unary(O.SIGMOID, x))), "sigmoid-sqrt-tanh")
    assert_bits_equal(got2, O.unary(O.RELU, x), "relu-identity")


def test_errors_come_back_as_values(case):
    case("session errors")
    # an operator this backend has no kernel for: refused when the session is built
    m = Model()
    a = m.new_val_named_and_shaped("a", [2, 3])
    c = m.new_val()
    m.add_node(Op.NonMaxSuppression, [a, a], [c])
    m.add_input(a)
    m.add_output(c)
    with pytest.raises(AltiusHipError) as e:
        HipSessionBuilder(m).build()
    assert e.value.code == ERR_SHAPE and "NonMaxSuppression" in e.value.message

    # ... and at run time when shapes were not known at build time (session.rs:200)
    m = Model()
    a, c = m.new_val_named("a"), m.new_val()
    m.add_node(Op.NonMaxSuppression, [a, a], [c])
    m.add_input(a)
    m.add_output(c)
    sess = HipSessionBuilder(m).build()
    with pytest.raises(AltiusHipError) as e:
        sess.run([np.zeros([2, 3], np.float32)])
    assert "NonMaxSuppression" in e.value.message
    # shapes are fine but there is no kernel: SessionError::Message, as the reference reports it
    m = Model()
    a, c = m.new_val_named_and_shaped("a", [1, 1, 4, 4]), m.new_val()
    m.add_node(Op.ReduceMin, [a], [c], axes=[1])
    m.add_input(a)
    m.add_output(c)
    sess = HipSessionBuilder(m).build()
    with pytest.raises(AltiusHipError) as e:
        sess.run([np.zeros([1, 1, 4, 4], np.float32)])
    assert e.value.code == ERR_UNSUPPORTED and "ReduceMin: Kernel not implemented" in e.value.message   # session.rs:209-213

    sess = HipSessionBuilder(binary_model(Op.Add)).build()
    with pytest.raises(AltiusHipError) as e:   # shapes that do not broadcast (test_ops_bin.py:31-40)
        sess.run([np.zeros([1, 3, 28, 28], np.float32), np.zeros([3, 1, 2], np.float32)])
    assert e.value.code == ERR_SHAPE
    with pytest.raises(AltiusHipError) as e:   # too few inputs
        sess.run([np.zeros([2], np.float32)])
    assert e.value.code == ERR_ARG
    with pytest.raises(AltiusHipError) as e:   # the arithmetic kernels are f32; large integer tensors are refused ...
        sess.run([np.zeros([5000], np.int64), np.zeros([5000], np.int64)])
    assert e.value.code == ERR_UNSUPPORTED and "I64" in e.value.message
    (z,) = sess.run([np.array([1, 2], np.int64), np.array([10, -20], np.int64)])   # ... shape-sized ones are host arithmetic
    assert z.dtype == np.int64 and z.tolist() == [11, -18]
    # the session is still usable after errors
    (z,) = sess.run([np.ones([2], np.float32), np.ones([2], np.float32)])
    assert z.tolist() == [2.0, 2.0]

    # Softmax / LayerNormalization over an axis that is not the last (session.rs:999, 1444-1447)
    for op, extra in ((Op.Softmax, []), (Op.LayerNormalization, [np.ones(3, np.float32), np.ones(3, np.float32)])):
        m = Model()
        a = m.new_val_named_and_shaped("a", [2, 3, 4])
        ins = [a] + [m.new_initializer(t) for t in extra]
        c = m.new_val()
        m.add_node(op, ins, [c], axis=1)
        m.add_input(a)
        m.add_output(c)
        sess = HipSessionBuilder(m).build()
        with pytest.raises(AltiusHipError) as e:
            sess.run([np.zeros([2, 3, 4], np.float32)])
        assert e.value.code == ERR_UNSUPPORTED

    with pytest.raises(AltiusHipError):        # no such GPU
        HipSessionBuilder(binary_model(Op.Add)).with_device(99).build()


def test_graphs_that_make_no_sense_come_back_as_errors(case):
    """Tensors no device holds, values nobody produces, cycles: the reference unwraps and panics; here each is an
    error code, the process lives and the next session works."""
    case("session: nonsense graphs")
    one = np.ones(4, np.float32)

    def outcome(m, feeds):
        sess = HipSessionBuilder(m).build()
        try:
            sess.run(feeds)
        except AltiusHipError as e:
            return e.code
        finally:
            sess.close()
        return 0

    def start():
        m = Model()
        x = m.new_val_named_and_shaped("x", [4])
        m.add_input(x)
        return m, x

    m, x = start()  # an index range of 2^40 values
    lo, hi, step = (m.new_initializer(np.array(v, np.int64)) for v in (0, 1 << 40, 1))
    r = m.new_val()
    m.add_node(Op.Range, [lo, hi, step], [r])
    m.add_output(r)
    assert outcome(m, [one]) == ERR_OOM
    for extents in ([1 << 33, 1 << 33], [1 << 20, 1 << 20]):  # 2^66 elements (wraps to 4 in 64 bits) and 4 TB
        m = Model()
        x = m.new_val_named_and_shaped("x", [1])
        m.add_input(x)
        y = m.new_val()
        m.add_node(Op.Expand, [x, m.new_initializer(np.array(extents, np.int64))], [y])
        m.add_output(y)
        assert outcome(m, [np.ones(1, np.float32)]) == ERR_OOM
    m, x = start()  # a cycle
    y, z = m.new_val(), m.new_val()
    m.add_node(Op.ReLU, [z], [y])
    m.add_node(Op.Sqrt, [y], [z])
    m.add_output(z)
    assert outcome(m, [one]) == ERR_UNSUPPORTED
    m, x = start()  # a node that reads its own output
    y = m.new_val()
    m.add_node(Op.Add, [x, y], [y])
    m.add_output(y)
    assert outcome(m, [one]) == ERR_UNSUPPORTED
    m, x = start()  # a value nobody produces
    y, orphan = m.new_val(), m.new_val()
    m.add_node(Op.ReLU, [orphan], [y])
    m.add_output(y)
    assert outcome(m, [one]) == ERR_UNSUPPORTED
    m, x = start()  # nothing to compute: the input is the output, or there is no output
    m.add_output(x)
    sess = HipSessionBuilder(m).build()
    (got,) = sess.run([one])
    assert got.tolist() == one.tolist()
    m, x = start()
    assert HipSessionBuilder(m).build().run([one]) == []
    sess = HipSessionBuilder(binary_model(Op.Add)).build()
    (z,) = sess.run([one, one])
    assert z.tolist() == [2.0] * 4


def test_session_model_accessor_and_threads_option(case):
    case("session model()")
    m = binary_model(Op.Sub)
    sess = HipSessionBuilder(m).with_intra_op_num_threads(16).build()
    view = sess.model()
    assert [n["op_name"] for n in view.nodes()] == ["Sub"] and view.inputs == m.inputs
    (z,) = sess.run([np.full([5], 3, np.float32), np.full([5], 1, np.float32)])
    assert z.tolist() == [2.0] * 5


def test_io_tensors_live_in_recycled_pinned_memory(case):
    """Inputs made through the C ABI and outputs made by run() are pinned blocks from the pool;
    in steady state a run page-locks nothing new."""
    case("session pinned I/O")
    c = synth.cfg2(batch=2)
    x = c["x"]                                   # 1.2 MB
    m = Model()
    xin = m.new_val_named_and_shaped("x", x.shape)
    y = m.new_val()
    m.add_node(Op.LayerNormalization, [xin, m.new_initializer(c["gamma"]), m.new_initializer(c["beta"])], [y],
               axis=-1, epsilon=1e-5, stash_type=1)
    m.add_input(xin)
    m.add_output(y)
    sess = HipSessionBuilder(m).build()
    want = O.layer_norm(x, c["gamma"], c["beta"], 1e-5)
    host_pool_trim()
    base = host_pool_stats()
    t = Tensor.from_numpy(x)
    assert host_pool_stats()[0] > base[0] and host_pool_stats()[2] == base[2] + 1     # one page-locked block
    (out,) = sess.run([t], copy=False)
    assert_close(out, want, what="pinned run")
    assert host_pool_stats()[2] == base[2] + 2                                         # input + output
    del out
    for _ in range(3):
        (out,) = sess.run([t], copy=False)
        assert_close(out, want, what="pinned run, recycled output")
        del out
    st = host_pool_stats()
    assert st[2] == base[2] + 2 and st[3] >= base[3] + 3                               # nothing new, 3 reuses
    del t
    assert host_pool_stats()[0] == base[0]
    assert host_pool_trim() >= 2 * x.nbytes and host_pool_stats()[1] == 0
    (out,) = sess.run([x])                                                             # still works after a trim
    assert_close(out, want, what="after trim")


@pytest.mark.parametrize("shape,mask_shape,scale_kind", [
    ((4, 12, 197, 197), (4, 1, 1, 197), None),          # configs[4]: Add(mask) -> Softmax
    ((2, 12, 197, 197), (2, 1, 1, 197), "Div"),         # scores / sqrt(d) + mask
    ((2, 4, 17, 17), None, "Mul"),                      # the ViT test graph's scale only
    ((3, 2, 5, 2048), (3, 1, 1, 2048), "Mul"),          # rows too long for the one-kernel route: separate kernels, same result
    ((2, 3, 40, 512), (1, 1, 1, 512), "Div"),           # one mask row for everything
])
def test_softmax_with_absorbed_scale_and_mask(case, shape, mask_shape, scale_kind):
    """fuse_softmax_prologue: one Softmax node in place of [Mul|Div] -> [Add mask] -> Softmax, with the bits of
    the three nodes run one after the other."""
    case(f"session softmax prologue {shape} {mask_shape} {scale_kind}")
    m = Model()
    x = m.new_val_named_and_shaped("scores", list(shape))
    cur = x
    inputs = [synth.normal(61, list(shape))]
    if scale_kind:
        nxt = m.new_val()
        m.add_node(Op.Div if scale_kind == "Div" else Op.Mul, [cur, m.new_initializer(np.array(8.0 if scale_kind == "Div" else 0.125, np.float32))], [nxt])
        cur = nxt
    m.add_input(x)
    if mask_shape is not None:
        mv = m.new_val_named_and_shaped("mask", list(mask_shape))
        nxt = m.new_val()
        m.add_node(Op.Add, [cur, mv], [nxt])
        cur = nxt
        m.add_input(mv)
        inputs.append(synth.attention_mask(62, list(mask_shape), p_masked=0.2))
    p = m.new_val_named("p")
    m.add_node(Op.Softmax, [cur], [p], axis=-1)
    m.add_output(p)
    fused = m.clone()
    assert fused.fuse_softmax_prologue() == 1 and [n["op_name"] for n in fused.nodes()] == ["Softmax"]
    (want,) = HipSessionBuilder(m).build().run(inputs)
    (got,) = HipSessionBuilder(fused).build().run(inputs)
    assert_bits_equal(got, want, "one node vs three")
    z = inputs[0]
    if scale_kind:
        z = O.binary(O.DIV if scale_kind == "Div" else O.MUL, z, np.array(8.0 if scale_kind == "Div" else 0.125, np.float32))
    if mask_shape is not None:
        z = O.binary(O.ADD, z, inputs[1])
    assert_close(got, O.softmax(z), what="vs oracle chain")


def test_run_from_several_threads(case):
    """InterpreterSession::run takes &self and may be called from several threads at once (per-thread value maps,
    session.rs:52-58).  Here a session gives each of the calls that overlap a lane of its own (stream, buffer pool,
    initializers), and sessions of different threads run side by side as well; every call must return its own
    inputs' result."""
    import threading

    case("session: concurrent run() calls")
    c = synth.cfg2(batch=16)
    m = Model()
    x = m.new_val_named_and_shaped("x", c["x"].shape)
    out, _, _ = layer_norm_chain(m, x, c["gamma"], c["beta"], eps=float(c["eps"]))
    m.add_input(x)
    m.add_output(out)
    shared = HipSessionBuilder(m).build()
    inputs = [synth.normal(300 + i, c["x"].shape, std=1.0 + i) for i in range(4)]
    want = [oracle_ln_chain(v, c["gamma"], c["beta"], c["eps"]) for v in inputs]
    errors = []
    start = threading.Barrier(4)
    assert shared.lanes() == 1

    def worker(i, own_session):
        try:
            sess = HipSessionBuilder(m.clone()).build() if own_session else shared
            start.wait()
            for _ in range(8):
                (got,) = sess.run([inputs[i]])
                assert_close(got, want[i], what=f"thread {i}")
        except Exception as e:  # noqa: BLE001 - reported below, in the main thread
            errors.append((i, repr(e)))

    for own in (False, True):
        threads = [threading.Thread(target=worker, args=(i, own)) for i in range(4)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
    assert not errors, errors
    # 32 calls of a few milliseconds each, started together from four threads, overlapped at least once
    assert 2 <= shared.lanes() <= 4, shared.lanes()
    (alone,) = shared.run([inputs[0]])
    assert_close(alone, want[0], what="a call after the threads have gone")
    assert 2 <= shared.lanes() <= 4


# ---- what a session built with no switches returns -----------------------------------------------

def matmul_model(m_rows, k, n, w):
    """x [m, k] -> MatMul with a weight initializer [k, n]."""
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [m_rows, k])
    y = m.new_val_named("y")
    m.add_input(x)
    m.add_node(Op.MatMul, [x, m.new_initializer(w)], [y])
    m.add_output(y)
    return m


def test_default_session_gives_the_reference_result_for_infinite_operands(case):
    """compute_mat_mul (session.rs:621-684) is fp32 arithmetic: an infinite operand value gives +-inf in its
    row.  A session built with no switches must return exactly that, also at a size where AHIP_GEMM_AUTO
    would take the bf16 matrix cores; a session that opts in to AHIP_GEMM_BF16X3 or AHIP_GEMM_AUTO returns NaN
    for most of those rows (the documented difference: inf in the leading plane meets the lower planes of the
    other operand, inf * 0 or inf - inf), the reference's +-inf for the rest, and agrees everywhere else."""
    from altius_amd import device as D

    case("default session: MatMul with +-inf operands, 2048 x 1024 x 1024")
    rng = np.random.default_rng(11)
    rows, k, n = 2048, 1024, 1024      # 2^31 multiply-adds, whole 256 x 256 tiles: the AUTO rule picks bf16 x 3
    a = rng.standard_normal((rows, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.05).astype(np.float32)
    assert not (w == 0).any()
    a[3, 17] = np.inf
    a[700, 1000] = -np.inf
    a[2047, 0] = np.inf
    want = O.matmul(a, w)
    inf_rows = [3, 700, 2047]
    assert np.isinf(want[inf_rows]).all() and not np.isnan(want).any()
    assert np.array_equal(np.sign(want[3]), np.sign(w[17])) and np.array_equal(np.sign(want[700]), -np.sign(w[1000]))

    (got,) = HipSessionBuilder(matmul_model(rows, k, n, w)).build().run([a])
    finite = np.ones(rows, bool)
    finite[inf_rows] = False
    assert np.array_equal(got[inf_rows], want[inf_rows]), "the rows of the infinite operands"
    assert np.isfinite(got[finite]).all()
    np.testing.assert_allclose(got[finite], want[finite], rtol=1e-4, atol=1e-4)  # summation order only

    for algo in (D.GEMM_BF16X3, D.GEMM_AUTO):
        (fast,) = HipSessionBuilder(matmul_model(rows, k, n, w)).with_gemm_algorithm(algo).build().run([a])
        nan = np.isnan(fast[inf_rows])
        assert nan.mean() > 0.5, "bf16 x 3: inf in the leading plane against the other operand's lower planes"
        assert np.array_equal(fast[inf_rows][~nan], want[inf_rows][~nan]), "where it is not NaN it is the reference's infinity"
        assert np.isfinite(fast[finite]).all()
        np.testing.assert_allclose(fast[finite], want[finite], rtol=1e-4, atol=1e-4)


def test_default_session_runs_a_masked_attention_block_as_the_three_operators(case):
    """MatMul -> Div -> Add(mask) -> Softmax -> MatMul with 64-wide heads: a session built with no switches gives,
    bit for bit, what the session that copies everything and runs every operator on its own gives, and matches
    the oracle's three operators at the MatMul tolerance.  Opting in to the one-kernel attention changes the
    result by its documented 2e-4 relative and nothing more."""
    case("default session: masked attention block")
    rng = np.random.default_rng(12)
    b, h, tq, tk, d = 2, 3, 50, 70, 64
    q, k, v = (rng.standard_normal((b, h, t, d)).astype(np.float32) for t in (tq, tk, tk))
    mask = np.where(rng.random((b, 1, 1, tk)) < 0.2, np.float32(-1e4), np.float32(0)).astype(np.float32)

    def build():
        m = Model(opset_version=13)
        ins = [m.new_val_named_and_shaped(nm, list(x.shape)) for nm, x in (("q", q), ("k", k), ("v", v))]
        for i in ins:
            m.add_input(i)
        kt, s, s2, s3, p, o = (m.new_val() for _ in range(6))
        m.add_node(Op.Transpose, [ins[1]], [kt], perm=[0, 1, 3, 2])
        m.add_node(Op.MatMul, [ins[0], kt], [s])
        m.add_node(Op.Div, [s, m.new_initializer(np.array(8.0, np.float32))], [s2])
        m.add_node(Op.Add, [s2, m.new_initializer(mask)], [s3])
        m.add_node(Op.Softmax, [s3], [p], axis=-1)
        m.add_node(Op.MatMul, [p, ins[2]], [o])
        m.add_output(o)
        m.fuse_softmax_prologue()
        m.fuse_transpose_matmul()
        return m

    feeds = [q, k, v]
    (default,) = HipSessionBuilder(build()).build().run(feeds)
    (separate,) = HipSessionBuilder(build()).with_strided_views(False).build().run(feeds)
    assert_bits_equal(default, separate, "default session vs every operator on its own")

    s = O.binary(O.ADD, O.binary(O.DIV, O.matmul(q, np.ascontiguousarray(k.transpose(0, 1, 3, 2))), np.float32(8.0)), mask)
    want = O.matmul(O.softmax(s), v)
    assert_close(default, want, rtol=1e-4, atol=1e-5, what="default session vs the oracle's three operators")

    sess = HipSessionBuilder(build()).with_fused_attention().build()
    (fused,) = sess.run(feeds)
    assert sess.copies_avoided() == 2  # the first product and the Softmax went into the attention kernel
    assert not np.array_equal(fused, default)
    np.testing.assert_allclose(fused, default, rtol=2e-4, atol=2e-5)
