"""FusedElemwise on the GPU: a chain of element-wise operators in one kernel must give the bits of
the same operators applied one after the other -- by the CPU oracle where it has the function, and by
this backend's own stand-alone kernels (each pinned against the oracle in test_gpu_ops.py) for all of them."""
import numpy as np
import pytest

import oracle as O
from altius_amd import device as D
from altius_amd import synth
from altius_amd._lib import ERR_ARG, ERR_UNSUPPORTED, FUSED_ACC as ACC, AltiusHipError
from altius_amd.graph import Model, Op
from altius_amd.graphs import erf_gelu_chain, layer_norm_chain, single_input_model, squeeze_excite
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu


def chain_by_oracle(inputs, steps):
    """The steps one after the other on the CPU oracle (operators it implements only)."""
    acc = None
    for st in steps:
        kind, op, lhs, rhs = st[:4]
        a = acc if lhs == ACC else inputs[lhs]
        if kind == "u":
            alpha, beta = (list(st[4:6]) + [0.0, 0.0])[:2]
            acc = O.leaky_relu(a, alpha) if op == D.LEAKYRELU else O.unary(op, a, alpha, beta)
        else:
            acc = O.binary(op, a, acc if rhs == ACC else inputs[rhs])
    return acc


def chain_by_kernels(ctx, inputs, steps):
    """The steps one after the other through the stand-alone GPU kernels."""
    acc = None
    for st in steps:
        kind, op, lhs, rhs = st[:4]
        a = acc if lhs == ACC else inputs[lhs]
        if kind == "u":
            alpha, beta = (list(st[4:6]) + [0.0, 0.0])[:2]
            acc = ctx.unary(op, a, alpha, beta)
        else:
            acc = ctx.binary(op, a, acc if rhs == ACC else inputs[rhs])
    return acc


ERF_GELU = [("b", D.DIV, 0, 1), ("u", D.ERF, ACC, 0), ("b", D.ADD, ACC, 2), ("b", D.MUL, 0, ACC), ("b", D.MUL, ACC, 3)]


@pytest.mark.parametrize("shape", [(32, 197, 64), (5, 7, 12), (3, 50), (1001,), (4,), (1,), ()])
def test_erf_gelu_chain_one_kernel(case, ctx, shape):
    """Div -> Erf -> Add -> Mul x -> Mul 0.5 with x read twice: flat geometry, lengths that are and are not
    multiples of four, a single element."""
    case(f"fused erf-gelu {shape}")
    x = synth.normal(3, list(shape), std=1.5)
    ins = [x, np.array(1.4142135, np.float32), np.array(1.0, np.float32), np.array(0.5, np.float32)]
    got = ctx.fused_elemwise(ins, ERF_GELU)
    assert_bits_equal(got, chain_by_oracle(ins, ERF_GELU), f"vs oracle {shape}")
    assert_bits_equal(got, chain_by_kernels(ctx, ins, ERF_GELU), f"vs kernels {shape}")


@pytest.mark.parametrize("rows,cols", [(394, 768), (50, 36), (33, 197), (7, 5), (6, 1)])
def test_layernorm_tail_with_row_and_column_operands(case, ctx, rows, cols):
    """(var + eps) -> sqrt -> d / . -> * gamma -> + beta: one value per row ([rows,1]), a scalar, the dense
    tensor and two row vectors ([cols]) in one kernel; the square root is the divisor, i.e. the previous
    result as SECOND operand.  Column counts that are not multiples of four take the one-element kernel."""
    case(f"fused layernorm tail {rows}x{cols}")
    d = synth.normal(1, [rows, cols])
    var = np.abs(synth.normal(2, [rows, 1])) + np.float32(0.1)
    gamma, beta = synth.normal(3, [cols], mean=1.0, std=0.02), synth.normal(4, [cols], std=0.02)
    ins = [var, np.array(1e-5, np.float32), d, gamma, beta]
    steps = [("b", D.ADD, 0, 1), ("u", D.SQRT, ACC, 0), ("b", D.DIV, 2, ACC), ("b", D.MUL, ACC, 3), ("b", D.ADD, ACC, 4)]
    got = ctx.fused_elemwise(ins, steps)
    assert got.shape == (rows, cols)
    assert_bits_equal(got, chain_by_oracle(ins, steps), "vs oracle")


def test_attention_mask_and_scale(case, ctx):
    """scores / sqrt(d) + mask[N,1,1,C]: three merged axes [N, H*R, C]; C = 197 (one-element kernel) and
    C = 200 (four per lane with a broadcast middle axis)."""
    for c in (197, 200):
        case(f"fused scale+mask C={c}")
        scores = synth.normal(5, [3, 4, 9, c])
        mask = np.where(synth.uniform(6, [3, 1, 1, c]) < 0.1, np.float32(-1e4), np.float32(0))
        ins = [scores, np.array(8.0, np.float32), mask]
        steps = [("b", D.DIV, 0, 1), ("b", D.ADD, ACC, 2)]
        assert_bits_equal(ctx.fused_elemwise(ins, steps), chain_by_oracle(ins, steps), f"C={c}")


def test_every_step_code(case, ctx):
    """Each operator of the chain kernel against its stand-alone kernel, special values included; Pow
    takes a*a for a single exponent of 2 only when told so, powf otherwise."""
    case("fused: every step code")
    x = np.concatenate([synth.normal(7, [1000], std=3.0),
                        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-40, -1e-40, 88.0, -104.0, 1e30], np.float32)])
    x = x[:1008]
    for op, alpha, beta in ((D.SQRT, 0, 0), (D.ERF, 0, 0), (D.GELU, 0, 0), (D.SIGMOID, 0, 0), (D.HARDSIGMOID, 1 / 6, 0.5),
                            (D.RELU, 0, 0), (D.TANH, 0, 0), (D.LEAKYRELU, 0.01, 0), (D.EXP, 0, 0), (D.ROUND, 0, 0),
                            (D.CLIP, -1.0, 2.0)):
        steps = [("b", D.ADD, 0, 1), ("u", op, ACC, 0, alpha, beta)]
        ins = [x, np.array(0.0, np.float32)]
        assert_bits_equal(ctx.fused_elemwise(ins, steps), chain_by_kernels(ctx, ins, steps), f"unary code {op}")
    y = synth.normal(8, [1008], std=2.0)
    for op in (D.ADD, D.SUB, D.MUL, D.DIV, D.POW):
        steps = [("u", D.RELU, 0, 0), ("b", op, ACC, 1), ("b", op, 1, ACC)]
        assert_bits_equal(ctx.fused_elemwise([x, y], steps), chain_by_kernels(ctx, [x, y], steps), f"binary code {op}")
    two, three = np.array(2.0, np.float32), np.array(3.0, np.float32)
    sq = ctx.fused_elemwise([x, two], [("b", D.POW, 0, 1, 0.0, 0.0, 1)])
    assert_bits_equal(sq, x * x, "Pow(x, 2) on the scalar-exponent path is x*x")
    assert_bits_equal(sq, ctx.binary(D.POW, x, two), "as the stand-alone kernel does")
    assert_bits_equal(ctx.fused_elemwise([x, three], [("b", D.POW, 0, 1, 0.0, 0.0, 1)]), ctx.binary(D.POW, x, three), "powf otherwise")
    full_two = np.full_like(x, 2.0)
    assert_bits_equal(ctx.fused_elemwise([x, full_two], [("b", D.POW, 0, 1)]), ctx.binary(D.POW, x, full_two), "equal shapes: powf")


def test_compiled_chains_equal_the_interpreter(case, ctx):
    """The chains the library holds compiled code for, in the operand orders exporters produce (either order
    of a commutative step), through both executors and against the oracle."""
    case("fused: compiled chains vs interpreter")
    x = synth.normal(31, [64, 256], std=1.5)
    y = synth.normal(32, [64, 256])
    g, b = synth.normal(33, [256], mean=1.0, std=0.1), synth.normal(34, [256], std=0.1)
    var = np.abs(synth.normal(35, [64, 1])) + np.float32(0.1)
    c = lambda v: np.array(v, np.float32)
    cases = {
        "erf-gelu": ([x, c(1.4142135), c(1.0), c(0.5)], ERF_GELU),
        "erf-gelu, operands swapped": ([x, c(1.4142135), c(1.0), c(0.5)],
                                       [("b", D.DIV, 0, 1), ("u", D.ERF, ACC, 0), ("b", D.ADD, 2, ACC), ("b", D.MUL, ACC, 0), ("b", D.MUL, 3, ACC)]),
        "layernorm tail": ([var, c(1e-5), x, g, b],
                           [("b", D.ADD, 0, 1), ("u", D.SQRT, ACC, 0), ("b", D.DIV, 2, ACC), ("b", D.MUL, ACC, 3), ("b", D.ADD, ACC, 4)]),
        "normalise, scale, shift": ([x, var, g, b], [("b", D.DIV, 0, 1), ("b", D.MUL, ACC, 2), ("b", D.ADD, 3, ACC)]),
        "mul add": ([x, g, y], [("b", D.MUL, 0, 1), ("b", D.ADD, ACC, 2)]),
        "add relu": ([x, b], [("b", D.ADD, 0, 1), ("u", D.RELU, ACC, 0)]),
        "add gelu": ([x, b], [("b", D.ADD, 0, 1), ("u", D.GELU, ACC, 0)]),
        "add add": ([x, b, y], [("b", D.ADD, 0, 1), ("b", D.ADD, 2, ACC)]),
        "silu": ([x], [("u", D.SIGMOID, 0, 0), ("b", D.MUL, 0, ACC)]),
        "hard swish": ([x], [("u", D.HARDSIGMOID, 0, 0, 1 / 6, 0.5), ("b", D.MUL, ACC, 0)]),
    }
    try:
        for name, (ins, steps) in cases.items():
            ctx.fused_use_compiled_chains(True)
            compiled = ctx.fused_elemwise(ins, steps)
            ctx.fused_use_compiled_chains(False)
            interpreted = ctx.fused_elemwise(ins, steps)
            assert_bits_equal(compiled, interpreted, f"{name}: compiled vs interpreted")
            assert_bits_equal(compiled, chain_by_oracle(ins, steps), f"{name}: vs oracle")
    finally:
        ctx.fused_use_compiled_chains(True)


def test_unaligned_and_six_operands(case, ctx):
    case("fused: six operands, both operands the previous result")
    ins = [synth.normal(20 + k, [64, 40]) for k in range(6)]
    steps = [("b", D.ADD, 0, 1), ("b", D.MUL, ACC, ACC), ("b", D.SUB, ACC, 2), ("b", D.MUL, 3, ACC), ("b", D.ADD, ACC, 4),
             ("b", D.SUB, 5, ACC), ("u", D.TANH, ACC, 0)]
    assert_bits_equal(ctx.fused_elemwise(ins, steps), chain_by_oracle(ins, steps), "six operands")


def test_refusals(case, ctx):
    case("fused: refusals")
    x = synth.normal(1, [8])
    with pytest.raises(AltiusHipError) as e:                 # the first step has no previous result
        ctx.fused_elemwise([x], [("u", D.RELU, ACC, 0)])
    assert e.value.code == ERR_ARG
    with pytest.raises(AltiusHipError) as e:
        ctx.fused_elemwise([x], [("b", D.ADD, 0, 3)])
    assert e.value.code == ERR_ARG
    with pytest.raises(AltiusHipError) as e:
        ctx.fused_elemwise([x] * 7, [("b", D.ADD, 0, 6)])
    assert e.value.code == ERR_UNSUPPORTED
    with pytest.raises(AltiusHipError) as e:
        ctx.fused_elemwise([x], [("u", D.RELU, 0, 0)] * 17)
    assert e.value.code == ERR_UNSUPPORTED
    a, b = synth.normal(2, [2, 1, 3, 1, 2]), synth.normal(3, [1, 4, 1, 5, 1])
    with pytest.raises(AltiusHipError) as e:                 # five axes that do not merge
        ctx.fused_elemwise([a, b], [("b", D.ADD, 0, 1)])
    assert e.value.code == ERR_UNSUPPORTED
    assert ctx.fused_elemwise([np.zeros([0, 4], np.float32)], [("u", D.RELU, 0, 0)]).shape == (0, 4)


# ---- through the session ------------------------------------------------------------------------

def run_both(model, x, extended=True):
    """The model node by node, and after fuse_elemwise_ops; returns (unfused, fused, fused model)."""
    fused = model.clone()
    n = fused.fuse_elemwise_ops(extended=extended)
    (want,) = HipSessionBuilder(model).build().run([x])
    (got,) = HipSessionBuilder(fused).build().run([x])
    return want, got, fused, n


def test_session_erf_gelu_chain(case):
    case("session: erf-GELU chain as one FusedElemwise")
    c = synth.cfg3(batch=2)
    m = single_input_model(c["x"].shape, lambda m, x: erf_gelu_chain(m, x, float(c["sqrt2"])))
    want, got, fused, n = run_both(m, c["x"])
    assert n == 1 and [k["op_name"] for k in fused.nodes()] == ["FusedElemwise"]
    assert_bits_equal(got, want, "fused vs node by node")
    t = O.binary(O.DIV, c["x"], np.array(c["sqrt2"], np.float32))
    t = O.binary(O.ADD, O.unary(O.ERF, t), np.array(1.0, np.float32))
    assert_bits_equal(got, O.binary(O.MUL, O.binary(O.MUL, c["x"], t), np.array(0.5, np.float32)), "fused vs oracle chain")


@pytest.mark.parametrize("extended", [False, True])
def test_session_layernorm_chain(case, extended):
    case(f"session: LayerNorm chain, elementwise fusion (extended={extended})")
    c = synth.cfg2(batch=3)
    m = single_input_model(c["x"].shape, lambda m, x: layer_norm_chain(m, x, c["gamma"], c["beta"], float(c["eps"]))[0])
    want, got, fused, n = run_both(m, c["x"], extended)
    assert n == (1 if extended else 2)
    assert len(fused.nodes()) == (5 if extended else 7)
    assert_bits_equal(got, want, "fused vs node by node")


def test_session_squeeze_excite_and_fallback_route(case):
    """HardSigmoid -> Mul onto [N,C,7,7] (49 columns: the one-element kernel), and a chain whose operands
    need five axes: the session runs it operator by operator with the same result."""
    case("session: squeeze-excite fused; chain that falls back")
    c = synth.cfg3(batch=2)
    m = single_input_model(c["se"].shape, lambda m, x: squeeze_excite(m, x, c["alpha"], c["beta"]))
    want, got, fused, n = run_both(m, c["se"])
    assert n == 1 and [k["op_name"] for k in fused.nodes()] == ["ReduceMean", "FusedElemwise"]
    assert_bits_equal(got, want, "squeeze-excite")

    a, b = synth.normal(2, [2, 1, 3, 1, 2]), synth.normal(3, [1, 4, 1, 5, 1])
    m = Model()
    va = m.new_val_named_and_shaped("a", a.shape)
    t1, t2 = m.new_val(), m.new_val()
    m.add_node(Op.Mul, [va, m.new_initializer(b)], [t1])
    m.add_node(Op.Sigmoid, [t1], [t2])
    m.add_input(va)
    m.add_output(t2)
    want, got, fused, n = run_both(m, a)
    assert n == 1 and got.shape == (2, 4, 3, 5, 2)
    assert_bits_equal(got, want, "fallback route")
    assert_bits_equal(got, O.unary(O.SIGMOID, a * b), "fallback route vs oracle")


def test_session_pow_paths_inside_a_chain(case):
    """Pow with a one-element exponent of 2 inside a chain is x*x, as in the unfused kernel, under either rule
    (the reference's rule fuses Sub -> Pow here because both second operands are scalars, and leaves the Mul)."""
    case("session: Pow inside chains")
    x = synth.normal(11, [6, 40], std=2.0)
    m = Model()
    vx = m.new_val_named_and_shaped("x", x.shape)
    t1, t2, t3 = m.new_val(), m.new_val(), m.new_val()
    m.add_node(Op.Sub, [vx, m.new_initializer(np.array(0.25, np.float32))], [t1])
    m.add_node(Op.Pow, [t1, m.new_initializer(np.array(2.0, np.float32))], [t2])
    m.add_node(Op.Mul, [t2, m.new_initializer(synth.normal(12, [40]))], [t3])
    m.add_input(vx)
    m.add_output(t3)
    want, got, fused, n = run_both(m, x)
    assert n == 1 and len(fused.nodes()) == 1
    assert_bits_equal(got, want, "extended rule")
    d = x - np.float32(0.25)
    assert_bits_equal(got, (d * d) * synth.normal(12, [40]), "x*x, not powf")
    want, got, fused, n = run_both(m, x, extended=False)      # Sub -> Pow fuse (both second operands are scalars), Mul stays
    assert n == 1 and [k["op_name"] for k in fused.nodes()] == ["FusedElemwise", "Mul"]
    assert_bits_equal(got, want, "reference rule")
