"""Seeded sweeps over shapes nobody picked by hand: broadcast binary operators, row kernels at every
length class, reductions over every (outer, reduced, inner) geometry class, and fused chains, each
against the CPU oracle.  The seeds are fixed; a failure names the case that produced it."""
import numpy as np
import pytest

import oracle as O
from altius_amd import device as D
from altius_amd._lib import ERR_UNSUPPORTED, FUSED_ACC as ACC, AltiusHipError
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu

EXTENTS = [1, 1, 2, 3, 4, 5, 7, 8, 12, 16, 31, 33, 64, 100, 197]


def random_broadcast_pair(rng, max_elems=200_000):
    """Two shapes that broadcast together the way NumPy does it (right-aligned, 1 stretches)."""
    while True:
        rank = int(rng.integers(1, 6))
        out = [int(rng.choice(EXTENTS)) for _ in range(rank)]
        if np.prod(out) > max_elems:
            continue
        shapes = []
        for _ in range(2):
            r = int(rng.integers(0, rank + 1))
            s = out[rank - r:]
            shapes.append([d if rng.random() < 0.6 else 1 for d in s])
        # make sure every output extent is really present in one of the operands
        full = np.broadcast_shapes(tuple(shapes[0]), tuple(shapes[1]))
        return shapes[0], shapes[1], full


def test_binary_operators_on_random_broadcasts(case, ctx):
    rng = np.random.default_rng(2024)
    ops = [(D.ADD, O.ADD), (D.SUB, O.SUB), (D.MUL, O.MUL), (D.DIV, O.DIV)]
    for i in range(160):
        sa, sb, full = random_broadcast_pair(rng)
        a = rng.standard_normal(sa).astype(np.float32)
        b = (rng.standard_normal(sb) + 2.5).astype(np.float32)
        g, o = ops[i % 4]
        case(f"random binary #{i}: op {g} {sa} with {sb}")
        got = ctx.binary(g, a, b)
        assert got.shape == tuple(full)
        assert_bits_equal(got, O.binary(o, a, b), f"#{i} {sa} {sb}")


def test_binary_operators_on_the_patterns_with_kernels_of_their_own(case, ctx):
    """The broadcast patterns that models produce (a trailing vector, one value per row, one value per channel, one
    vector per outer index, either operand order), over extents on both sides of every kernel's conditions (rows that
    are and are not whole float4s, short and long rows), against NumPy's IEEE results bit for bit."""
    rng = np.random.default_rng(515)
    ops = [(D.ADD, np.add), (D.SUB, np.subtract), (D.MUL, np.multiply), (D.DIV, np.divide)]
    extents = [1, 2, 3, 4, 5, 7, 8, 12, 16, 33, 49, 64, 100, 197, 256, 516, 1028]
    for i in range(500):
        rank = int(rng.integers(2, 5))
        dims = [int(rng.choice(extents)) for _ in range(rank)]
        while np.prod(dims) > 1_500_000:
            dims[int(rng.integers(0, rank))] = 2
        kind = int(rng.integers(0, 4))
        small = list(dims)
        if kind == 0:
            small = dims[-1:]                                   # trailing vector
        elif kind == 1:
            small[-1] = 1                                       # one value per row
        elif kind == 2:
            j = int(rng.integers(0, rank - 1))
            small = [dims[j]] + [1] * (rank - 1 - j)            # one value per channel
        else:
            for ax in range(1, rank - 1):
                small[ax] = 1                                   # one vector per outer index
        x = rng.standard_normal(dims).astype(np.float32)
        y = (rng.standard_normal(small) + 3.0).astype(np.float32)
        if rng.random() < 0.3:
            x, y = y, x
        op, f = ops[int(rng.integers(0, 4))]
        case(f"pattern {i}: op {op} {list(x.shape)} {list(y.shape)}")
        assert_bits_equal(ctx.binary(op, x, y), f(x, y), f"case {i}: {list(x.shape)} op {list(y.shape)}")


def test_row_kernels_on_random_lengths(case, ctx):
    rng = np.random.default_rng(7)
    lengths = list(rng.integers(1, 1100, size=40)) + [255, 256, 257, 511, 512, 513, 767, 768, 1023, 1024, 1025, 1400, 2049]
    for i, n in enumerate(lengths):
        n = int(n)
        rows = int(rng.integers(1, 70))
        x = (rng.standard_normal((rows, n)) * 2).astype(np.float32)
        case(f"random rows #{i}: [{rows}, {n}]")
        assert_close(ctx.softmax(x), O.softmax(x), what=f"softmax [{rows},{n}]")
        g = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
        b = (0.1 * rng.standard_normal(n)).astype(np.float32)
        assert_close(ctx.layer_norm(x, g, b, 1e-5), O.layer_norm(x, g, b, 1e-5), what=f"layernorm [{rows},{n}]")
        if n <= 1024 and rows >= 2:
            mask = np.where(rng.random((1, n)) < 0.2, np.float32(-1e4), np.float32(0)).astype(np.float32)
            got = ctx.softmax_prologue(x, 2, np.float32(3.0), mask)
            z = O.binary(O.ADD, O.binary(O.DIV, x, np.array(3.0, np.float32)), mask)
            assert_bits_equal(got, ctx.softmax(z), f"softmax prologue [{rows},{n}] vs separate kernels")


def test_reductions_on_random_geometries(case, ctx):
    rng = np.random.default_rng(99)
    for i in range(90):
        outer = int(rng.choice([1, 2, 3, 7, 40, 300]))
        red = int(rng.choice([1, 2, 5, 17, 64, 197, 768, 1000, 5000]))
        inner = int(rng.choice([1, 1, 2, 3, 5, 8, 33, 64, 197, 255, 1023]))
        if outer * red * inner > 3_000_000:
            continue
        x = rng.standard_normal((outer, red, inner)).astype(np.float32)
        case(f"random reduce #{i}: [{outer}, {red}, {inner}]")
        got_max = ctx.reduce(D.REDUCE_MAX, x, outer, red, inner).reshape(outer, inner)
        assert_bits_equal(got_max, x.max(1), f"max [{outer},{red},{inner}]")
        got_mean = ctx.reduce(D.REDUCE_MEAN, x, outer, red, inner).reshape(outer, inner)
        np.testing.assert_allclose(got_mean, x.astype(np.float64).mean(1), rtol=1e-5, atol=2e-6,
                                   err_msg=f"mean [{outer},{red},{inner}]")


def test_fused_chains_on_random_broadcasts(case, ctx):
    """Random chains of 2..6 steps over 1..4 operands with random broadcast shapes, through whichever
    executor takes them, against the oracle's step-by-step result; geometry the kernel refuses must be
    refused as 'unsupported', never computed wrongly."""
    rng = np.random.default_rng(31337)
    unary = [D.SQRT, D.ERF, D.GELU, D.SIGMOID, D.RELU, D.TANH]
    binary = [D.ADD, D.SUB, D.MUL, D.DIV]
    ran = refused = 0
    for i in range(120):
        rank = int(rng.integers(1, 5))
        out = [int(rng.choice(EXTENTS)) for _ in range(rank)]
        if np.prod(out) > 100_000:
            continue
        n_in = int(rng.integers(1, 5))
        ins = [(rng.standard_normal(out) + 3.0).astype(np.float32)]          # the first operand has the full shape
        for _ in range(n_in - 1):
            r = int(rng.integers(0, rank + 1))
            s = [d if rng.random() < 0.5 else 1 for d in out[rank - r:]]
            ins.append((rng.standard_normal(s) + 3.0).astype(np.float32))
        steps = [("b", int(rng.choice(binary)), 0, int(rng.integers(0, n_in)))]
        for _ in range(int(rng.integers(1, 6))):
            if rng.random() < 0.4:
                steps.append(("u", int(rng.choice(unary)), ACC, 0))
            else:
                k = int(rng.integers(0, n_in))
                steps.append(("b", int(rng.choice(binary)), ACC, k) if rng.random() < 0.7 else ("b", int(rng.choice(binary)), k, ACC))
        case(f"random chain #{i}: out {out}, operands {[list(a.shape) for a in ins]}, steps {steps}")
        acc = None
        with np.errstate(all="ignore"):
            for kind, op, lhs, rhs in steps:
                a = acc if lhs == ACC else ins[lhs]
                acc = O.unary(op, a) if kind == "u" else O.binary(op, a, acc if rhs == ACC else ins[rhs])
        try:
            got = ctx.fused_elemwise(ins, steps)
        except AltiusHipError as e:
            assert e.code == ERR_UNSUPPORTED, e
            refused += 1
            continue
        ran += 1
        assert_bits_equal(got, np.broadcast_to(acc, got.shape), f"chain #{i}")
    assert ran > 60 and refused < ran
