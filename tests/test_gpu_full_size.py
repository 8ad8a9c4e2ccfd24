"""Parity at the benchmark's full sizes (BASELINE.json configs[4], batch 256; configs[2]/[3] at
batch 32), through the oracle where it finishes in seconds with its thread pool and through
size-independent properties: IEEE closed forms for the exact ops, rows summing to one, idempotence
of max, linearity of the mean, invariance of LayerNormalization under shifts."""
import os

import numpy as np
import pytest

import oracle as O
from altius_amd import device as D
from altius_amd import synth
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu

THREADS = min(16, os.cpu_count() or 1)


@pytest.fixture(scope="module")
def cfg4():
    return synth.cfg4(batch=256)


def test_cfg4_masked_add_then_softmax(ctx, case, cfg4):
    case("full cfg4 Add+Softmax [256,12,197,197]")
    scores, mask = cfg4["scores"], cfg4["mask"]
    z = ctx.binary(D.ADD, scores, mask)
    assert_bits_equal(z, scores + mask, "cfg4 add")                    # IEEE closed form, numpy broadcasting
    p = ctx.softmax(z)
    assert_close(p, O.softmax(z, threads=THREADS), what="cfg4 softmax")
    sums = p.reshape(-1, 197).sum(-1, dtype=np.float64)
    assert np.max(np.abs(sums - 1.0)) < 2e-6                            # every one of the 605 184 rows
    masked = np.broadcast_to(mask, z.shape) != 0
    assert np.all(p[masked] < 1e-30) and np.all(p >= 0)
    # Softmax commutes with permuting a row: reversed rows give reversed results (sum order aside).
    rows = np.ascontiguousarray(z.reshape(-1, 197)[:4096, ::-1])
    assert_close(ctx.softmax(rows)[:, ::-1], p.reshape(-1, 197)[:4096], what="softmax of reversed rows")


def test_cfg4_reduce_max_axis1(ctx, case, cfg4):
    case("full cfg4 ReduceMax [256,768,197]")
    x = cfg4["rmax_in"]
    m = ctx.reduce(D.REDUCE_MAX, x, 256, 768, 197)
    assert_bits_equal(m, x.max(1), "cfg4 reducemax")                    # order-independent, exact
    assert_bits_equal(m, O.reduce(O.REDUCE_MAX, x, [1], False), "cfg4 reducemax vs oracle")
    # idempotence: the maximum of maxima over a split of the axis is the maximum
    halves = np.maximum(ctx.reduce(D.REDUCE_MAX, np.ascontiguousarray(x[:, :384]), 256, 384, 197),
                        ctx.reduce(D.REDUCE_MAX, np.ascontiguousarray(x[:, 384:]), 256, 384, 197))
    assert_bits_equal(halves, m, "max of maxima")


def test_cfg4_div_scalar(ctx, case, cfg4):
    case("full cfg4 Div [256,197,768]")
    x, s = cfg4["div_in"], np.array(cfg4["div_scalar"], np.float32)
    q = ctx.binary(D.DIV, x, s)
    assert_bits_equal(q, x / s, "cfg4 div")
    assert_bits_equal(q, O.binary(O.DIV, x, s), "cfg4 div vs oracle")


def test_cfg4_sized_layernorm_chain_ops(ctx, case, cfg4):
    """The operators of the LayerNormalization chain on [256,197,768] (155 MB, so the kernels take their
    non-temporal variants): per-row Sub and Div, Mul by a vector, ReduceMean, LayerNormalization."""
    case("full-size chain operators on [256,197,768]")
    x = cfg4["div_in"]
    rows = x.shape[0] * x.shape[1]
    mean = ctx.reduce(D.REDUCE_MEAN, x, rows, 768, 1).reshape(256, 197, 1)
    assert_close(mean, O.reduce(O.REDUCE_MEAN, x, [-1], True), what="mean over 768")
    # exact in any order: mean(-x) = -mean(x)
    assert_bits_equal(ctx.reduce(D.REDUCE_MEAN, -x, rows, 768, 1).reshape(mean.shape), -mean, "mean(-x) = -mean(x)")
    assert_bits_equal(ctx.binary(D.SUB, x, mean), x - mean, "x - mean")
    assert_bits_equal(ctx.binary(D.SUB, mean, x), mean - x, "mean - x")
    dev = np.abs(mean) + np.float32(0.75)
    assert_bits_equal(ctx.binary(D.DIV, x, dev), x / dev, "x / dev")
    gamma = synth.normal(5, (768,), mean=1.0, std=0.02)
    beta = synth.normal(6, (768,), mean=0.0, std=0.02)
    assert_bits_equal(ctx.binary(D.MUL, x, gamma), x * gamma, "x * gamma")
    assert_bits_equal(ctx.binary(D.ADD, beta, x), beta + x, "beta + x")
    y = ctx.layer_norm(x, gamma, beta, 1e-5)
    assert_close(y, O.layer_norm(x, gamma, beta, 1e-5, threads=THREADS), what="layernorm [256,197,768]")
    p = ctx.softmax(x)
    assert_close(p, O.softmax(x, threads=THREADS), what="softmax [256,197,768]")
    np.testing.assert_allclose(p.sum(-1, dtype=np.float64), 1.0, atol=2e-6)


def test_cfg2_layernorm_full(ctx, case):
    case("full cfg2 LayerNormalization [32,197,768]")
    c = synth.cfg2(batch=32)
    y = ctx.layer_norm(c["x"], c["gamma"], c["beta"], 1e-5)
    assert_close(y, O.layer_norm(c["x"], c["gamma"], c["beta"], 1e-5, threads=THREADS), what="cfg2 layernorm")
    # normalised rows: (y - beta) / gamma has mean 0 and variance 1 - eps/(var+eps)
    n = (y.astype(np.float64) - c["beta"]) / c["gamma"]
    assert np.max(np.abs(n.mean(-1))) < 1e-5
    assert np.max(np.abs(n.var(-1) - 1.0)) < 1e-3
    # shifting a row by a constant that is exact in fp32 leaves LayerNormalization unchanged up to rounding
    shifted = ctx.layer_norm(c["x"][:2] + np.float32(4.0), c["gamma"], c["beta"], 1e-5)
    np.testing.assert_allclose(shifted, y[:2], rtol=0, atol=2e-5)


def test_cfg3_gelu_and_mean_full(ctx, case):
    case("full cfg3 Gelu [32,197,3072] and ReduceMean [32,576,7,7]")
    c = synth.cfg3(batch=32)
    g = ctx.unary(D.GELU, c["x"])
    assert_bits_equal(g, O.unary(O.GELU, c["x"], threads=THREADS), "cfg3 gelu")
    se = c["se"]
    mean = ctx.reduce(D.REDUCE_MEAN, se, 32 * 576, 49, 1).reshape(32, 576, 1, 1)
    assert_close(mean, O.reduce(O.REDUCE_MEAN, se, [2, 3], True), what="cfg3 mean")
    # linearity: mean(2x) == 2 mean(x) exactly (scaling by 2 is exact), mean(x) + mean(-x) == 0
    twice = ctx.reduce(D.REDUCE_MEAN, se * np.float32(2), 32 * 576, 49, 1).reshape(mean.shape)
    assert_bits_equal(twice, mean * np.float32(2), "mean(2x) = 2 mean(x)")
    neg = ctx.reduce(D.REDUCE_MEAN, -se, 32 * 576, 49, 1).reshape(mean.shape)
    assert_bits_equal(neg, -mean, "mean(-x) = -mean(x)")


def test_cfg4_masked_softmax_in_one_kernel(ctx, case, cfg4):
    """Add(mask) + Softmax fused at the full configs[4] size: the bits of the two kernels, on all 605 184 rows."""
    case("full cfg4 Add(mask)+Softmax in one kernel [256,12,197,197]")
    scores, mask = cfg4["scores"], cfg4["mask"]
    fused = ctx.softmax_prologue(scores, 0, 1.0, mask)
    assert_bits_equal(fused, ctx.softmax(ctx.binary(D.ADD, scores, mask)), "fused vs Add then Softmax")


def test_cfg3_erf_gelu_chain_in_one_kernel(ctx, case):
    """The 5-node erf-GELU chain as one FusedElemwise kernel at the full configs[3] size, against the oracle's chain."""
    from altius_amd._lib import FUSED_ACC as ACC

    case("full cfg3 erf-GELU chain in one kernel [32,197,3072]")
    c = synth.cfg3(batch=32)
    x = c["x"]
    s = lambda v: np.array(v, np.float32)
    steps = [("b", D.DIV, 0, 1), ("u", D.ERF, ACC, 0), ("b", D.ADD, ACC, 2), ("b", D.MUL, 0, ACC), ("b", D.MUL, ACC, 3)]
    got = ctx.fused_elemwise([x, s(c["sqrt2"]), s(1.0), s(0.5)], steps)
    t = O.binary(O.ADD, O.unary(O.ERF, O.binary(O.DIV, x, s(c["sqrt2"]), threads=THREADS), threads=THREADS), s(1.0), threads=THREADS)
    assert_bits_equal(got, O.binary(O.MUL, O.binary(O.MUL, x, t, threads=THREADS), s(0.5), threads=THREADS), "fused chain vs oracle chain")
