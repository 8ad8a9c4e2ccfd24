"""Data-movement kernels and the added element-wise ones, through the C ABI, against the CPU
oracle and numpy's own routines (bit equality: nothing here rounds except Cast, BatchNormalization,
LeakyRelu, Exp).  Shapes cover the transformer cases (head split/merge, K^T, qkv split, cls-token
concat, embedding gather), every element size, odd extents around the 64-wide tile, empty tensors."""
import numpy as np
import pytest

from altius_amd import device as D
from altius_amd._lib import AltiusHipError, ERR_ARG
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(11)


def rand(shape, dtype=np.float32):
    if dtype == np.bool_:
        return RNG.random(shape) > 0.5
    if np.issubdtype(dtype, np.integer):
        return RNG.integers(-1000, 1000, size=shape).astype(dtype)
    return RNG.standard_normal(shape).astype(dtype)


TRANSPOSES = [
    ((2, 197, 12, 64), (0, 2, 1, 3)),      # split heads: rows of 64 move whole (16-byte copies)
    ((2, 12, 197, 64), (0, 2, 1, 3)),      # merge heads
    ((2, 12, 197, 64), (0, 1, 3, 2)),      # K^T: tiled, 197 is not a multiple of the tile
    ((3, 197, 768), (1, 0, 2)),
    ((64, 64), (1, 0)), ((65, 63), (1, 0)), ((1, 129), (1, 0)), ((300, 7), (1, 0)),
    ((2, 3, 4, 5), (3, 2, 1, 0)), ((2, 3, 4, 5), (1, 3, 0, 2)), ((2, 3, 4, 5), (0, 1, 2, 3)),
    ((5, 1, 7, 1, 3), (4, 3, 2, 1, 0)), ((2, 3, 4, 5, 6, 2), (5, 0, 3, 1, 4, 2)),
    ((8, 3, 14, 14), (0, 2, 3, 1)),        # NCHW -> NHWC
    ((7,), (0,)), ((0, 5), (1, 0)), ((4, 0, 3), (2, 0, 1)),
    # both extents and pitches whole float4s: 16-byte accesses on both sides, tiles dealt diagonally
    ((256, 320), (1, 0)), ((3, 64, 28, 28), (0, 2, 3, 1)), ((3, 28, 28, 64), (0, 3, 1, 2)), ((68, 132), (1, 0)),
    ((5, 100, 72), (0, 2, 1)), ((100, 5, 72), (2, 1, 0)), ((24, 16, 20, 32), (3, 2, 1, 0)), ((1000, 16), (1, 0)),
    # dense transposed matrices too large for one block: panels of 64 columns where 64 rows of LDS hold the row axis, of 32
    # otherwise; odd and even row counts, either side of both limits
    ((3, 197, 768), (0, 2, 1)), ((2, 600, 112), (0, 2, 1)), ((1001, 64), (1, 0)), ((2, 3, 500, 96), (0, 1, 3, 2)), ((510, 160), (1, 0)),
    ((3, 100, 128), (0, 2, 1)), ((2, 255, 192), (0, 2, 1)), ((2, 257, 192), (0, 2, 1)), ((2, 511, 64), (0, 2, 1)),
    # 4-byte elements in 64 x 64 patches with 16-byte accesses wherever the rows start: odd extents on either side
    ((5000, 70), (1, 0)), ((70, 5000), (1, 0)), ((2001, 129), (1, 0)), ((3, 1029, 67), (0, 2, 1)), ((4099, 68), (1, 0)), ((3, 130, 5, 66), (0, 3, 2, 1)),
    # which side of a patch moves 16 bytes at a time: reads where rows start on 16-byte boundaries, writes only where they
    # start on 128-byte boundaries; more patches than the eight XCDs take in one turn, with and without a batch axis
    ((4096, 68), (1, 0)), ((3, 4096, 68), (0, 2, 1)), ((2052, 132), (1, 0)), ((2, 2052, 132), (0, 2, 1)), ((2052, 131), (1, 0)),
    ((2048, 131), (1, 0)), ((2, 1024, 67), (0, 2, 1)), ((1100, 1028), (1, 0)), ((1031, 1033), (1, 0)), ((9, 577, 129), (0, 2, 1)),
]


@pytest.mark.parametrize("shape,perm", TRANSPOSES)
@pytest.mark.parametrize("dtype", [np.float32, np.int64, np.bool_])
def test_transpose(ctx, oracle, case, shape, perm, dtype):
    case(f"transpose {shape} perm {perm} {np.dtype(dtype).name}")
    x = rand(shape, dtype)
    got = ctx.transpose(x, perm)
    assert_bits_equal(got, oracle.transpose(x, perm), "vs oracle")
    assert_bits_equal(got, np.ascontiguousarray(np.transpose(x, perm)), "vs numpy")


def test_slice_concat_split_expand_tile_as_strided_copies(ctx, oracle, case):
    case("strided copies")
    x = rand((4, 6, 10))
    st = x.strides
    es = lambda a: [s // a.itemsize for s in a.strides]
    # Slice x[1:3, :, 2:9:3]: dense output, input window with a step
    want = np.ascontiguousarray(x[1:3, :, 2:9:3])
    got = ctx.copy_strided(x, want.shape, es(want), [60, 10, 3], want.shape, in_offset=1 * 60 + 2)
    assert_bits_equal(got, want, "slice")
    # Concat on axis 1 of [2,3,4] and [2,5,4]: each input is written into its window of the output
    a, b = rand((2, 3, 4)), rand((2, 5, 4))
    out = np.zeros((2, 8, 4), np.float32)
    out = ctx.copy_strided(a, a.shape, [32, 4, 1], es(a), out.shape, out_init=out)
    out = ctx.copy_strided(b, b.shape, [32, 4, 1], es(b), out.shape, out_offset=3 * 4, out_init=out)
    assert_bits_equal(out, np.concatenate([a, b], axis=1), "concat")
    # Split of the last axis (qkv): three windows of the input
    qkv = rand((2, 197, 2304))
    parts = oracle.split(qkv, [768, 768, 768], 2, strict=True)
    for i, want in enumerate(parts):
        got = ctx.copy_strided(qkv, want.shape, es(want), es(qkv), want.shape, in_offset=768 * i)
        assert_bits_equal(got, want, f"split part {i}")
        assert_bits_equal(got, np.split(qkv, 3, axis=2)[i], "vs numpy")
    # Expand [3,1] -> [2,3,6] (stride 0) and Tile [2,3] x (2,2) as a rank-4 copy
    e = rand((3, 1))
    assert_bits_equal(ctx.copy_strided(e, (2, 3, 6), [18, 6, 1], [0, 1, 0], (2, 3, 6)), np.broadcast_to(e, (2, 3, 6)), "expand")
    t = rand((2, 3))
    got = ctx.copy_strided(t, (2, 2, 2, 3), [12, 6, 3, 1], [0, 3, 0, 1], (4, 6))
    assert_bits_equal(got, np.tile(t, (2, 2)), "tile")
    # int64 and bool elements
    for dt in (np.int64, np.bool_):
        v = rand((5, 9), dt)
        assert_bits_equal(ctx.copy_strided(v, (5, 4), [4, 1], [9, 2], (5, 4), in_offset=1), np.ascontiguousarray(v[:, 1:9:2]), "typed slice")
    # rank 0 and empty
    s = rand(())
    assert_bits_equal(ctx.copy_strided(s, (), [], [], ()), s, "scalar")
    assert ctx.copy_strided(rand((0, 3)), (0, 3), [3, 1], [3, 1], (0, 3)).shape == (0, 3)


def test_gather(ctx, oracle, case):
    case("gather")
    emb = rand((1000, 768))
    ids = RNG.integers(0, 1000, size=(1, 128)).astype(np.int64)
    assert_bits_equal(ctx.gather(emb, ids, 0), oracle.gather(emb, ids, 0, strict=True), "embedding lookup")
    d = rand((5, 6, 7))
    for axis, ix in [(0, [2, 2, 4]), (1, [[0, 5], [3, 3]]), (2, -1), (-2, [-6, 5]), (1, np.array([1, 0], np.int32))]:
        got = ctx.gather(d, np.asarray(ix), axis)
        assert_bits_equal(got, np.take(d, np.asarray(ix), axis=axis), f"axis {axis}")
        assert_bits_equal(got, oracle.gather(d, np.asarray(ix, np.int64), axis), "vs oracle")
    cls = rand((1, 197, 768))
    assert_bits_equal(ctx.gather(cls, np.array(0, np.int64), 1), cls[:, 0], "class token")
    for dt in (np.int64, np.bool_):
        v = rand((9, 4), dt)
        assert_bits_equal(ctx.gather(v, np.array([8, 0, 3]), 0), v[[8, 0, 3]], "typed")
    with pytest.raises(AltiusHipError) as e:
        ctx.gather(d, np.array([0, 6]), 1)                # index 6 on an axis of 6: reported at the next synchronisation
    assert e.value.code == ERR_ARG and "Gather" in e.value.message
    assert_bits_equal(ctx.gather(d, np.array([0, 5]), 1), d[:, [0, 5]], "the context works again afterwards")


def test_where_and_greater(ctx, oracle, case):
    case("where / greater")
    y = rand((2, 3, 5, 5))
    c = rand((2, 3, 5, 5), np.bool_)
    assert_bits_equal(ctx.where(c, np.float32(-1e9), y), oracle.where(c, np.float32(-1e9), y, strict=True), "pattern 1")
    c2 = rand((1, 1, 5, 5), np.bool_)
    assert_bits_equal(ctx.where(c2, y, np.float32(0.5)), oracle.where(c2, y, np.float32(0.5), strict=True), "pattern 2")
    c3 = rand((3, 1, 5), np.bool_)
    assert_bits_equal(ctx.where(c3, y, y[:, :1] * 2), np.where(c3, y, y[:, :1] * 2), "general broadcast")
    causal = np.tril(np.ones((1, 1, 64, 64), np.bool_))
    scores = rand((2, 12, 64, 64))
    assert_bits_equal(ctx.where(causal, scores, np.float32(-3.4e38)), np.where(causal, scores, np.float32(-3.4e38)), "causal mask")
    i = rand((4, 5), np.int64)
    assert_bits_equal(ctx.where(rand((4, 5), np.bool_) | True, i, i * 0), i, "int64")
    assert_bits_equal(ctx.greater(y, np.float32(0.1)), oracle.greater(y, np.float32(0.1), strict=True), "scalar rhs")
    assert_bits_equal(ctx.greater(y, y[:, :, :1]), y > y[:, :, :1], "broadcast rhs")
    assert not ctx.greater(np.array([np.nan, 1.0], np.float32), np.float32(np.nan)).any()


def test_cast(ctx, oracle, case):
    case("cast")
    specials = {
        np.float32: np.array([0.0, -0.0, 1e-30, np.nan, np.inf, -np.inf, 1.9, -1.9, 3e9, -3e9, 1e19, -1e19, 2147483520.0, 16777216.0],
                             np.float32),
        np.int32: np.array([0, 1, -1, 2**31 - 1, -2**31, 16777217], np.int32),
        np.int64: np.array([0, -1, 2**31, 2**32 + 5, -2**63, 2**63 - 1, 2**53 + 1, 16777217], np.int64),
        np.bool_: np.array([True, False]),
    }
    for src, x in specials.items():
        big = np.concatenate([x, rand(1000, src)])
        for dst in (np.float32, np.int32, np.int64, np.bool_):
            assert_bits_equal(ctx.cast(big, dst), oracle.cast(big, dst), f"{np.dtype(src).name} -> {np.dtype(dst).name}")


def test_batchnorm_leakyrelu_exp_round_clip_sum(ctx, oracle, case):
    case("batchnorm and element-wise additions")
    for shape in [(2, 3, 4, 5), (2, 16, 14, 14), (1, 5, 7, 7), (3, 8, 1, 1)]:
        x = rand(shape)
        c = shape[1]
        scale, bias, mean = rand(c), rand(c), rand(c)
        var = RNG.random(c).astype(np.float32) + np.float32(0.1)
        assert_bits_equal(ctx.batchnorm(x, scale, bias, mean, var, 1e-5), oracle.batchnorm(x, scale, bias, mean, var, 1e-5), f"batchnorm {shape}")
    z = np.concatenate([np.array([-2.0, -0.0, 0.0, 3.0, np.nan, -np.inf, np.inf], np.float32), rand(1001)])
    assert_bits_equal(ctx.unary(D.LEAKYRELU, z, 0.1), oracle.leaky_relu(z, 0.1), "leaky relu")
    assert_bits_equal(ctx.unary(D.LEAKYRELU, z, 0.01), oracle.leaky_relu(z, 0.01), "leaky relu default alpha")
    e = np.concatenate([np.array([0.0, -0.0, 1.0, -1.0, 88.0, 89.0, -104.0, np.nan, np.inf, -np.inf], np.float32), rand(1001) * 10])
    got = ctx.unary(D.EXP, e)
    want = np.exp(e.astype(np.float64))
    with np.errstate(over="ignore"):
        assert_close(got, want.astype(np.float32), rtol=2e-7, atol=1e-45, what="exp within 1 ulp of the exact value")
    assert got[0] == 1.0 and got[8] == np.inf and got[9] == 0.0 and np.isnan(got[7])
    r = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 2.4999, 2.5001, -0.0, 1e10, np.nan, np.inf], np.float32)
    assert_bits_equal(ctx.unary(D.ROUND, r), np.round(r), "round half to even")
    assert_bits_equal(ctx.unary(D.CLIP, z, -1.0, 2.0), np.where(np.isnan(z), z, np.clip(z, np.float32(-1.0), np.float32(2.0))), "clip")
    # plain sum (GlobalAveragePool's first half): small integers sum exactly in any order
    ints = RNG.integers(-8, 9, size=(6, 49)).astype(np.float32)
    assert_bits_equal(ctx.reduce(D.REDUCE_SUM, ints, 6, 49, 1).reshape(6), ints.sum(-1), "sum")
    p = rand((2, 3, 7, 7))
    gap = ctx.reduce(D.REDUCE_SUM, p, 6, 49, 1).reshape(2, 3, 1, 1) / np.float32(49)
    assert_close(gap, oracle.global_average_pool(p), what="global average pool")
