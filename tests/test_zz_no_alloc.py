"""ahip_reduce_static: the reduction entry point that allocates nothing (partial results in a fixed array of
the library's code object) against ahip_reduce, through the C ABI.  Same kernels and launch shapes, so the bar
is bit equality; both are also held to the oracle.  Collected last on purpose (file name)."""
import numpy as np
import pytest

from altius_amd import device as D
from altius_amd import synth
from altius_amd._lib import ERR_UNSUPPORTED, AltiusHipError, lib
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu


def both(ctx, kind, x, outer, red, inner):
    """(ahip_reduce, ahip_reduce_static) on the same device input, outputs pre-filled with a sentinel."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    dx = ctx.upload(x)
    sentinel = np.full(outer * inner, -12345.0, np.float32)
    d0, d1 = ctx.upload(sentinel), ctx.upload(sentinel)
    try:
        ctx.reduce_raw(kind, d0.ptr, dx.ptr, outer, red, inner)
        ctx.reduce_static_raw(kind, d1.ptr, dx.ptr, outer, red, inner)
        return ctx.download(d0, (outer, inner)), ctx.download(d1, (outer, inner))
    finally:
        for b in (dx, d0, d1):
            ctx.free(b)


# (outer, red, inner): every route that stages partial results -- long rows split over blocks, the span
# variant of the column reduction split over blocks, the general column reduction split over blocks --
# each followed by a SMALLER input of the same route, so the second call finds the first one's leftovers
# in the array, and by shapes that use no partial results at all.
PAIRS = [
    ((1, 3_000_000, 1), (1, 1_000_000, 1)),
    ((3, 400_000, 1), (2, 70_000, 1)),
    ((4, 768, 197), (2, 384, 197)),
    ((2, 4096, 200), (1, 2048, 72)),
    ((256, 768, 1), (7, 49, 1)),
]


@pytest.mark.parametrize("kind", [D.REDUCE_MAX, D.REDUCE_MEAN, D.REDUCE_SUM])
@pytest.mark.parametrize("first,second", PAIRS)
def test_reduce_static_matches_reduce_on_two_calls_in_a_row(ctx, oracle, case, kind, first, second):
    for tag, (outer, red, inner) in (("first", first), ("second, smaller", second)):
        case(f"reduce_static kind {kind} {tag} [{outer},{red},{inner}]")
        x = synth.normal(900 + red % 97, (outer, red, inner))
        plain, static = both(ctx, kind, x, outer, red, inner)
        assert_bits_equal(static, plain, f"static vs ahip_reduce [{outer},{red},{inner}]")
        if kind == D.REDUCE_MAX:
            assert_bits_equal(static, x.max(axis=1), "max vs numpy")
        elif kind == D.REDUCE_MEAN:
            ref = oracle.reduce(oracle.REDUCE_MEAN, x, [1], False)
            assert_close(static, ref.reshape(outer, inner), rtol=1e-5, atol=1e-6, what="static vs oracle")
        else:  # the oracle has no plain sum: float64, at the accuracy of an fp32 sum of `red` terms
            assert_close(static, x.astype(np.float64).sum(axis=1), rtol=1e-5, atol=2e-7 * red, what="sum vs float64")


def test_reduce_static_rejects_what_does_not_fit(ctx, case):
    """A shape whose partial results exceed the fixed array fails with a clear error and writes nothing;
    ahip_reduce takes the same shape (its buffer is larger)."""
    case("reduce_static capacity")
    cap = lib().ahip_reduce_static_capacity()
    assert cap == 1 << 18
    outer, red, inner = 3, 2048, 4096  # 3 slabs x 22 slices x 4096 columns of partial results
    x = synth.normal(77, (outer, red, inner))
    dx = ctx.upload(x)
    sentinel = np.full(outer * inner, -7.0, np.float32)
    do = ctx.upload(sentinel)
    try:
        with pytest.raises(AltiusHipError) as e:
            ctx.reduce_static_raw(D.REDUCE_MAX, do.ptr, dx.ptr, outer, red, inner)
        assert e.value.code == ERR_UNSUPPORTED
        assert "fixed buffer" in str(e.value) and str(cap) in str(e.value)
        assert_bits_equal(ctx.download(do, (outer * inner,)), sentinel, "nothing written")
        ctx.reduce_raw(D.REDUCE_MAX, do.ptr, dx.ptr, outer, red, inner)
        assert_bits_equal(ctx.download(do, (outer, inner)), x.max(axis=1), "ahip_reduce takes it")
        # and the entry point still works afterwards
        ctx.reduce_static_raw(D.REDUCE_MAX, do.ptr, dx.ptr, 1, outer * red * inner, 1)
        assert ctx.download(do, (1,))[0] == x.max()
    finally:
        ctx.free(dx)
        ctx.free(do)


def test_reduce_static_on_a_second_context(case):
    """The array belongs to the GPU, not to a context: a context created later resolves the same address
    and gets the same results."""
    case("reduce_static second context")
    x = synth.normal(5, (1, 2_000_000, 1))
    with D.Context(0) as other:
        plain, static = both(other, D.REDUCE_MAX, x, 1, 2_000_000, 1)
    assert_bits_equal(static, plain, "second context")
    assert static[0, 0] == x.max()
