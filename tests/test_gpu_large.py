"""Tensors past the 32-bit marks: more than 2^32 bytes (1.35 G elements) and more than 2^31 elements (2.2 G).

The reference indexes with usize and has no such marks; here element offsets inside the kernels are 64-bit or the
launcher splits the work, and this file checks it where it shows: windows of the result at the start, either side of
element 2^30 (byte 2^32), either side of element 2^31, and at the end, against NumPy / the oracle on the same values.
The input is a 64 MiB block of seeded values repeated, so that any window can be rebuilt on the host without holding
9 GB there."""
import ctypes

import numpy as np
import pytest

from altius_amd import device as D
from altius_amd import synth
from altius_amd._lib import check
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu

ROW = 768 * 197                       # every size is a whole number of rows of 768 and of 197
N_BYTES = ROW * 8900                  # 1 346 534 400 elements: 5.4 GB, byte offsets pass 2^32
N_ELEMS = ROW * 14600                 # 2 208 921 600 elements: 8.8 GB, element offsets pass 2^31
PERIOD = 1 << 24


@pytest.fixture(scope="module")
def big(ctx):
    chunk = synth.normal(91, (PERIOD,), mean=0.1, std=1.3)
    d_in = ctx.alloc(N_ELEMS * 4)
    d_out = ctx.alloc(N_ELEMS * 4)
    for start in range(0, N_ELEMS, PERIOD):
        count = min(PERIOD, N_ELEMS - start)
        check(ctx.L.ahip_h2d_async(ctx.handle, d_in.ptr + start * 4, chunk.ctypes.data, count * 4), ctx.handle)
    ctx.sync()
    yield chunk, d_in, d_out
    ctx.free(d_in)
    ctx.free(d_out)


def values(chunk, start, count):
    """Elements [start, start + count) of the repeated block."""
    return chunk[(np.arange(start, start + count, dtype=np.int64) % PERIOD)]


def windows(n, unit, width=6):
    """Starts (in units of `unit` elements) of windows at the beginning, at every 32-bit mark inside n, and at the end."""
    total = n // unit
    marks = [0, total - width]
    for mark in (1 << 30, 1 << 31):
        if mark < n:
            marks.append(max(0, mark // unit - width // 2))
    return sorted(set(marks))


@pytest.mark.parametrize("n", [N_BYTES, N_ELEMS])
def test_elementwise_past_the_32_bit_marks(ctx, case, big, n):
    case(f"Sqrt, Add, Mul by a vector, Div by a scalar on {n} elements")
    chunk, d_in, d_out = big
    span = 8192

    def check_windows(expect, what):
        for w in windows(n, span, 2):
            got = ctx.download(d_out, (span,), offset_bytes=w * span * 4)
            with np.errstate(all="ignore"):
                assert_bits_equal(got, expect(values(chunk, w * span, span), w * span), f"{what} at element {w * span}")

    ctx.unary_raw(D.SQRT, d_out.ptr, d_in.ptr, n)
    check_windows(lambda x, at: np.sqrt(x), "Sqrt")
    dims = [n]
    ones = D.strides_for_broadcasting([n], dims)
    ctx.binary_raw(D.ADD, d_out.ptr, d_in.ptr, d_in.ptr, dims, ones, ones)
    check_windows(lambda x, at: x + x, "Add")
    vec = synth.normal(92, (768,), mean=1.0, std=0.3)
    d_vec = ctx.upload(vec)
    dims = [n // 768, 768]
    ctx.binary_raw(D.MUL, d_out.ptr, d_in.ptr, d_vec.ptr, dims, D.strides_for_broadcasting(dims, dims),
                   D.strides_for_broadcasting([768], dims))
    check_windows(lambda x, at: x * vec[(np.arange(at, at + len(x)) % 768)], "Mul by a vector")
    d_s = ctx.upload(np.array([synth.DIV_SCALAR], np.float32))
    ctx.binary_raw(D.DIV, d_out.ptr, d_in.ptr, d_s.ptr, [n], D.strides_for_broadcasting([n], [n]), D.strides_for_broadcasting([], [n]))
    check_windows(lambda x, at: x / synth.DIV_SCALAR, "Div by a scalar")
    ctx.free(d_vec)
    ctx.free(d_s)


@pytest.mark.parametrize("n", [N_BYTES, N_ELEMS])
def test_row_operators_past_the_32_bit_marks(ctx, oracle, case, big, n):
    case(f"Softmax over rows of 197, LayerNormalization and ReduceMean over rows of 768, ReduceMax over axis 1, {n} elements")
    chunk, d_in, d_out = big
    ctx.softmax_raw(d_out.ptr, d_in.ptr, n // 197, 197)
    for w in windows(n, 197):
        got = ctx.download(d_out, (6, 197), offset_bytes=w * 197 * 4)
        assert_close(got, oracle.softmax(values(chunk, w * 197, 6 * 197).reshape(6, 197)), what=f"Softmax at row {w}")
    g = synth.normal(93, (768,), mean=1.0, std=0.02)
    b = synth.normal(94, (768,), mean=0.0, std=0.02)
    d_g, d_b = ctx.upload(g), ctx.upload(b)
    ctx.layernorm_raw(d_out.ptr, d_in.ptr, d_g.ptr, d_b.ptr, n // 768, 768, 1e-5)
    for w in windows(n, 768):
        got = ctx.download(d_out, (6, 768), offset_bytes=w * 768 * 4)
        assert_close(got, oracle.layer_norm(values(chunk, w * 768, 6 * 768).reshape(6, 768), g, b, 1e-5), what=f"LayerNormalization at row {w}")
    ctx.reduce_raw(D.REDUCE_MEAN, d_out.ptr, d_in.ptr, n // 768, 768, 1)
    for w in windows(n, 768):
        got = ctx.download(d_out, (6,), offset_bytes=w * 4)
        want = oracle.reduce(oracle.REDUCE_MEAN, values(chunk, w * 768, 6 * 768).reshape(6, 768), [1], False)
        assert_close(got, want, what=f"ReduceMean at row {w}")
    slabs = n // ROW
    ctx.reduce_raw(D.REDUCE_MAX, d_out.ptr, d_in.ptr, slabs, 768, 197)
    for w in windows(n, ROW, 2):
        got = ctx.download(d_out, (2, 197), offset_bytes=w * 197 * 4)
        assert_bits_equal(got, values(chunk, w * ROW, 2 * ROW).reshape(2, 768, 197).max(1), f"ReduceMax at slab {w}")
    ctx.free(d_g)
    ctx.free(d_b)
