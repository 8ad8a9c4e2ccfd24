"""The one-kernel attention (Softmax(scale(Q K^T)) V with the scores in registers), through the C ABI and through
the session that recognises MatMul -> Softmax -> MatMul.  Pinned by the definition in float64 and by the three
separate operators (whose Softmax is itself held to the oracle elsewhere): same exp, same normalisation, other
summation orders.  Unscaled scores of 64-wide N(0,1) vectors reach +-30, where an fp32 rounding of the score
already moves exp by 3e-5 relative: the bars are 2e-4 relative, 2e-5 absolute."""
import ctypes

import numpy as np
import pytest

from altius_amd._lib import ERR_UNSUPPORTED, AltiusHipError, check

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(99)


def reference(q, k, v, scale_op, scale):
    s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2)
    s = s * scale if scale_op == 1 else s / scale if scale_op == 2 else s
    e = np.exp(s - s.max(-1, keepdims=True))
    return (e / e.sum(-1, keepdims=True)) @ v.astype(np.float64)


@pytest.mark.parametrize("batch,tq,tk", [((2, 3), 197, 197), ((1,), 1, 1), ((4,), 32, 32), ((2,), 33, 31), ((3,), 70, 256), ((1,), 300, 100),
                                         ((2, 2), 64, 129), ((1,), 257, 224), ((5,), 7, 200)])
@pytest.mark.parametrize("scale_op", [0, 1, 2])
def test_attention_matches_its_definition_and_the_separate_operators(ctx, case, batch, tq, tk, scale_op):
    case(f"attention batch {batch} tq {tq} tk {tk} scale_op {scale_op}")
    q = RNG.standard_normal(batch + (tq, 64)).astype(np.float32)
    k = RNG.standard_normal(batch + (tk, 64)).astype(np.float32)
    v = RNG.standard_normal(batch + (tk, 64)).astype(np.float32)
    scale = np.float32(0.125) if scale_op == 1 else np.float32(8.0)
    got = ctx.attention(q, k, v, scale_op, float(scale))
    np.testing.assert_allclose(got, reference(q, k, v, scale_op, scale), rtol=2e-4, atol=2e-5)
    s = ctx.matmul(q, np.ascontiguousarray(np.swapaxes(k, -1, -2)))
    s = s * scale if scale_op == 1 else s / scale if scale_op == 2 else s
    sep = ctx.matmul(ctx.softmax(s.astype(np.float32)), v)
    np.testing.assert_allclose(got, sep, rtol=2e-4, atol=2e-5)


def test_attention_with_peaked_and_masked_like_scores(ctx, case):
    """Large score ranges (one key dominating, keys at -1e4 relative) exercise the exp clamp and the row maximum."""
    case("attention, peaked scores")
    q = (RNG.standard_normal((2, 50, 64)) * 6).astype(np.float32)
    k = (RNG.standard_normal((2, 90, 64)) * 6).astype(np.float32)
    v = RNG.standard_normal((2, 90, 64)).astype(np.float32)
    got = ctx.attention(q, k, v)
    np.testing.assert_allclose(got, reference(q, k, v, 0, 1.0), rtol=2e-3, atol=2e-4)
    rows = got.reshape(-1, 64)
    assert np.isfinite(rows).all()


def test_attention_with_masks(ctx, case):
    case("attention with per-key masks")
    q = RNG.standard_normal((3, 2, 40, 64)).astype(np.float32)
    k = RNG.standard_normal((3, 2, 70, 64)).astype(np.float32)
    v = RNG.standard_normal((3, 2, 70, 64)).astype(np.float32)
    for mask in (np.where(RNG.random(70) < 0.3, -1e4, 0.0).astype(np.float32), np.where(RNG.random((3, 70)) < 0.3, -1e4, 0.0).astype(np.float32)):
        got = ctx.attention(q, k, v, 2, 8.0, mask=mask)
        s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2) / 8.0 + (mask if mask.ndim == 1 else mask[:, None, None, :])
        e = np.exp(s - s.max(-1, keepdims=True))
        np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)


def test_attention_reads_heads_in_place(ctx, case):
    """Q, K, V as column blocks of one [b, t, 3 h d] tensor, O written as [b, t, h d]: row pitches and two-level batches."""
    case("attention on strided heads")
    b, t, h, d = 2, 45, 3, 64
    x = RNG.standard_normal((b, t, 3 * h * d)).astype(np.float32)
    dx, do = ctx.upload(x), ctx.alloc(b * t * h * d * 4)
    S = ctypes.c_size_t * 2
    try:
        ld = 3 * h * d
        check(ctx.L.ahip_attention(ctx.handle, do.ptr, dx.ptr, dx.ptr + h * d * 4, dx.ptr + 2 * h * d * 4, b, h, t, t, d, ld, ld, ld, h * d,
                                   S(t * ld, d), S(t * ld, d), S(t * ld, d), S(t * h * d, d), 1, 0.125, None, 0), ctx.handle)
        got = ctx.download(do, (b, t, h, d))
    finally:
        ctx.free(dx)
        ctx.free(do)
    q, k, v = (x[:, :, i * h * d:(i + 1) * h * d].reshape(b, t, h, d).transpose(0, 2, 1, 3) for i in range(3))
    np.testing.assert_allclose(got.transpose(0, 2, 1, 3), reference(q, k, v, 1, 0.125), rtol=2e-5, atol=2e-6)


def test_attention_refuses_what_it_cannot_do(ctx, case):
    case("attention refusals")
    q = np.zeros((4, 32), np.float32)               # heads that are not 64 wide
    with pytest.raises(AltiusHipError) as e:
        ctx.attention(q, q, q)
    assert e.value.code == ERR_UNSUPPORTED


@pytest.mark.parametrize("tq,tk", [(50, 257), (128, 512), (33, 1000), (300, 300)])
def test_long_sequences_are_streamed(ctx, case, tq, tk):
    """More than 256 keys: chunks of 64 keys through LDS with a running maximum and sum per query."""
    case(f"streamed attention tq {tq} tk {tk}")
    q = RNG.standard_normal((2, 2, tq, 64)).astype(np.float32)
    k = RNG.standard_normal((2, 2, tk, 64)).astype(np.float32)
    v = RNG.standard_normal((2, 2, tk, 64)).astype(np.float32)
    mask = np.where(RNG.random((2, tk)) < 0.2, -1e4, 0.0).astype(np.float32)
    got = ctx.attention(q, k, v, 1, 0.125, mask=mask)
    s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2) * 0.125 + mask[:, None, None, :]
    e = np.exp(s - s.max(-1, keepdims=True))
    np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("heads,tq,tk", [(256, 40, 70), (128, 197, 197), (96, 197, 130), (600, 33, 64), (12, 197, 197), (3, 500, 77)])
def test_every_block_shape(ctx, case, heads, tq, tk):
    """The launcher sizes its blocks to the work: 8, 4 or 2 query tiles per block when there are many (batch, head)
    pairs (the first four cases, in that order and 8 again), one query tile per block with the keys dealt out among
    its wavefronts when there are few (the last two)."""
    case(f"attention block shapes: {heads} heads, tq {tq}, tk {tk}")
    q = RNG.standard_normal((heads, tq, 64)).astype(np.float32)
    k = RNG.standard_normal((heads, tk, 64)).astype(np.float32)
    v = RNG.standard_normal((heads, tk, 64)).astype(np.float32)
    mask = np.where(RNG.random(tk) < 0.2, -1e4, 0.0).astype(np.float32)
    got = ctx.attention(q, k, v, 1, 0.125, mask=mask)
    s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2) * 0.125 + mask
    e = np.exp(s - s.max(-1, keepdims=True))
    np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)


def test_keys_split_over_wavefronts_with_empty_and_masked_parts(ctx, case):
    """Few heads: the keys of a chunk of 128 go to four wavefronts.  Fewer keys than wavefronts' tiles (some wavefronts
    have nothing to add), and a mask that removes every key of one wavefront's tile."""
    case("attention, keys split over wavefronts: idle and fully masked parts")
    for tk in (1, 31, 33, 64, 65, 127, 129, 200):
        q = RNG.standard_normal((2, 37, 64)).astype(np.float32)
        k = RNG.standard_normal((2, tk, 64)).astype(np.float32)
        v = RNG.standard_normal((2, tk, 64)).astype(np.float32)
        mask = np.zeros(tk, np.float32)
        if tk > 64:
            mask[32:64] = -1e4  # the second wavefront's whole tile
        got = ctx.attention(q, k, v, 2, 8.0, mask=mask)
        s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2) / 8.0 + mask
        e = np.exp(s - s.max(-1, keepdims=True))
        np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5, err_msg=f"tk {tk}")


# ---- the same kernel on the bf16 matrix cores (contexts whose products may take that route) --------------------------

@pytest.fixture()
def bf16_ctx():
    from altius_amd import device as D

    c = D.Context(0)
    c.gemm_set_algorithm(D.GEMM_BF16X3)
    yield c
    c.close()


@pytest.mark.parametrize("heads,tq,tk", [(300, 197, 197), (256, 40, 70), (600, 33, 64), (260, 300, 100), (256, 1, 1), (512, 64, 31),
                                         (256, 257, 224), (256, 5, 33)])
@pytest.mark.parametrize("scale_op", [0, 1, 2])
def test_attention_on_the_bf16_matrix_cores(bf16_ctx, ctx, case, heads, tq, tk, scale_op):
    """Enough (batch, head) pairs for full blocks: both products run as six bf16 MFMAs per k step on operands split
    into three bf16 planes (K, V on their way into LDS, Q in registers, the probabilities where the first product
    leaves them).  Held to the definition in float64 at the fp32 kernel's bars, and to the fp32 kernel itself."""
    case(f"bf16 attention: {heads} heads, tq {tq}, tk {tk}, scale_op {scale_op}")
    q = RNG.standard_normal((heads, tq, 64)).astype(np.float32)
    k = RNG.standard_normal((heads, tk, 64)).astype(np.float32)
    v = RNG.standard_normal((heads, tk, 64)).astype(np.float32)
    scale = np.float32(0.125) if scale_op == 1 else np.float32(8.0)
    mask = np.where(RNG.random(tk) < 0.2, -1e4, 0.0).astype(np.float32) if scale_op else None
    if mask is not None:
        mask[0] = 0.0
    got = bf16_ctx.attention(q, k, v, scale_op, float(scale), mask=mask)
    s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2)
    s = s * scale if scale_op == 1 else s / scale if scale_op == 2 else s
    if mask is not None:
        s = s + mask
    e = np.exp(s - s.max(-1, keepdims=True))
    np.testing.assert_allclose(got, (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got, ctx.attention(q, k, v, scale_op, float(scale), mask=mask), rtol=2e-4, atol=2e-5)


def test_bf16_attention_reads_heads_in_place_with_a_mask_per_batch(bf16_ctx, case):
    case("bf16 attention on strided heads, one mask row per batch")
    b, t, h, d = 24, 45, 12, 64
    x = RNG.standard_normal((b, t, 3 * h * d)).astype(np.float32)
    mask = np.where(RNG.random((b, t)) < 0.3, -1e4, 0.0).astype(np.float32)
    mask[:, 0] = 0.0
    dx, do, dm = bf16_ctx.upload(x), bf16_ctx.alloc(b * t * h * d * 4), bf16_ctx.upload(mask)
    S = ctypes.c_size_t * 2
    try:
        ld = 3 * h * d
        check(bf16_ctx.L.ahip_attention(bf16_ctx.handle, do.ptr, dx.ptr, dx.ptr + h * d * 4, dx.ptr + 2 * h * d * 4, b, h, t, t, d, ld, ld, ld,
                                        h * d, S(t * ld, d), S(t * ld, d), S(t * ld, d), S(t * h * d, d), 1, 0.125, dm.ptr, t), bf16_ctx.handle)
        got = bf16_ctx.download(do, (b, t, h, d))
    finally:
        for m in (dx, do, dm):
            bf16_ctx.free(m)
    q, k, v = (x[:, :, i * h * d:(i + 1) * h * d].reshape(b, t, h, d).transpose(0, 2, 1, 3) for i in range(3))
    s = q.astype(np.float64) @ np.swapaxes(k.astype(np.float64), -1, -2) * 0.125 + mask[:, None, None, :]
    e = np.exp(s - s.max(-1, keepdims=True))
    np.testing.assert_allclose(got.transpose(0, 2, 1, 3), (e / e.sum(-1, keepdims=True)) @ v, rtol=2e-4, atol=2e-5)


def test_bf16_attention_special_values(bf16_ctx, case):
    """Values the hardware conversion would round up to infinity are truncated (the planes still add up to the value);
    an exact representation: integer-valued operands give the exact result of the definition wherever the probabilities
    are exact (one key: probability 1); an infinite operand gives NaN (for most elements; +inf, the fp32 result, for the rest), as in the product on this route."""
    case("bf16 attention: huge, integer-valued and infinite operands")
    heads, tq = 256, 40
    q = RNG.integers(-3, 4, (heads, tq, 64)).astype(np.float32)
    k = RNG.integers(-3, 4, (heads, 1, 64)).astype(np.float32)
    v = (RNG.integers(-(2 ** 23), 2 ** 23, (heads, 1, 64))).astype(np.float32)
    v[0, 0, :4] = [3.4e38, -3.4e38, 3.3895e38, 1e-30]  # (below 2^-109 the third plane runs out of exponent)
    got = bf16_ctx.attention(q, k, v)
    np.testing.assert_array_equal(got, np.broadcast_to(v, got.shape))  # one key: O = V, every bit of it
    k2 = RNG.standard_normal((heads, 70, 64)).astype(np.float32)
    v2 = RNG.standard_normal((heads, 70, 64)).astype(np.float32)
    v2[3, 5, 7] = np.inf
    out = bf16_ctx.attention(q, k2, v2, 1, 0.125)
    col = out[3, :, 7]  # NaN (inf times a zero lower plane of a probability) or the fp32 kernel's +inf, never a finite number
    assert (np.isnan(col) | (col == np.inf)).all() and np.isnan(col).mean() > 0.5
    assert np.isfinite(out[3, :, :7]).all() and np.isfinite(np.delete(out, 3, axis=0)).all()
