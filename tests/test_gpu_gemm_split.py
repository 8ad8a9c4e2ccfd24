"""The fp32 GEMM that runs on the bf16 matrix cores (three bf16 planes per operand, six MFMAs per product),
through the C ABI.  What pins it: operands that bf16 holds exactly give exact products and sums, so integer
matrices must come out bit for bit; an identity operand must reproduce full 24-bit values exactly (the three
planes add back up to the value); on random operands the error against float64 must stay inside the forward
bound of an fp32 accumulation and be no worse, on average, than the fp32 matrix-core kernel's."""
import numpy as np
import pytest

import oracle as O
from altius_amd import device as D
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(77)


@pytest.fixture
def split(ctx):
    ctx.gemm_set_algorithm(D.GEMM_BF16X3)
    yield ctx
    ctx.gemm_set_algorithm(D.GEMM_DEFAULT)


def ints(*shape):
    return RNG.integers(-4, 5, size=shape).astype(np.float32)


def rel_error(got, a, b):
    """|C - exact| / (|A||B|), element-wise, against a float64 product."""
    exact = a.astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64) + 1e-300
    return np.abs(got.astype(np.float64) - exact) / scale


SHAPES = [(5, 10, 15), (1, 1, 1), (256, 16, 256), (257, 17, 255), (255, 15, 257), (300, 7, 3), (64, 300, 64), (513, 33, 130),
          (394, 768, 2304), (1000, 129, 520), (31, 1000, 700)]


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_exact_on_integers_and_bounded_on_reals(split, case, m, k, n):
    case(f"bf16x3 gemm {m}x{k}x{n}")
    a, b = ints(m, k), ints(k, n)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    assert_bits_equal(split.matmul(a, b), want, "integer operands")
    a, b = RNG.standard_normal((m, k)).astype(np.float32), RNG.standard_normal((k, n)).astype(np.float32)
    got = split.matmul(a, b)
    err = rel_error(got, a, b)
    assert err.max() <= (k + 2) * 2.0 ** -24, f"error {err.max():.3e} beyond the fp32 accumulation bound"
    assert np.allclose(got, O.matmul(a, b), rtol=1e-5, atol=1e-5 * np.sqrt(k)), "differs from the oracle"


def test_identity_reproduces_every_bit(split, case):
    """x * I and I * x: each output is one operand value times 1.0, so the three planes must add back up to it."""
    case("bf16x3 gemm identity")
    n = 300
    x = (RNG.standard_normal((n, n)) * np.exp(RNG.uniform(-20, 20, (n, n)))).astype(np.float32)
    x[0, :8] = [np.float32(16777215.0), np.float32(1.0000001), np.float32(-3.4028235e38), np.float32(3.3895314e38),
                np.float32(1.17549435e-38), np.float32(0.1), np.float32(-0.0), np.float32(8388609.0)]
    eye = np.eye(n, dtype=np.float32)
    assert_bits_equal(split.matmul(x, eye) + np.float32(0), x + np.float32(0), "identity on the right")
    assert_bits_equal(split.matmul(eye, x) + np.float32(0), x + np.float32(0), "identity on the left")


def test_each_product_lands_in_its_place(split, case):
    case("bf16x3 gemm placement")
    m, k, n = 270, 37, 290
    a = np.zeros((m, k), np.float32)
    b = np.zeros((k, n), np.float32)
    a[:, 5] = np.arange(1, m + 1)
    b[5, :] = np.arange(1, n + 1) * 8
    assert_bits_equal(split.matmul(a, b), np.outer(np.arange(1, m + 1), np.arange(1, n + 1) * 8).astype(np.float32), "outer product")
    # one non-zero k at a time over a depth that spans several stages and the padded tail
    a, b = ints(40, 50), ints(50, 30)
    for kk in (0, 7, 8, 15, 16, 31, 32, 47, 49):
        az, bz = np.zeros_like(a), np.zeros_like(b)
        az[:, kk], bz[kk, :] = a[:, kk], b[kk, :]
        assert_bits_equal(split.matmul(az, bz), np.outer(a[:, kk], b[kk, :]).astype(np.float32), f"k = {kk}", zero_sign_free=True)


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_transposes_alpha_beta_and_every_c_shape(split, case, ta, tb):
    case(f"bf16x3 gemm transA={ta} transB={tb}")
    for m, k, n in [(5, 10, 15), (130, 70, 129), (260, 64, 300), (3, 1, 2)]:
        a, b = ints(*((k, m) if ta else (m, k))), ints(*((n, k) if tb else (k, n)))
        for c in (None, ints(n), ints(m, n), ints(1, n), ints(m, 1), ints(1)):
            got = split.gemm(a, b, c, alpha=2.0, beta=3.0, trans_a=ta, trans_b=tb)
            assert_bits_equal(got, O.gemm(a, b, c, alpha=2.0, beta=3.0, trans_a=ta, trans_b=tb),
                              f"gemm {m}x{k}x{n} c={None if c is None else c.shape}")


def test_unaligned_operands_and_pitches(split, case):
    case("bf16x3 gemm on unaligned pointers / padded pitches")
    a, b = ints(33, 21), ints(21, 19)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    da, db = split.upload(np.concatenate([np.zeros(1, np.float32), a.ravel()])), split.upload(np.concatenate([np.zeros(3, np.float32), b.ravel()]))
    dc = split.alloc((33 * 23 + 1) * 4)
    split.memset(dc, 0)
    try:
        split.gemm_raw(dc.offset(4), da.offset(4), db.offset(12), None, 1, 33, 19, 21, ldc=23)
        got = split.download(dc, (33 * 23 + 1,))[1:].reshape(33, 23)[:, :19]
        assert_bits_equal(got, want, "offset pointers, ldc 23")
    finally:
        for x in (da, db, dc):
            split.free(x)


def test_non_finite_values_propagate(split, case):
    """NaN operands give NaN as in fp32.  An infinite operand gives NaN where fp32 gives an infinity: its product with
    the (zero) low planes of the other operand is inf * 0.  Entries that no non-finite operand reaches are exact."""
    case("bf16x3 gemm with inf / nan")
    a, b = ints(20, 24), ints(24, 18)
    a[3, 5], a[7, 0], b[2, 4] = np.inf, np.nan, -np.inf
    with np.errstate(invalid="ignore"):
        want = a.astype(np.float64) @ b.astype(np.float64)
    got = split.matmul(a, b)
    assert np.array_equal(np.isnan(got), ~np.isfinite(want))
    fin = np.isfinite(want)
    assert_bits_equal(got[fin], want[fin].astype(np.float32), "finite entries")
    # an overflow inside the accumulation is an infinity, as in fp32
    big = np.full((4, 8), 3e38, np.float32)
    assert np.all(np.isposinf(split.matmul(big, np.ones((8, 5), np.float32))))


def test_registered_constant_is_split_once_and_stays_valid(split, case):
    case("bf16x3 gemm with a registered constant operand")
    a1, a2, w = ints(70, 40), ints(300, 40), ints(40, 50)
    dw = split.upload(w)
    split.gemm_register_constant(dw)
    try:
        for a in (a1, a2, a1):
            da, dc = split.upload(a), split.alloc(a.shape[0] * 50 * 4)
            try:
                split.gemm_raw(dc.ptr, da.ptr, dw.ptr, None, 1, a.shape[0], 50, 40)
                assert_bits_equal(split.download(dc, (a.shape[0], 50)), (a.astype(np.float64) @ w.astype(np.float64)).astype(np.float32),
                                  "product with cached planes")
            finally:
                split.free(da)
                split.free(dc)
    finally:
        split.gemm_unregister_constant(dw)
        split.free(dw)
    # after unregistering, a new buffer (possibly at the same address) with other contents is split afresh
    w2 = ints(40, 50)
    assert_bits_equal(split.gemm(a1, w2), (a1.astype(np.float64) @ w2.astype(np.float64)).astype(np.float32), "fresh operand")


def test_no_less_accurate_than_the_fp32_matrix_cores(ctx, case):
    """Same operands through both kernels: the split kernel's error against float64 is, on average and at worst,
    not above the fp32 kernel's (with a 25 % allowance for the different summation orders)."""
    case("bf16x3 vs fp32 MFMA accuracy")
    m, k, n = 2048, 3072, 2048  # more tiles than CUs: the fp32 kernel walks all of k in one block, its usual summation
    a = RNG.standard_normal((m, k)).astype(np.float32)
    b = (RNG.standard_normal((k, n)) * 0.05).astype(np.float32)
    try:
        ctx.gemm_set_algorithm(D.GEMM_FP32)
        e32 = rel_error(ctx.matmul(a, b), a, b)
        ctx.gemm_set_algorithm(D.GEMM_BF16X3)
        e16 = rel_error(ctx.matmul(a, b), a, b)
    finally:
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)
    print(f"rms error / |A||B|: fp32 MFMA {np.sqrt((e32 ** 2).mean()):.3e}, bf16 x 3 {np.sqrt((e16 ** 2).mean()):.3e}; "
          f"max {e32.max():.3e} vs {e16.max():.3e}")
    assert np.sqrt((e16 ** 2).mean()) <= 1.25 * np.sqrt((e32 ** 2).mean())
    assert e16.max() <= 1.25 * e32.max()


# Shapes whose last round of blocks per XCD is partly filled, so tiles are cut along k inside the kernel:
# 16 tiles -> 2 per XCD -> up to 8 slices each; 48 tiles -> 6 per XCD -> 5 slices; 9 tiles (7 XCDs with 2, ragged).
CUT_SHAPES = [(1024, 512, 1024), (1024, 2048, 1024), (2048, 640, 1536), (700, 1024, 600), (256, 4096, 256)]


@pytest.mark.parametrize("m,k,n", CUT_SHAPES)
def test_k_cut_inside_the_kernel_and_its_fallback_give_the_same_exact_products(split, case, m, k, n):
    """The slices of a tile are added up inside one XCD's L2 only on a context whose probe showed that blocks with
    equal ids mod 8 share an XCD; with the cut forced off (what such a context falls back to) every tile is computed by one block.  Both
    must give the exact products of integer operands, bit for bit, on repeated launches (the counters and the
    partial sums of the previous launch are still in place)."""
    shown, enabled = split.gemm_in_kernel_k_cut()
    case(f"bf16x3 k cut {m}x{k}x{n}; placement shown {shown}, cut enabled {enabled}")
    assert enabled
    a, b = ints(m, k), ints(k, n)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    bias = ints(n)
    try:
        for cut in (True, False, True):
            split.gemm_set_in_kernel_k_cut(cut)
            assert split.gemm_in_kernel_k_cut() == (shown, cut)
            for _ in range(2):
                assert_bits_equal(split.matmul(a, b), want, f"cut {cut}")
            assert_bits_equal(split.gemm(a, b, bias, alpha=2.0, beta=3.0), 2 * want + 3 * bias, f"cut {cut}, alpha / beta / bias")
        ar, br = RNG.standard_normal((m, k)).astype(np.float32), RNG.standard_normal((k, n)).astype(np.float32)
        split.gemm_set_in_kernel_k_cut(True)
        with_cut = split.matmul(ar, br)
        split.gemm_set_in_kernel_k_cut(False)
        without = split.matmul(ar, br)
        for got in (with_cut, without):
            assert rel_error(got, ar, br).max() <= (k + 2) * 2.0 ** -24
    finally:
        split.gemm_set_in_kernel_k_cut(True)


def test_this_part_deals_blocks_to_xcds_in_turn(ctx, case):
    """What the library measures at context creation on an MI355X in its default partition mode: 256 CUs, eight
    consecutive blocks on eight XCDs, block i where block i % 8 ran.  (On a part where this does not hold the
    library only loses the in-kernel cut.)"""
    case("placement probe")
    shown, enabled = ctx.gemm_in_kernel_k_cut()
    assert enabled
    assert shown, "the probe did not find blocks dealt to the XCDs in turn: the bf16 GEMM runs without its in-kernel k cut"


def test_auto_takes_the_split_kernel_at_model_size(ctx, case):
    """[12608, 768] x [768, 2304] (a quarter of the ViT-B/16 batch-256 QKV projection) under the AHIP_GEMM_AUTO rule,
    with a bias row: sampled rows against float64."""
    case("auto-selected gemm 12608x768x2304")
    m, k, n = 12608, 768, 2304
    a = RNG.standard_normal((m, k)).astype(np.float32)
    b = (RNG.standard_normal((k, n)) * 0.03).astype(np.float32)
    bias = RNG.standard_normal(n).astype(np.float32)
    try:
        ctx.gemm_set_algorithm(D.GEMM_AUTO)
        got = ctx.gemm(a, b, bias)
    finally:
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)
    rows = RNG.choice(m, 64, replace=False)
    exact = a[rows].astype(np.float64) @ b.astype(np.float64)
    scale = np.abs(a[rows]).astype(np.float64) @ np.abs(b).astype(np.float64)
    err = np.abs(got[rows].astype(np.float64) - (exact + bias)) / (scale + np.abs(bias))
    assert err.max() <= (k + 3) * 2.0 ** -24
    assert np.sqrt((err ** 2).mean()) < 1e-7
