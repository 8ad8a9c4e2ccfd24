"""MatMul / Gemm on the matrix cores, through the C ABI and the session.  The accumulation order of a
GEMM is implementation-defined (the reference's own lives in the matrixmultiply crate), so parity is
what the mathematics fixes: exact results on integer-valued operands, the forward error bound
|C - exact| <= K * 2^-24 * |A||B| on random ones (and numpy.allclose, the reference's own test bar,
against the oracle), every tile-edge case, transposes, alpha / beta / bias, batch broadcasting."""
import numpy as np
import pytest

import oracle as O
from altius_amd.graph import Model, Op
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(31)


def ints(*shape):
    return RNG.integers(-4, 5, size=shape).astype(np.float32)


def check_bound(got, a, b, what):
    exact = np.matmul(a.astype(np.float64), b.astype(np.float64))
    k = a.shape[-1]
    bound = (k + 2) * 2.0 ** -24 * np.matmul(np.abs(a).astype(np.float64), np.abs(b).astype(np.float64)) + 1e-30
    err = np.abs(got.astype(np.float64) - exact)
    assert got.shape == exact.shape, f"{what}: shape {got.shape} vs {exact.shape}"
    assert np.all(err <= bound), f"{what}: error {err.max():.3e} beyond the bound (worst ratio {np.max(err / bound):.2f})"
    assert np.allclose(got, O.matmul(a, b), rtol=1e-5, atol=1e-5 * np.sqrt(k)), f"{what}: differs from the oracle"


SHAPES = [((5, 10), (10, 15)), ((3, 5, 10), (10, 15)), ((3, 5, 10), (3, 10, 15)), ((1, 5, 10), (10, 15)),       # test_ops_matmul.py
          ((128, 16), (16, 128)), ((129, 17), (17, 127)), ((1, 1), (1, 1)), ((64, 300), (300, 64)), ((257, 33), (33, 130)),
          ((2, 197, 768), (768, 2304)), ((2, 12, 197, 64), (2, 12, 64, 197)), ((2, 12, 197, 197), (2, 12, 197, 64)),
          ((1, 6, 3, 4), (1, 6, 4, 5)), ((7, 1, 9, 8), (8, 11)), ((4, 20, 31), (1, 31, 6)), ((300, 7), (7, 3))]


@pytest.mark.parametrize("sa,sb", SHAPES)
def test_matmul_exact_on_integers_and_bounded_on_reals(ctx, case, sa, sb):
    case(f"matmul {sa} x {sb}")
    a, b = ints(*sa), ints(*sb)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)
    assert_bits_equal(ctx.matmul(a, b), want, "integer operands")
    assert_bits_equal(O.matmul(a, b), want, "oracle agrees")
    a, b = RNG.standard_normal(sa).astype(np.float32), RNG.standard_normal(sb).astype(np.float32)
    check_bound(ctx.matmul(a, b), a, b, "random operands")


def test_matmul_each_product_lands_in_its_place(ctx, case):
    """Unit vectors pick single entries: C = A[:, p] (outer) B[q, :] catches a transposed or permuted fragment."""
    case("matmul placement")
    m, k, n = 70, 37, 90
    a = np.zeros((m, k), np.float32)
    b = np.zeros((k, n), np.float32)
    a[:, 5] = np.arange(1, m + 1)
    b[5, :] = np.arange(1, n + 1) * 1000
    assert_bits_equal(ctx.matmul(a, b), np.outer(np.arange(1, m + 1), np.arange(1, n + 1) * 1000).astype(np.float32), "outer product")
    eye = np.eye(150, dtype=np.float32)
    x = RNG.standard_normal((150, 150)).astype(np.float32)
    assert_bits_equal(ctx.matmul(eye, x), x, "identity on the left")
    assert_bits_equal(ctx.matmul(x, eye), x, "identity on the right")


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_gemm(ctx, case, ta, tb):
    case(f"gemm transA={ta} transB={tb}")
    for m, k, n in [(5, 10, 15), (130, 70, 129), (64, 64, 64), (3, 1, 2)]:
        a, b = ints(*((k, m) if ta else (m, k))), ints(*((n, k) if tb else (k, n)))
        for c in (None, ints(n), ints(m, n), ints(1, n), ints(m, 1), ints(1)):
            got = ctx.gemm(a, b, c, alpha=2.0, beta=3.0, trans_a=ta, trans_b=tb)
            assert_bits_equal(got, O.gemm(a, b, c, alpha=2.0, beta=3.0, trans_a=ta, trans_b=tb), f"gemm {m}x{k}x{n} c={None if c is None else c.shape}")
        ar, br = a + RNG.standard_normal(a.shape).astype(np.float32), b + RNG.standard_normal(b.shape).astype(np.float32)
        got = ctx.gemm(ar, br, None, trans_a=ta, trans_b=tb)
        check_bound(got, ar.T if ta else ar, br.T if tb else br, "random gemm")


def test_unaligned_operands_take_the_scalar_loads(ctx, case):
    case("gemm on unaligned pointers / odd pitches")
    a, b = ints(33, 21), ints(21, 19)                 # pitches 21 and 19: no 16-byte rows
    assert_bits_equal(ctx.matmul(a, b), a @ b, "odd pitches")
    da = ctx.upload(np.concatenate([np.zeros(1, np.float32), ints(64 * 32)]))
    db = ctx.upload(np.concatenate([np.zeros(3, np.float32), ints(32 * 48)]))
    dc = ctx.alloc(64 * 48 * 4 + 4)
    ctx.gemm_raw(dc.ptr + 4, da.ptr + 4, db.ptr + 12, None, 1, 64, 48, 32)
    A = ctx.download(da, (64 * 32 + 1,))[1:].reshape(64, 32)
    B = ctx.download(db, (32 * 48 + 3,))[3:].reshape(32, 48)
    assert_bits_equal(ctx.download(dc, (64 * 48 + 1,))[1:].reshape(64, 48), A @ B, "offset bases")
    for x in (da, db, dc):
        ctx.free(x)


def test_attention_block_through_the_session(case):
    """LayerNorm -> qkv MatMul + bias -> split -> heads -> QK^T * scale -> Softmax -> PV -> merge -> proj + residual,
    against the same chain on the oracle."""
    case("session: one attention block")
    B, T, H, NH = 2, 50, 64, 4
    D = H // NH
    x = RNG.standard_normal((B, T, H)).astype(np.float32)
    g, be = RNG.standard_normal(H).astype(np.float32), RNG.standard_normal(H).astype(np.float32)
    wqkv, bqkv = (RNG.standard_normal((H, 3 * H)) * 0.1).astype(np.float32), RNG.standard_normal(3 * H).astype(np.float32)
    wo, bo = (RNG.standard_normal((H, H)) * 0.1).astype(np.float32), RNG.standard_normal(H).astype(np.float32)
    m = Model(opset_version=13)
    v = m.new_val_named_and_shaped("x", x.shape)
    I = lambda a: m.new_initializer(np.asarray(a))
    n = lambda: m.new_val()
    ln, qkv, qkvb, q, k, vv = n(), n(), n(), n(), n(), n()
    m.add_node(Op.LayerNormalization, [v, I(g), I(be)], [ln], axis=-1, epsilon=1e-5)
    m.add_node(Op.MatMul, [ln, I(wqkv)], [qkv])
    m.add_node(Op.Add, [qkv, I(bqkv)], [qkvb])
    m.add_node(Op.Split, [qkvb, I(np.array([H, H, H], np.int64))], [q, k, vv], axis=2)
    heads = []
    for t in (q, k, vv):
        r, tr = n(), n()
        m.add_node(Op.Reshape, [t, I(np.array([B, T, NH, D], np.int64))], [r])
        m.add_node(Op.Transpose, [r], [tr], perm=[0, 2, 1, 3])
        heads.append(tr)
    kt, s, ss, p, ctxv, ct, cm, proj, pb, y = (n() for _ in range(10))
    m.add_node(Op.Transpose, [heads[1]], [kt], perm=[0, 1, 3, 2])
    m.add_node(Op.MatMul, [heads[0], kt], [s])
    m.add_node(Op.Mul, [s, I(np.array(1.0 / np.sqrt(D), np.float32))], [ss])
    m.add_node(Op.Softmax, [ss], [p], axis=-1)
    m.add_node(Op.MatMul, [p, heads[2]], [ctxv])
    m.add_node(Op.Transpose, [ctxv], [ct], perm=[0, 2, 1, 3])
    m.add_node(Op.Reshape, [ct, I(np.array([B, T, H], np.int64))], [cm])
    m.add_node(Op.MatMul, [cm, I(wo)], [proj])
    m.add_node(Op.Add, [proj, I(bo)], [pb])
    m.add_node(Op.Add, [v, pb], [y])
    m.add_input(v)
    m.add_output(y)
    (got,) = HipSessionBuilder(m).build().run([x])

    l = O.layer_norm(x, g, be, 1e-5)
    qkv_ = O.binary(O.ADD, O.matmul(l, wqkv), bqkv)
    qh, kh, vh = (np.ascontiguousarray(t.reshape(B, T, NH, D).transpose(0, 2, 1, 3)) for t in np.split(qkv_, 3, axis=2))
    sc = O.binary(O.MUL, O.matmul(qh, np.ascontiguousarray(kh.transpose(0, 1, 3, 2))), np.array(1.0 / np.sqrt(D), np.float32))
    pr = O.softmax(sc)
    cv = np.ascontiguousarray(O.matmul(pr, vh).transpose(0, 2, 1, 3)).reshape(B, T, H)
    want = O.binary(O.ADD, x, O.binary(O.ADD, O.matmul(cv, wo), bo))
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)


def test_gemm_head_through_the_session(case):
    case("session: Gemm classifier head")
    x, w, b = RNG.standard_normal((8, 768)).astype(np.float32), (RNG.standard_normal((1000, 768)) * 0.05).astype(np.float32), ints(1000)
    m = Model()
    v = m.new_val_named_and_shaped("x", x.shape)
    y = m.new_val()
    m.add_node(Op.Gemm, [v, m.new_initializer(w), m.new_initializer(b)], [y], transB=1)
    m.add_input(v)
    m.add_output(y)
    (got,) = HipSessionBuilder(m).build().run([x])
    assert np.allclose(got, O.gemm(x, w, b, trans_b=True), rtol=1e-5, atol=1e-4)
    check_bound(got - b, x, w.T, "gemm head")


@pytest.mark.parametrize("x_shape,w_shape", [([5, 10], [10, 15]), ([3, 197, 64], [64, 192]), ([2, 3, 50, 32], [2, 3, 32, 70]),
                                             ([4, 300, 256], [256, 130])])
def test_matmul_with_absorbed_bias_has_the_bits_of_matmul_then_add(case, x_shape, w_shape):
    """fuse_matmul_bias: the bias row goes into the product's epilogue as acc + bias, the one addition the
    separate Add node performs."""
    from altius_amd.graph import Model, Op
    from altius_amd.session import HipSessionBuilder

    case(f"matmul + bias {x_shape} x {w_shape}")
    rng = np.random.default_rng(5)
    x = rng.standard_normal(x_shape).astype(np.float32)
    w = (rng.standard_normal(w_shape) * 0.1).astype(np.float32)
    b = rng.standard_normal(w_shape[-1]).astype(np.float32)
    m = Model()
    vx = m.new_val_named_and_shaped("x", x_shape)
    p, y = m.new_val(), m.new_val()
    m.add_node(Op.MatMul, [vx, m.new_initializer(w)], [p])
    m.add_node(Op.Add, [p, m.new_initializer(b)], [y])
    m.add_input(vx)
    m.add_output(y)
    fused = m.clone()
    assert fused.fuse_matmul_bias() == 1 and len(fused.nodes()) == 1
    (want,) = HipSessionBuilder(m).build().run([x])
    (got,) = HipSessionBuilder(fused).build().run([x])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    np.testing.assert_allclose(got, np.matmul(x.astype(np.float64), w.astype(np.float64)) + b, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("a_shape,b_shape,ta,tb", [([2, 12, 197, 64], [2, 12, 197, 64], False, True), ([6, 5], [4, 6], True, True),
                                                   ([3, 40, 70], [3, 40, 33], True, False), ([4, 50, 32], [64, 32], False, True)])
def test_transposes_folded_into_the_product(case, a_shape, b_shape, ta, tb):
    """fuse_transpose_matmul: MatMul on the untransposed tensors with trans flags against Transpose -> MatMul; the
    accumulation order does not change, so the bits do not either."""
    case(f"matmul with folded transposes {a_shape} {b_shape} ta={ta} tb={tb}")
    rng = np.random.default_rng(8)
    a = rng.standard_normal(a_shape).astype(np.float32)
    b = rng.standard_normal(b_shape).astype(np.float32)
    swap = lambda r: list(range(r - 2)) + [r - 1, r - 2]
    m = Model()
    va, vb = m.new_val_named_and_shaped("a", a_shape), m.new_val_named_and_shaped("b", b_shape)
    xa, xb = va, vb
    if ta:
        xa = m.new_val()
        m.add_node(Op.Transpose, [va], [xa], perm=swap(len(a_shape)))
    if tb:
        xb = m.new_val()
        m.add_node(Op.Transpose, [vb], [xb], perm=swap(len(b_shape)))
    y = m.new_val()
    m.add_node(Op.MatMul, [xa, xb], [y])
    m.add_input(va)
    m.add_input(vb)
    m.add_output(y)
    fused = m.clone()
    assert fused.fuse_transpose_matmul() == 1 and [n["op_name"] for n in fused.nodes()] == ["MatMul"]
    (want,) = HipSessionBuilder(m).build().run([a, b])
    (got,) = HipSessionBuilder(fused).build().run([a, b])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    A = np.swapaxes(a, -1, -2) if ta else a
    Bm = np.swapaxes(b, -1, -2) if tb else b
    np.testing.assert_allclose(got, np.matmul(A.astype(np.float64), Bm.astype(np.float64)), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("m,k,n", [(197, 768, 2304), (197, 3072, 768), (100, 1024, 64), (8, 4096, 130), (300, 512, 300)])
def test_few_tiles_and_a_long_k_are_cut_along_k(ctx, case, m, k, n):
    """Few output tiles and k >= 512: k runs as batches of slices into a workspace and a second kernel adds the slices up
    in order (bias, alpha and beta applied there).  Exact on integers, bounded on reals, every C0 shape, both transposes."""
    from altius_amd import device as D

    case(f"split-k gemm {m}x{k}x{n}")
    try:
        ctx.gemm_set_algorithm(D.GEMM_FP32)
        for ta, tb in ((False, False), (True, True), (False, True)):
            a, b = ints(*((k, m) if ta else (m, k))), ints(*((n, k) if tb else (k, n)))
            for c in (None, ints(n), ints(m, n), ints(m, 1)):
                got = ctx.gemm(a, b, c, alpha=2.0, beta=3.0, trans_a=ta, trans_b=tb)
                assert_bits_equal(got, O.gemm(a, b, c, alpha=2.0, beta=3.0, trans_a=ta, trans_b=tb), f"ta={ta} tb={tb} c={None if c is None else c.shape}")
        a, b = RNG.standard_normal((m, k)).astype(np.float32), RNG.standard_normal((k, n)).astype(np.float32)
        check_bound(ctx.matmul(a, b), a, b, "random operands")
    finally:
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)


def _laid_out(x, pad, offset):
    """x [batch, rows, cols] as a flat array with `pad` unused floats behind every row and `offset` in front."""
    batch, rows, cols = x.shape
    full = np.zeros((batch, rows, cols + pad), np.float32)
    full[:, :, :cols] = x
    return np.concatenate([np.zeros(offset, np.float32), full.ravel()]), cols + pad


def _many_small(ctx, a, b, trans_b=False, pad=(0, 0), offset=(0, 0), shared_b=False):
    """C[z] = A[z] B[z] for a [batch, m, k] and b [batch, k, n] through one ahip_gemm call; B is handed over as
    [batch, n, k] when trans_b, rows are `pad` floats longer than their contents, bases `offset` floats past 16-byte
    boundaries.  Every extent handed to the library is taken from the arrays that were uploaded."""
    batch, m, k = a.shape
    n = b.shape[-1]
    flat_a, lda = _laid_out(a, pad[0], offset[0])
    bb = b[:1] if shared_b else b
    flat_b, ldb = _laid_out(np.ascontiguousarray(bb.transpose(0, 2, 1)) if trans_b else bb, pad[1], offset[1])
    da, db, dc = ctx.upload(flat_a), ctx.upload(flat_b), ctx.alloc(batch * m * n * 4)
    try:
        assert flat_a.size >= offset[0] + (batch - 1) * m * lda + (m - 1) * lda + k
        rows_b = n if trans_b else k
        assert flat_b.size >= offset[1] + ((0 if shared_b else batch - 1) * rows_b + rows_b - 1) * ldb + (k if trans_b else n)
        ctx.gemm_raw(dc.ptr, da.ptr + 4 * offset[0], db.ptr + 4 * offset[1], None, batch, m, n, k, trans_b=trans_b, lda=lda, ldb=ldb,
                     a_bs=m * lda, b_bs=0 if shared_b else rows_b * ldb, c_bs=m * n)
        return ctx.download(dc, (batch, m, n))
    finally:
        for x in (da, db, dc):
            ctx.free(x)


# batch, m, n, k: the shapes that take the kernels of many small products (128 or more products, m <= 208 and either
# k <= 64 and n <= 208 or n <= 64), at their limits, and their neighbours that do not
MANY_SMALL = [(144, 197, 197, 64), (144, 197, 64, 197), (128, 208, 208, 64), (300, 197, 197, 64), (300, 197, 64, 197), (128, 1, 1, 1),
              (129, 33, 7, 3), (130, 193, 190, 33), (128, 100, 17, 64), (128, 208, 64, 300), (128, 30, 64, 65), (130, 16, 16, 1000),
              (128, 192, 48, 128), (128, 209, 64, 64), (128, 197, 209, 64), (127, 197, 197, 64), (128, 64, 65, 65),
              (128, 50, 20, 97), (128, 197, 64, 130), (128, 17, 33, 81), (128, 40, 64, 113)]  # k cut into chunks of 64+48, 48+48+48, 48+48, 64+64


@pytest.mark.parametrize("batch,m,n,k", MANY_SMALL)
def test_many_small_products(ctx, case, batch, m, n, k):
    case(f"{batch} products [{m},{k}] x [{k},{n}]")
    a, b = ints(batch, m, k), ints(batch, k, n)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64)).astype(np.float32)
    got = {}
    for trans_b in (False, True):
        got[trans_b] = _many_small(ctx, a, b, trans_b)
        assert_bits_equal(got[trans_b], want, f"integer operands, trans_b={trans_b}")
    # rows that are no whole float4s and bases off the 16-byte grid: the single-value loads
    assert_bits_equal(_many_small(ctx, a, b, False, pad=(1, 3), offset=(1, 2)), want, "odd pitches and bases")
    assert_bits_equal(_many_small(ctx, a, b, True, pad=(3, 1), offset=(3, 1)), want, "odd pitches and bases, trans_b")
    assert_bits_equal(_many_small(ctx, a, b[:1].repeat(batch, 0), False, shared_b=True),
                      np.matmul(a.astype(np.float64), b[:1].astype(np.float64)).astype(np.float32), "one B for every product")
    a, b = RNG.standard_normal(a.shape).astype(np.float32), RNG.standard_normal(b.shape).astype(np.float32)
    r0, r1 = _many_small(ctx, a, b, False), _many_small(ctx, a, b, True)
    check_bound(r0, a, b, "random operands")
    # a product and the same product through the other layout of B add the same numbers in the same order
    assert_bits_equal(r1, r0, "B stored [n, k] against B stored [k, n]")
    assert_bits_equal(_many_small(ctx, a, b, True, pad=(1, 2), offset=(2, 3)), r0, "padded, offset operands against dense ones")


def test_many_small_products_land_in_their_places(ctx, case):
    """Every (head, row, column) gets its own value: a tile written to the wrong head, row or column shows."""
    case("placement of 300 x [197,64] x [64,197] and 300 x [197,197] x [197,64]")
    batch, m = 300, 197
    for n, k in ((197, 64), (64, 197)):
        a = np.zeros((batch, m, k), np.float32)
        b = np.zeros((batch, k, n), np.float32)
        p = np.arange(batch) % k                      # head z multiplies through k = z % k only
        a[np.arange(batch), :, p] = np.arange(1, m + 1)[None, :] + 256.0 * (np.arange(batch) % 7)[:, None]
        b[np.arange(batch), p, :] = np.arange(1, n + 1)[None, :] * 2048.0
        want = a[np.arange(batch), :, p][:, :, None] * b[np.arange(batch), p, :][:, None, :]
        for trans_b in (False, True):
            assert_bits_equal(_many_small(ctx, a, b, trans_b), want.astype(np.float32), f"n={n} k={k} trans_b={trans_b}")
