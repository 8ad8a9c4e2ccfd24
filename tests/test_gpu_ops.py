"""Parity of the HIP kernels with the CPU oracle, called through the C ABI.

Bars (BASELINE.json): bit-exact for Add/Sub/Mul/Div, Sqrt, Relu, HardSigmoid,
Pow(x, 2), ReduceMax and all broadcast indexing; 1e-5 relative / 1e-6 absolute
for everything whose row sums are accumulated in a different order than the
reference's 8-lane accumulators (Softmax, LayerNormalization, ReduceMean).
The element-wise approximations (Gelu, Sigmoid, Erf) are deterministic
per-element formulas and are held to bit equality as well.
"""
import numpy as np
import pytest

from altius_amd import device as D
from altius_amd import synth
from altius_amd._lib import ERR_ARG, ERR_UNSUPPORTED, AltiusHipError
from conftest import assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu

BIN = {"Add": (D.ADD, 0), "Sub": (D.SUB, 1), "Mul": (D.MUL, 2), "Div": (D.DIV, 3)}

# Shape pairs of the reference's own binary-op tests
# (crates/altius_py/tests/test_ops_bin.py:11-140, crates/session_interpreter/tests/op_bin.rs:62-76)
# plus the benchmark configurations' broadcast patterns at reduced batch.
BIN_SHAPES = [
    ([1, 2], [1, 2]),
    ([3, 1, 10], [3, 1, 10]),
    ([1, 2, 3, 4, 5, 6, 7], [1, 2, 3, 4, 5, 6, 7]),
    ([16, 3, 224, 224], [16, 3, 224, 224]),
    ([1, 3, 28, 28], [3, 1, 1]),
    ([1, 12, 9, 9], [1, 1, 1, 9]),
    ([4, 1, 2], [3, 1]),
    ([3, 28, 28], [3, 28, 1]),
    ([3, 15, 15], [15]),
    ([3, 28, 28], [1]),
    ([1], [3, 28, 28]),
    ([3, 28, 28], []),
    ([1, 197, 768], [768]),            # cfg0
    ([4, 12, 197, 197], [4, 1, 1, 197]),  # cfg4 mask pattern
    ([8, 197, 768], [8, 197, 1]),      # cfg2 Sub/Div
    ([8, 576, 7, 7], [8, 576, 1, 1]),  # cfg3 squeeze-excite
    ([5, 1, 7, 1, 3], [1, 6, 1, 2, 3]),  # two-sided, rank 5
    ([2, 3, 4, 5, 6, 7], [7]),
    ([1, 1, 1], [1]),
    ([7], [7]),
    ([1023], [1023]),
    ([2, 0, 3], [3]),                  # empty
    ([3, 40, 30], [3, 1, 30]),         # row broadcast staged in LDS, blocks spanning two outer indices
    ([3, 1, 30], [3, 40, 30]),         # the same with the operands swapped
    ([5, 2, 6], [5, 1, 6]),            # row broadcast too short for the LDS kernel
    ([2, 3, 1031], [1031]),            # bias with an odd length
    ([7, 5], [5]),
    # rows of whole float4s with a vector along the row or one value per row (two-axis kernel), both operand orders
    ([8, 197, 768], [768]),
    ([768], [8, 197, 768]),
    ([8, 197, 1], [8, 197, 768]),
    ([33, 1028], [1028]),              # last block partly filled
    ([33, 1028], [33, 1]),
    ([3, 5, 4], [3, 5, 1]),
    ([1, 4], [3, 5, 4]),
    ([64, 197, 3072], [3072]),         # above the size at which accesses become non-temporal
    ([64, 197, 3072], [64, 197, 1]),
    # the same kernel's three-axis forms: one vector per outer index, one value per channel
    ([2, 4, 10, 1028], [2, 1, 1, 1028]),  # a mask on rows too long for the kernel that stages it in LDS
    ([2, 1, 1, 1028], [2, 4, 10, 1028]),
    ([2, 3, 8, 8], [3, 1, 1]),           # per-channel bias on NCHW
    ([1, 3, 1, 1], [2, 3, 8, 8]),
    ([4, 6, 4, 4], [4, 6, 1, 1]),        # squeeze-excite gate
    ([5, 7, 2, 6], [7, 1, 1]),
    ([128, 96, 56, 56], [96, 1, 1]),     # non-temporal variant
    # one value per row or channel on rows that are not whole float4s (lanes straddling two rows, ragged end)
    ([5, 7, 3, 3], [7, 1, 1]),
    ([7, 1, 1], [5, 7, 3, 3]),
    ([3, 5, 7], [3, 5, 1]),
    ([2, 3, 5], [3, 1]),
    ([3, 5, 1], [3, 5, 7]),
    ([9, 4], [9, 1]),
    ([64, 576, 7, 7], [576, 1, 1]),
    ([768, 1024, 7, 7], [768, 1024, 1, 1]),  # non-temporal variant
    # a vector of two or three values (an RGB mean on NHWC): a lane's four elements cycle through it
    ([5, 67, 3], [3]),
    ([3], [2, 224, 224, 3]),
    ([333, 2], [2]),
    ([4096, 4096, 3], [3]),              # non-temporal variant
]


@pytest.mark.parametrize("name", list(BIN))
@pytest.mark.parametrize("sa,sb", BIN_SHAPES)
def test_binary_bit_exact(ctx, oracle, case, name, sa, sb):
    case(f"binary {name} {sa} {sb}")
    op, oop = BIN[name]
    a = synth.uniform(11, sa) + np.float32(0.25)
    b = synth.uniform(12, sb) + np.float32(0.25)
    expected = oracle.binary(oop, a, b)
    actual = ctx.binary(op, a, b)
    assert_bits_equal(actual, expected, f"{name} {sa} {sb}")
    # The oracle itself agrees with numpy's IEEE arithmetic and broadcasting.
    ref = {"Add": a + b, "Sub": a - b, "Mul": a * b, "Div": a / b}[name]
    assert_bits_equal(expected, ref.astype(np.float32), f"oracle vs numpy {name}")


@pytest.mark.parametrize("threshold", [0, 2**64 - 1])
def test_streamed_loads_change_no_bit(oracle, case, threshold):
    """Dense operands of at least `ahip_set_load_streaming_threshold` bytes are read with non-temporal loads while the
    result is stored the ordinary way: the same values either way, for every element-wise kernel that has the variant
    (flat, a row staged in LDS, a vector / column beside rows of float4s, unary)."""
    case(f"element-wise operators with the load streaming threshold at {threshold}")
    c = D.Context(0)
    try:
        c.set_load_streaming_threshold(threshold)
        for sa, sb in [([3, 1, 10], [3, 1, 10]), ([16, 3, 224, 224], [16, 3, 224, 224]), ([3, 28, 28], []), ([4, 12, 197, 197], [4, 1, 1, 197]),
                       ([3, 1, 30], [3, 40, 30]), ([8, 197, 768], [768]), ([8, 197, 1], [8, 197, 768]), ([2, 3, 8, 8], [3, 1, 1]),
                       ([2, 4, 10, 1028], [2, 1, 1, 1028])]:
            a = synth.uniform(21, sa) + np.float32(0.25)
            b = synth.uniform(22, sb) + np.float32(0.25)
            for name, (op, oop) in BIN.items():
                assert_bits_equal(c.binary(op, a, b), oracle.binary(oop, a, b), f"{name} {sa} {sb} threshold {threshold}")
        x = synth.normal(23, [4, 197, 3072], std=2.0)
        for name, (op, oop) in UNARY.items():
            v = np.abs(x) if name == "Sqrt" else x
            alpha, beta = (1.0 / 6.0, 0.5) if name == "HardSigmoid" else (0.0, 0.0)
            assert_bits_equal(c.unary(op, v, alpha, beta), oracle.unary(oop, v, alpha, beta), f"{name} threshold {threshold}")
    finally:
        c.close()


def test_binary_known_answer(ctx, case):
    """[1,3,...,15] + [2,4,...,16] = [3,7,...,31] (crates/session/tests/ort.rs:17-25)."""
    case("binary KAT")
    a = np.arange(1, 16, 2, dtype=np.float32)
    b = np.arange(2, 17, 2, dtype=np.float32)
    assert ctx.binary(D.ADD, a, b).tolist() == [3, 7, 11, 15, 19, 23, 27, 31]


def test_binary_special_values(ctx, oracle, case):
    case("binary special values")
    s = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, 1e-38, 2.5],
                 dtype=np.float32)
    a = np.repeat(s, len(s)).reshape(len(s), len(s))
    b = np.tile(s, len(s)).reshape(len(s), len(s))
    for name, (op, oop) in BIN.items():
        with np.errstate(all="ignore"):
            assert_bits_equal(ctx.binary(op, a, b), oracle.binary(oop, a, b), f"special {name}")


def test_binary_unaligned_pointers(ctx, oracle, case):
    """Operands at addresses that are not 16-byte aligned take the scalar kernels."""
    case("binary unaligned")
    n = 4099
    a = synth.normal(21, (n + 1,))
    b = synth.normal(22, (n + 3,))
    da, db = ctx.upload(a), ctx.upload(b)
    do = ctx.alloc((n + 1) * 4)
    ctx.binary_raw(D.MUL, do.ptr + 4, da.ptr + 4, db.ptr + 12, [n], [1], [1])
    got = ctx.download(do, (n,), offset_bytes=4)
    assert_bits_equal(got, a[1:] * b[3:], "unaligned flat")
    # strided with unaligned pieces: [17, 5] * [5]
    x = synth.normal(23, (17 * 5 + 1,))
    y = synth.normal(24, (5 + 1,))
    dx, dy = ctx.upload(x), ctx.upload(y)
    ctx.binary_raw(D.ADD, do.ptr + 4, dx.ptr + 4, dy.ptr + 4, [17, 5], [5, 1], [0, 1])
    got = ctx.download(do, (17, 5), offset_bytes=4)
    assert_bits_equal(got, x[1:].reshape(17, 5) + y[1:], "unaligned strided")
    for t in (da, db, do, dx, dy):
        ctx.free(t)


def test_binary_broadcast_mismatch_is_an_error(ctx, case):
    """[1,3,28,28] + [3,1,2] cannot broadcast (test_ops_bin.py:31-40): an error value, not an abort."""
    case("binary mismatch")
    from altius_amd._lib import AltiusHipError, ERR_SHAPE

    with pytest.raises(AltiusHipError) as e:
        ctx.binary(D.ADD, np.zeros([1, 3, 28, 28], np.float32), np.zeros([3, 1, 2], np.float32))
    assert e.value.code == ERR_SHAPE


@pytest.mark.parametrize("sa,sb", [([1, 2], [1, 2]), ([1, 2, 3, 4, 5, 6, 7], [1, 2, 3, 4, 5, 6, 7]),
                                   ([128, 3, 8, 8], [128, 3, 8, 8]), ([128, 3, 8, 8], [1]),
                                   ([8, 197, 768], [])])
def test_pow(ctx, oracle, case, sa, sb):
    """Pow shapes of test_ops_bin.py:123-140.  powf is a libm call on both sides."""
    case(f"pow {sa} {sb}")
    a = synth.uniform(31, sa) + np.float32(0.5)
    b = synth.uniform(32, sb) * np.float32(3.0)
    assert_close(ctx.binary(D.POW, a, b), oracle.binary(4, a, b), what=f"pow {sa} {sb}")


def test_pow_square_is_exact(ctx, oracle, case):
    """Pow(x, 2) with a scalar exponent is x*x (session.rs:588-591): bit-exact."""
    case("pow square")
    x = synth.normal(33, (8, 197, 768))
    for two in (np.array(2.0, np.float32), np.array([2.0], np.float32)):
        got = ctx.binary(D.POW, x, two)
        assert_bits_equal(got, x * x, "pow(x,2)")
        assert_bits_equal(got, oracle.binary(4, x, two), "pow(x,2) vs oracle")


UNARY = {
    "Sqrt": (D.SQRT, 0),
    "Erf": (D.ERF, 1),
    "Gelu": (D.GELU, 2),
    "Sigmoid": (D.SIGMOID, 3),
    "HardSigmoid": (D.HARDSIGMOID, 4),
    "Relu": (D.RELU, 5),
    "Tanh": (D.TANH, 6),
}


@pytest.mark.parametrize("name", list(UNARY))
@pytest.mark.parametrize("shape", [[1, 2], [3, 1, 28, 28], [3, 1, 7, 7], [1, 2, 3], [4, 197, 3072], [1], [0], [4097]])
def test_unary_bit_exact(ctx, oracle, case, name, shape):
    """Shapes of crates/altius_py/tests/test_ops_elemwise.py:22-152 plus cfg3 at reduced batch."""
    case(f"unary {name} {shape}")
    op, oop = UNARY[name]
    x = synth.normal(41, shape, std=2.0)
    if name == "Sqrt":
        x = np.abs(x)
    alpha, beta = (1.0 / 6.0, 0.5) if name == "HardSigmoid" else (0.0, 0.0)
    expected = oracle.unary(oop, x, alpha, beta)
    actual = ctx.unary(op, x, alpha, beta)
    assert_bits_equal(actual, expected, f"{name} {shape}")


@pytest.mark.parametrize("name", list(UNARY))
def test_unary_special_values(ctx, oracle, case, name):
    case(f"unary special {name}")
    op, oop = UNARY[name]
    x = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4e38, -3.4e38, 1e-38,
                  88.0, -88.0, 89.0, -104.0, 104.0, 9.0, -9.0, 10.0, 38.0, 39.0, 50.0, -50.0, 0.5, 6.0, -6.0],
                 dtype=np.float32)
    with np.errstate(all="ignore"):
        expected = oracle.unary(oop, x, 0.2, 0.5)
    actual = ctx.unary(op, x, 0.2, 0.5)
    # Relu of -0.0: the reference leaves the sign of the zero unspecified.
    assert_bits_equal(actual, expected, f"special {name}", zero_sign_free=(name == "Relu"))


def test_erf_against_the_exact_interpolant(ctx, case):
    """Op::Erf without the oracle: fastapprox::faster::erf (session.rs:929) restated as the exact
    piecewise-linear interpolant of 2^t in rational arithmetic (tests/erf_exact.py), over every
    branch of the bit trick: the clip, subnormals, the exponent-255 segment, the wrap into the sign
    bit, the saturated cast, NaN and infinities."""
    import erf_exact

    case("erf vs exact interpolant")
    x = erf_exact.erf_vectors()
    want = erf_exact.erf_expected(x)
    got = ctx.unary(D.ERF, x)
    assert_bits_equal(got, want, "erf vs interpolant")
    assert ctx.unary(D.ERF, np.float32([np.nan]))[0] == -1.0  # Rust's `as u32` turns NaN into 0
    assert ctx.unary(D.ERF, np.float32([50.0]))[0] == -1.0    # the exponent field wraps into the sign bit


def test_hardsigmoid_default_attributes(ctx, oracle, case):
    """ONNX defaults alpha=0.2, beta=0.5 (crates/core/src/onnx/load.rs:321-324)."""
    case("hardsigmoid defaults")
    x = synth.normal(42, (3, 1, 28, 28), std=3.0)
    got = ctx.unary(D.HARDSIGMOID, x, 0.2, 0.5)
    assert_bits_equal(got, oracle.unary(4, x, 0.2, 0.5), "hardsigmoid")
    exact = np.clip(np.float64(np.float32(0.2)) * x.astype(np.float64) + 0.5, 0, 1).astype(np.float32)
    assert_bits_equal(got, exact, "hardsigmoid vs float64 fma")


SOFTMAX_SHAPES = [[1, 2, 3], [3, 28, 28], [16, 512, 512], [2, 12, 197, 197], [5, 1], [7, 64], [3, 65], [9, 256],
                  [3, 1000], [2, 1024], [3, 1025], [2, 4096], [2, 5000], [1, 70001],
                  [3, 1028], [5, 1280], [9, 1536], [3, 2048], [2, 2560], [4, 3072], [2, 4092], [2, 4100],  # rows of 1025..4096 whole float4s stay in registers
                  [2, 5120], [3, 8192], [2, 8196], [2, 16384], [1, 12000], [2, 16388], [2, 5001],  # up to 16384: in a block's registers
                  [3, 1284], [3, 2052], [2, 3076], [2, 4608], [2, 6144], [2, 6148], [2, 12288],  # either side of every block width
                  [5, 384], [7, 640], [6, 896], [3, 1088], [9, 1152], [13, 320],  # a wavefront per row, last chunk partly filled
                  [7, 1030], [5, 2049], [3, 4097], [3, 9999], [2, 16381], [2, 16383], [2, 50257],  # rows that start anywhere: the aligned cover of a row in registers
                  [2, 6147], [2, 6149], [2, 7001], [2, 12291], [2, 12293], [2, 24579], [1, 32771], [1, 36001], [1, 40961],  # either side of each step in its float4 per thread
                  [2, 20000], [2, 32768], [1, 49152], [2, 65536], [2, 30522], [1, 65533], [1, 65540],  # 6 to 16 float4 per thread up to 65536 elements, three passes above
                  [9, 1026], [6, 1281], [7, 1535], [5, 1537], [5, 1793], [4, 2047], [3, 2050],  # rows that start anywhere, a wavefront per row: 5 to 8 float4 per lane
                  [2, 49156], [1, 52000], [2, 53248], [1, 53245], [1, 53249]]  # thirteen float4 per thread, and just past them


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
def test_softmax(ctx, oracle, case, shape):
    """Shapes of test_ops_elemwise.py:107-126 plus row lengths around every kernel boundary."""
    case(f"softmax {shape}")
    x = synth.normal(51, shape)
    got = ctx.softmax(x)
    assert_close(got, oracle.softmax(x), what=f"softmax {shape}")
    np.testing.assert_allclose(got.sum(-1, dtype=np.float64), 1.0, atol=2e-6)


def test_softmax_masked_rows(ctx, oracle, case):
    """cfg4: scores + mask(-1e4) then Softmax; masked entries underflow to exact zeros or denormals."""
    case("softmax masked")
    c = synth.cfg4(batch=2)
    z = c["scores"] + c["mask"]
    got = ctx.softmax(z)
    exp = oracle.softmax(z)
    assert_close(got, exp, what="masked softmax")
    masked = np.broadcast_to(c["mask"], z.shape) != 0
    assert masked.any() and np.all(got[masked] < 1e-30)
    # Fully masked and constant rows, huge and tiny magnitudes, NaN in a row.
    x = np.zeros((6, 197), np.float32)
    x[0] = -1e4
    x[1] = 3.0
    x[2, ::2] = 1e30
    x[3, 5] = -np.inf
    x[4] = synth.normal(52, (197,)) * 1e-30
    x[5, 7] = np.nan
    with np.errstate(all="ignore"):
        assert_close(ctx.softmax(x), oracle.softmax(x), what="softmax edge rows")


LN_SHAPES = [[1, 20, 10], [2, 197, 768], [3, 5, 197], [4, 1], [5, 64], [3, 1024], [2, 1028], [2, 4100], [3, 3072],
             [5, 1280], [9, 1536], [3, 2048], [2, 2560], [2, 4092], [7, 4096], [2, 1026],
             [100, 49], [70, 197], [300, 64], [1000, 10], [64, 255], [65, 1], [200, 130], [4, 700, 192],  # short rows in groups through LDS
             [2, 5120], [3, 8192], [2, 8196], [2, 16384], [1, 12000], [2, 16388], [2, 5001],  # rows up to 16384 in a block's registers
             [3, 1284], [3, 2052], [2, 3076], [2, 4608], [2, 6144], [2, 6148], [2, 12288],  # either side of every block width
             [5, 384], [7, 640], [6, 896], [3, 1088], [9, 1152], [1, 512], [13, 320],  # a wavefront per row, last chunk partly filled, rows not a multiple of the block's four
             [7, 1030], [5, 2049], [3, 4097], [3, 9999], [2, 16383], [2, 50257],  # rows that start anywhere: the aligned cover of a row in registers
             [2, 6147], [2, 6149], [2, 9219], [2, 9221], [2, 13315], [2, 13317], [2, 18435], [2, 18437],  # either side of each step in its float4 per thread
             [2, 24579], [2, 24581], [1, 32771], [1, 32773], [1, 36001], [1, 40961],
             [2, 20000], [2, 32768], [1, 49152], [2, 65536], [2, 30522], [1, 65533], [1, 65540],  # 6 to 16 float4 per thread up to 65536 elements, three passes above
             [9, 1025], [6, 1281], [7, 1535], [5, 1537], [5, 1793], [4, 2047], [3, 2050],  # rows that start anywhere, a wavefront per row: 5 to 8 float4 per lane
             [2, 49156], [1, 52000], [2, 53248], [1, 53245], [1, 53249]]  # thirteen float4 per thread, and just past them


@pytest.mark.parametrize("shape", LN_SHAPES)
def test_layernorm(ctx, oracle, case, shape):
    """[1,20,10] is the reference's test (crates/altius_py/tests/test_ops_norm.py:16-18)."""
    case(f"layernorm {shape}")
    x = synth.normal(61, shape, mean=0.3, std=1.7)
    g = synth.normal(62, (shape[-1],), mean=1.0, std=0.02)
    b = synth.normal(63, (shape[-1],), mean=0.0, std=0.02)
    got = ctx.layer_norm(x, g, b, 1e-5)
    assert_close(got, oracle.layer_norm(x, g, b, 1e-5), what=f"layernorm {shape}")
    # and the textbook formula at the reference's own tolerance (test_ops_norm.py:86)
    xd = x.astype(np.float64)
    ref = (xd - xd.mean(-1, keepdims=True)) / np.sqrt(xd.var(-1, keepdims=True) + 1e-5) * g + b
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("off", [1, 2, 3])
def test_flat_operators_on_large_views_that_start_off_a_boundary(ctx, oracle, case, off):
    """Every tensor `off` floats past a 16-byte boundary: four elements per lane through 16-byte accesses that are only
    4-byte aligned; not a bit may differ from the aligned call."""
    case(f"Gelu / Add / Mul by a scalar / Sub from a scalar on 70001 elements, every tensor +{off} floats")
    n = 70001
    a, b = synth.normal(81, (n + off,)), synth.normal(82, (n + off,), mean=2.0)
    da, db = ctx.upload(a), ctx.upload(b)
    do = ctx.alloc((n + 4) * 4)
    ds = ctx.upload(np.array([1.7], np.float32))
    pa, pb, po = da.ptr + 4 * off, db.ptr + 4 * off, do.ptr + 4 * off
    ctx.unary_raw(D.GELU, po, pa, n)
    assert_bits_equal(ctx.download(do, (n,), offset_bytes=4 * off), oracle.unary(oracle.GELU, a[off:]), "Gelu")
    ctx.binary_raw(D.ADD, po, pa, pb, [n], [1], [1])
    assert_bits_equal(ctx.download(do, (n,), offset_bytes=4 * off), a[off:] + b[off:], "Add")
    ctx.binary_raw(D.MUL, po, pa, ds.ptr, [n], [1], [0])
    assert_bits_equal(ctx.download(do, (n,), offset_bytes=4 * off), a[off:] * np.float32(1.7), "Mul by a scalar")
    ctx.binary_raw(D.SUB, po, ds.ptr, pb, [n], [0], [1])
    assert_bits_equal(ctx.download(do, (n,), offset_bytes=4 * off), np.float32(1.7) - b[off:], "Sub from a scalar")
    for t in (da, db, do, ds):
        ctx.free(t)


UNALIGNED_ROWS = [(7, 768), (5, 197), (3, 1280), (2, 4096), (2, 8192), (3, 1000), (9, 64), (5, 2048), (6, 1500), (2, 51200)]


@pytest.mark.parametrize("rows,length", UNALIGNED_ROWS)
@pytest.mark.parametrize("in_off,out_off", [(1, 0), (0, 3), (2, 2)])
def test_row_and_unary_operators_on_unaligned_pointers(ctx, oracle, case, rows, length, in_off, out_off):
    """The reference's tensors are plain slices of floats: nothing promises 16-byte alignment.  Input and output start
    in_off / out_off floats past an aligned address (other kernels take such calls, with their own order of summation,
    so the sums are checked against the oracle, not against the aligned call's bits)."""
    case(f"Softmax / LayerNormalization / ReduceMean / ReduceMax / Gelu on [{rows},{length}], input +{in_off} floats, output +{out_off}")
    x = synth.normal(71, (rows, length), mean=0.2, std=1.5)
    g = synth.normal(72, (length,), mean=1.0, std=0.05)
    b = synth.normal(73, (length,), mean=0.0, std=0.05)
    n = rows * length
    pad = np.zeros(in_off, np.float32)
    dx = ctx.upload(np.concatenate([pad, x.ravel()]))
    dg, db = ctx.upload(np.concatenate([pad, g])), ctx.upload(np.concatenate([pad, b]))
    do = ctx.alloc((n + 4) * 4)
    px, pg, pb, po = dx.ptr + 4 * in_off, dg.ptr + 4 * in_off, db.ptr + 4 * in_off, do.ptr + 4 * out_off
    ctx.softmax_raw(po, px, rows, length)
    assert_close(ctx.download(do, (rows, length), offset_bytes=4 * out_off), oracle.softmax(x), what="Softmax")
    ctx.layernorm_raw(po, px, pg, pb, rows, length, 1e-5)
    assert_close(ctx.download(do, (rows, length), offset_bytes=4 * out_off), oracle.layer_norm(x, g, b, 1e-5), what="LayerNormalization")
    ctx.reduce_raw(D.REDUCE_MEAN, po, px, rows, length, 1)
    assert_close(ctx.download(do, (rows, 1), offset_bytes=4 * out_off), oracle.reduce(oracle.REDUCE_MEAN, x, [1], True), what="ReduceMean")
    ctx.reduce_raw(D.REDUCE_MAX, po, px, 1, rows, length)
    assert_bits_equal(ctx.download(do, (1, length), offset_bytes=4 * out_off), x.max(0, keepdims=True), "ReduceMax over rows")
    ctx.unary_raw(D.GELU, po, px, n)
    assert_bits_equal(ctx.download(do, (rows, length), offset_bytes=4 * out_off), oracle.unary(oracle.GELU, x), "Gelu")
    for t in (dx, dg, db, do):
        ctx.free(t)


# More rows than blocks fit the device, of lengths that take 1024 threads: the kernels that request a row ahead.
MANY_LONG_ROWS = [(1100, 5120), (1029, 6144), (1500, 8192), (1031, 8196), (1100, 12288), (1111, 16384), (1040, 16380), (2100, 5004)]


@pytest.mark.parametrize("rows,length", MANY_LONG_ROWS)
def test_softmax_and_layernorm_of_many_long_rows(ctx, oracle, case, rows, length):
    """The same rows a few at a time go through the kernels that hold one row per block and launch: not a bit may
    differ.  Against the oracle on the first, the last and some rows between, a NaN and an all-equal row among them."""
    case(f"softmax / layernorm of {rows} rows of {length}")
    x = synth.normal(71, (rows, length), mean=0.2, std=1.5)
    x[3, 17] = np.nan
    x[rows - 1] = 2.5
    x[5, ::3] = -1e4
    g = synth.normal(72, (length,), mean=1.0, std=0.02)
    b = synth.normal(73, (length,), mean=0.0, std=0.02)
    pick = np.r_[0:8, rows // 2 : rows // 2 + 4, rows - 6 : rows]
    with np.errstate(all="ignore"):
        got = ctx.softmax(x)
        few = np.concatenate([ctx.softmax(x[i : i + 500]) for i in range(0, rows, 500)])
        assert_bits_equal(got, few, "softmax: many rows vs a few at a time")
        assert_close(got[pick], oracle.softmax(x[pick]), what="softmax of many long rows")
        got = ctx.layer_norm(x, g, b, 1e-5)
        few = np.concatenate([ctx.layer_norm(x[i : i + 500], g, b, 1e-5) for i in range(0, rows, 500)])
        assert_bits_equal(got, few, "layernorm: many rows vs a few at a time")
        assert_close(got[pick], oracle.layer_norm(x[pick], g, b, 1e-5), what="layernorm of many long rows")


@pytest.mark.parametrize("rows,length", [(40001, 197), (36 * 1100 + 7, 193), (12000, 700), (9003, 900), (33000, 205)])
def test_softmax_of_many_rows_in_wide_groups(ctx, oracle, case, rows, length):
    """Rows whose smallest line-aligned group takes the wide block, tens of thousands of them: not a bit may differ
    from the same rows a few thousand at a time, with the scale and mask prologue and without; ragged last groups,
    row counts that are not whole float4s in total."""
    case(f"softmax of {rows} rows of {length}")
    x = synth.normal(81, (rows, length), std=2.0)
    x[11, 5] = np.nan
    x[rows - 1] = -3.0
    with np.errstate(all="ignore"):
        got = ctx.softmax(x)
        few = np.concatenate([ctx.softmax(x[i : i + 3000]) for i in range(0, rows, 3000)])
        assert_bits_equal(got, few, "softmax: all rows vs a few thousand at a time")
        pick = np.r_[0:16, rows // 2 : rows // 2 + 8, rows - 8 : rows]
        assert_close(got[pick], oracle.softmax(x[pick]), what="softmax of many rows")
        per_mask = 1000 if rows % 1000 == 0 else 3 if rows % 3 == 0 else 1
        mask = np.where(synth.normal(82, (rows // per_mask, length)) > 1.2, np.float32(-1e4), np.float32(0))
        fused = ctx.softmax_prologue(x, 2, 8.0, mask)
        z = x / np.float32(8.0) + np.repeat(mask, per_mask, axis=0)
        assert_bits_equal(fused, ctx.softmax(z), "prologue vs the operators")


REDUCE_CASES = [
    # (shape, axes, keepdims)
    ([1, 50, 70], [-1], True),         # test_ops_reduce.py:10-18
    ([8, 4, 5, 5], [2, 3], True),      # test_ops_reduce.py:21-30
    ([8, 197, 768], [-1], True),       # cfg2
    ([8, 576, 7, 7], [2, 3], True),    # cfg3 squeeze-excite
    ([4, 768, 197], [1], False),       # cfg4 pattern
    ([4, 768, 197], [1], True),
    ([3, 10, 5000], [2], True),        # long rows, wave path limit
    ([2, 3, 70000], [2], False),       # long rows, block path
    ([1, 2000000], [1], False),        # split rows through scratch
    ([5, 33, 2], [1], False),          # narrow inner
    ([2, 100, 300], [1], False),       # several column tiles
    ([2, 4000, 64], [1], False),       # split columns through scratch
    ([7, 1, 9], [1], True),
    ([70, 197], [1], False),           # short / unaligned rows staged through LDS in groups: a ragged last group
    ([3000, 1], [1], True),            # rows of one element
    ([100, 1001], [1], False),         # 64 lanes per row
    ([500, 333], [1], True),           # 32 lanes per row
    ([2, 999, 7, 7], [2, 3], True),    # 16 lanes per row, several groups
    ([4096, 64], [1], False),          # short aligned rows
    ([6, 5], [0], False),
    ([1, 18, 197], [1], False),        # 16-byte flat column kernel with two left-over rows
    ([1, 17, 5], [1], False),          # the same, one left-over row, one wave of columns
    ([2, 100, 30], [1], True),         # flat kernel, aligned slabs
    ([3, 17, 5], [1], False),          # unaligned slabs: dword column kernel
    ([2, 2049, 255], [1], False),      # flat kernel split over blocks, odd row count
    ([300, 64, 6], [1], False),
    ([3, 640, 7], [1], False),         # span kernel, one float4 step per thread
    ([1, 4099, 33], [1], False),       # span kernel split over blocks, three left-over rows
    ([2, 130, 1023], [1], True),       # span kernel at its widest (four float4 steps per thread)
    ([5, 197, 768], [1], False),       # float4 columns, three tiles of 64 per slab (mean over tokens)
    ([9, 49, 1024], [1], True),        # the same, few rows per wavefront
    ([3, 1000, 8], [1], False),        # float4 columns, 32 rows per wavefront pass
    ([7, 333, 100], [1], False),       # 25 float4 per row: two rows per pass, 14 lanes idle
    ([2, 70, 260], [1], False),        # a second tile of one float4 column
    ([1, 5000, 256], [1], False),      # float4 columns, the reduced axis split over blocks through scratch
    ([11, 2, 4096], [1], False),       # two to four rows of many columns: a thread per float4 column
    ([5, 3, 260], [1], True),
    ([40, 4, 256], [1], False),
    ([1000, 7, 7], [1], False),        # small slabs staged through LDS in groups, a thread per output value
    ([333, 196, 3], [1], True),
    ([4099, 3, 4], [1], False),        # whole float4s, but too few rows for the float4-column kernel
    ([10001, 2, 3], [1], False),       # groups of 1364 slabs, a ragged last group
    ([3, 100, 20], [1], False),        # slabs of 2000 values: groups of four, the last one of three
    ([50, 64, 5], [1], False),         # few outputs per group: eight threads share a column, then three, then two
    ([7, 131, 20], [1], True),
    ([9, 9, 6], [1], False),
    ([3000, 196, 3], [1], False),      # groups of twelve slabs, seven threads per output
    ([7, 1030], [1], False),           # rows that start anywhere: single elements to the first 16-byte boundary, then float4s
    ([5, 2049], [1], True),
    ([3, 5001], [1], False),           # the same in the block kernel
    ([2, 50257], [1], False),
    ([1, 3, 70001], [2], False),
]


@pytest.mark.parametrize("shape,axes,keep", REDUCE_CASES)
def test_reduce_mean(ctx, oracle, case, shape, axes, keep):
    case(f"reduce_mean {shape} {axes}")
    x = synth.normal(71, shape, mean=0.5)
    exp = oracle.reduce(0, x, axes, keep)
    ax = sorted(a % len(shape) for a in axes)
    outer = int(np.prod(shape[:ax[0]], dtype=np.int64))
    red = int(np.prod(shape[ax[0]:ax[-1] + 1], dtype=np.int64))
    inner = int(np.prod(shape[ax[-1] + 1:], dtype=np.int64))
    got = ctx.reduce(D.REDUCE_MEAN, x, outer, red, inner).reshape(exp.shape)
    assert_close(got, exp, what=f"reduce_mean {shape}")
    np.testing.assert_allclose(got, x.astype(np.float64).mean(tuple(ax), keepdims=keep), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("shape,axes,keep", REDUCE_CASES)
def test_reduce_max_bit_exact(ctx, oracle, case, shape, axes, keep):
    case(f"reduce_max {shape} {axes}")
    x = synth.normal(72, shape)
    exp = oracle.reduce(1, x, axes, keep)
    ax = sorted(a % len(shape) for a in axes)
    outer = int(np.prod(shape[:ax[0]], dtype=np.int64))
    red = int(np.prod(shape[ax[0]:ax[-1] + 1], dtype=np.int64))
    inner = int(np.prod(shape[ax[-1] + 1:], dtype=np.int64))
    got = ctx.reduce(D.REDUCE_MAX, x, outer, red, inner).reshape(exp.shape)
    assert_bits_equal(got, exp, f"reduce_max {shape}")
    assert_bits_equal(got, x.max(tuple(ax), keepdims=keep), "reduce_max vs numpy")


@pytest.mark.parametrize("shape", [[1, 50, 70], [3, 1000, 1000], [1], [5]])
def test_reduce_max_all_axes(ctx, oracle, case, shape):
    """The one ReduceMax the reference implements: every axis, keepdims=0 (test_ops_reduce.py:33-41)."""
    case(f"reduce_max all {shape}")
    x = synth.normal(73, shape)
    info = {}
    exp = oracle.reduce(1, x, [], False, strict=True, info=info)
    assert not info["no_reference_kernel"]
    got = ctx.reduce(D.REDUCE_MAX, x, 1, x.size, 1).reshape(exp.shape)
    assert_bits_equal(got, exp, f"reduce_max all {shape}")


@pytest.mark.parametrize("shape,mask_shape", [((4, 12, 197, 197), (4, 1, 1, 197)), ((3, 2, 40, 50), (3, 1, 1, 50)),
                                              ((2, 3, 33, 64), (1, 1, 1, 64)), ((2, 2048, 7), (2, 1, 7)), ((5, 64, 7), (5, 1, 7)), ((6, 3, 9), (6, 1, 9)), ((96, 100), None), ((2, 3, 40, 512), (1, 1, 1, 512)), ((4, 2, 16, 1024), (4, 1, 1, 1024)), ((64, 256), None)])
@pytest.mark.parametrize("scale_op", [0, 1, 2])
def test_softmax_with_scale_and_mask_prologue(case, ctx, oracle, shape, mask_shape, scale_op):
    """softmax((x [*|/] c) + mask) in one kernel has the bits of the oracle's Mul/Div, Add and Softmax one after
    the other when the kernel's lane layout sums each row in the same order as its plain Softmax -- checked here
    against this backend's own three kernels bit for bit, and against the oracle's chain at the parity bar."""
    case(f"softmax prologue {shape} mask {mask_shape} scale_op {scale_op}")
    if scale_op == 0 and mask_shape is None:
        pytest.skip("nothing to fuse")
    x = synth.normal(5, list(shape))
    mask = None if mask_shape is None else synth.attention_mask(6, list(mask_shape), p_masked=0.2)
    c = np.float32(0.125) if scale_op == 1 else np.float32(7.9)
    got = ctx.softmax_prologue(x, scale_op, c, mask)
    z_gpu, z_cpu = x, x
    if scale_op:
        op_g, op_o = (D.MUL, oracle.MUL) if scale_op == 1 else (D.DIV, oracle.DIV)
        z_gpu, z_cpu = ctx.binary(op_g, z_gpu, np.array(c, np.float32)), oracle.binary(op_o, z_cpu, np.array(c, np.float32))
    if mask is not None:
        z_gpu, z_cpu = ctx.binary(D.ADD, z_gpu, mask), oracle.binary(oracle.ADD, z_cpu, mask)
    assert_bits_equal(z_gpu, z_cpu, "the prologue's operators alone")
    assert_bits_equal(got, ctx.softmax(z_gpu), "fused vs three kernels")
    assert_close(got, oracle.softmax(z_cpu), what="fused vs oracle chain")


def test_softmax_prologue_refusals(case, ctx):
    case("softmax prologue: geometry the kernel does not take")
    x = synth.normal(1, [64, 16])
    with pytest.raises(AltiusHipError) as e:      # rows longer than the LDS kernel handles
        ctx.softmax_prologue(synth.normal(3, [4, 2048]), 1, 0.5, None)
    assert e.value.code == ERR_UNSUPPORTED
    with pytest.raises(AltiusHipError) as e:
        ctx.softmax_prologue(x, 3, 0.5, None)
    assert e.value.code == ERR_ARG
