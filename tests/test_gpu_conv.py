"""Conv2d (im2col + MFMA GEMM) and MaxPool through the C ABI and the session: exact on integer-valued
data against the oracle and the definition, bounded on random data; padding forms, strides, dilation,
groups, SAME_UPPER, and the ViT patch embedding feeding the token layout."""
import numpy as np
import pytest

import oracle as O
from altius_amd.graph import Model, Op
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal
from test_oracle import CONV_CASES, direct_conv

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(41)


@pytest.mark.parametrize("case_", CONV_CASES)
def test_conv2d(ctx, case, case_):
    case(f"conv2d {case_}")
    args = dict(strides=(1, 1), pads=(0, 0, 0, 0), dilations=(1, 1), group=1)
    args.update({k: v for k, v in case_.items() if k not in ("x", "w")})
    x = RNG.integers(-3, 4, size=case_["x"]).astype(np.float32)
    w = RNG.integers(-3, 4, size=case_["w"]).astype(np.float32)
    bias = RNG.integers(-3, 4, size=case_["w"][0]).astype(np.float32)
    for b in (bias, None):
        got = ctx.conv2d(x, w, b, **args)
        assert_bits_equal(got, O.conv2d(x, w, b, **args), "vs oracle")
        assert_bits_equal(got, direct_conv(x, w, b, **args).astype(np.float32), "vs the definition")
    xr, wr = RNG.standard_normal(case_["x"]).astype(np.float32), RNG.standard_normal(case_["w"]).astype(np.float32)
    k = int(np.prod(case_["w"][1:]))
    exact = direct_conv(xr, wr, bias, **args)
    bound = (k + 3) * 2.0 ** -24 * direct_conv(np.abs(xr), np.abs(wr), np.abs(bias), **args)
    got = ctx.conv2d(xr, wr, bias, **args)
    assert np.all(np.abs(got - exact) <= bound)
    assert np.allclose(got, O.conv2d(xr, wr, bias, **args), rtol=1e-5, atol=1e-5 * np.sqrt(k))


def test_max_pool(ctx, case):
    case("maxpool")
    x = RNG.standard_normal((2, 5, 33, 31)).astype(np.float32)
    x[0, 0, 0, 0] = np.nan
    for kernel, strides, pads in [((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 3), (2, 2), (1, 1, 1, 1)), ((3, 2), (1, 3), (0, 1, 2, 0)), ((33, 31), (1, 1), (0, 0, 0, 0))]:
        assert_bits_equal(ctx.max_pool(x, kernel, strides, pads), O.max_pool(x, kernel, strides, pads), f"maxpool {kernel} {strides} {pads}")
    lowest = np.full((1, 1, 2, 2), np.finfo(np.float32).min, np.float32)
    assert_bits_equal(ctx.max_pool(lowest, (2, 2), (2, 2)), np.zeros((1, 1, 1, 1), np.float32), "f32::MIN window")


def test_vit_patch_embedding_and_cnn_stem_through_the_session(case):
    case("session: Conv -> Reshape -> Transpose (ViT tokens); Conv SAME_UPPER -> Relu -> MaxPool")
    x = RNG.integers(-2, 3, size=(2, 3, 32, 32)).astype(np.float32)
    w = RNG.integers(-2, 3, size=(24, 3, 8, 8)).astype(np.float32)
    b = RNG.integers(-2, 3, size=24).astype(np.float32)
    m = Model(opset_version=13)
    v = m.new_val_named_and_shaped("x", x.shape)
    c, r, t = m.new_val(), m.new_val(), m.new_val()
    m.add_node(Op.Conv2d, [v, m.new_initializer(w), m.new_initializer(b)], [c], kernel_shape=[8, 8], strides=[8, 8])
    m.add_node(Op.Reshape, [c, m.new_initializer(np.array([2, 24, 16], np.int64))], [r])
    m.add_node(Op.Transpose, [r], [t], perm=[0, 2, 1])
    m.add_input(v)
    m.add_output(t)
    (tokens,) = HipSessionBuilder(m).build().run([x])
    want = direct_conv(x, w, b, (8, 8), (0, 0, 0, 0), (1, 1), 1).astype(np.float32).reshape(2, 24, 16).transpose(0, 2, 1)
    assert_bits_equal(tokens, want, "patch tokens")

    x2 = RNG.integers(-2, 3, size=(1, 3, 15, 17)).astype(np.float32)
    w2 = RNG.integers(-2, 3, size=(8, 3, 3, 3)).astype(np.float32)
    m = Model(opset_version=13)
    v = m.new_val_named_and_shaped("x", x2.shape)
    c, a, p = m.new_val(), m.new_val(), m.new_val()
    m.add_node(Op.Conv2d, [v, m.new_initializer(w2)], [c], kernel_shape=[3, 3], strides=[2, 2], auto_pad="SAME_UPPER")
    m.add_node(Op.ReLU, [c], [a])
    m.add_node(Op.MaxPool, [a], [p], kernel_shape=[2, 2], strides=[2, 2])
    m.add_input(v)
    m.add_output(p)
    (got,) = HipSessionBuilder(m).build().run([x2])
    # SAME_UPPER for 15x17, k 3, s 2: out 8x9, total pad 2 -> (1,1) and 2 -> (1,1)  (shape.rs:48-61)
    conv = direct_conv(x2, w2, None, (2, 2), (1, 1, 1, 1), (1, 1), 1).astype(np.float32)
    assert conv.shape == (1, 8, 8, 9)
    assert_bits_equal(got, O.max_pool(np.maximum(conv, 0), (2, 2), (2, 2)), "cnn stem")


def test_resize(ctx, case):
    case("resize")
    x = RNG.standard_normal((2, 3, 13, 17)).astype(np.float32)
    for out_hw in [(26, 34), (13, 17), (39, 51), (20, 25), (6, 8), (1, 1)]:
        for nearest in (True, False):
            assert_bits_equal(ctx.resize(x, out_hw, nearest), O.resize(x, out_hw, nearest), f"resize {out_hw} nearest={nearest}")
    # through the session, with `scales` (3 inputs) and with `sizes` (4 inputs)
    for extra, mode in (([np.zeros(0, np.float32), np.array([1, 1, 2, 2], np.float32)], "nearest"),
                        ([np.zeros(0, np.float32), np.zeros(0, np.float32), np.array([2, 3, 30, 40], np.int64)], "linear")):
        m = Model(opset_version=13)
        v = m.new_val_named_and_shaped("x", x.shape)
        y = m.new_val()
        m.add_node(Op.Resize, [v] + [m.new_initializer(e) for e in extra], [y], mode=mode, coordinate_transformation_mode="asymmetric",
                   nearest_mode="floor")
        m.add_input(v)
        m.add_output(y)
        (got,) = HipSessionBuilder(m).build().run([x])
        want = O.resize(x, (26, 34), True) if mode == "nearest" else O.resize(x, (30, 40), False)
        assert_bits_equal(got, want, f"session resize {mode}")
