"""compute_output_shapes for every operator (crates/core/src/analysis/shape.rs:21-657), checked
against what numpy produces for the same operation, plus the reference's own special cases."""
import numpy as np
import pytest

from altius_amd._lib import ERR_ARG, ERR_SHAPE, AltiusHipError
from altius_amd.graph import BOOL, F32, I32, I64, Model, Op

NP = {F32: np.float32, I64: np.int64, I32: np.int32, BOOL: np.bool_}


def infer(op, in_shapes, consts=None, n_out=1, opset=13, in_types=None, **attrs):
    """Shapes of the outputs of one node.  in_shapes: list of shapes (graph inputs) or None where
    `consts` gives an initializer for that operand."""
    m = Model(opset_version=opset)
    ins = []
    consts = consts or {}
    for i, s in enumerate(in_shapes):
        if i in consts:
            ins.append(m.new_initializer(np.asarray(consts[i]), name=f"c{i}"))
        else:
            v = m.new_val_named_and_shaped(f"x{i}", s, (in_types or {}).get(i, F32))
            m.add_input(v)
            ins.append(v)
    outs = [m.new_val_named(f"y{i}") for i in range(n_out)]
    m.add_node(op, ins, outs, **attrs)
    for o in outs:
        m.add_output(o)
    res = [m.infer_value_shape(o) for o in outs]
    return res if n_out > 1 else res[0]


def test_elementwise_and_typed_ops():
    for op in (Op.Identity, Op.Sqrt, Op.ReLU, Op.LeakyReLU, Op.Gelu, Op.Sigmoid, Op.Erf, Op.Tanh, Op.Clip, Op.HardSigmoid,
               Op.Round, Op.Exp, Op.Softmax):
        assert infer(op, [[2, 3, 4]]) == ([2, 3, 4], F32)
    assert infer(Op.BatchNormalization, [[2, 3, 4, 4], [3], [3], [3], [3]]) == ([2, 3, 4, 4], F32)
    assert infer(Op.Cast, [[2, 3]], to=7) == ([2, 3], I64)
    assert infer(Op.Cast, [[2, 3]], in_types={0: I64}, to=1) == ([2, 3], F32)
    assert infer(Op.Greater, [[4, 1, 3], [5, 1]]) == (list(np.broadcast_shapes((4, 1, 3), (5, 1))), BOOL)
    assert infer(Op.Where, [[1, 1, 5, 5], [2, 3, 5, 5], []], in_types={0: BOOL}) == ([2, 3, 5, 5], F32)


@pytest.mark.parametrize("shape,new", [([2, 3, 4], [6, 4]), ([2, 3, 4], [-1]), ([2, 3, 4], [2, -1, 2]), ([2, 3, 4], [0, 12]),
                                        ([2, 3, 4], [0, 0, -1]), ([7], [1, 7, 1])])
def test_reshape_like_numpy(shape, new):
    want = [shape[i] if d == 0 else d for i, d in enumerate(new)]
    want = list(np.zeros(shape).reshape(want).shape)
    assert infer(Op.Reshape, [shape, None], {1: np.array(new, np.int64)}) == (want, F32)


def test_reshape_errors_and_runtime_shapes():
    with pytest.raises(AltiusHipError) as e:
        infer(Op.Reshape, [[2, 3], None], {1: np.array([4, 2], np.int64)})
    assert e.value.code == ERR_SHAPE
    with pytest.raises(AltiusHipError):
        infer(Op.Reshape, [[2, 3], None], {1: np.array([-1, -1], np.int64)})
    # the shape operand is a graph input: nothing to infer before the run (ERR_ARG = shape stays unknown)
    with pytest.raises(AltiusHipError) as e:
        infer(Op.Reshape, [[2, 3], [2]], in_types={1: I64})
    assert e.value.code == ERR_ARG


def test_flatten_transpose_concat():
    assert infer(Op.Flatten, [[2, 3, 4, 5]]) == ([2, 60], F32)                         # axis 1 by default
    assert infer(Op.Flatten, [[2, 3, 4, 5]], axis=3) == ([24, 5], F32)
    assert infer(Op.Flatten, [[2, 3, 4, 5]], axis=0) == ([1, 120], F32)
    for perm in ([0, 2, 1, 3], [3, 2, 1, 0], [1, 0, 3, 2]):
        assert infer(Op.Transpose, [[2, 3, 4, 5]], perm=perm) == (list(np.zeros((2, 3, 4, 5)).transpose(perm).shape), F32)
    with pytest.raises(AltiusHipError):
        infer(Op.Transpose, [[2, 3, 4]], perm=[0, 0, 1])
    with pytest.raises(AltiusHipError):
        infer(Op.Transpose, [[2, 3, 4]], perm=[0, 1])
    assert infer(Op.Concat, [[2, 3, 4], [2, 5, 4], [2, 1, 4]], axis=1) == ([2, 9, 4], F32)
    assert infer(Op.Concat, [[2, 3, 4], [2, 3, 1]], axis=-1) == ([2, 3, 5], F32)
    with pytest.raises(AltiusHipError):
        infer(Op.Concat, [[2, 3, 4], [3, 3, 4]], axis=1)


def test_squeeze_unsqueeze_by_opset():
    assert infer(Op.Squeeze, [[1, 3, 1, 4]], opset=11, axes=[0, 2]) == ([3, 4], F32)                      # attribute
    assert infer(Op.Squeeze, [[1, 3, 1, 4], None], {1: np.array([2], np.int64)}, opset=13) == ([1, 3, 4], F32)  # input
    assert infer(Op.Squeeze, [[1, 3, 1, 4]], opset=13) == ([3, 4], F32)                                    # none: all ones
    with pytest.raises(AltiusHipError):
        infer(Op.Squeeze, [[1, 3, 1, 4]], opset=11, axes=[1])
    assert infer(Op.Unsqueeze, [[3, 4]], opset=11, axes=[0, 3]) == (list(np.expand_dims(np.zeros((3, 4)), (0, 3)).shape), F32)
    assert infer(Op.Unsqueeze, [[3, 4], None], {1: np.array([1], np.int64)}, opset=13) == ([3, 1, 4], F32)
    assert infer(Op.Unsqueeze, [[3, 4], None], {1: np.array([-1], np.int64)}, opset=13) == ([3, 4, 1], F32)


def test_reductions():
    assert infer(Op.ReduceMin, [[2, 3, 4]], axes=[1]) == ([2, 1, 4], F32)
    assert infer(Op.ReduceMin, [[2, 3, 4]], axes=[-1, 0], keepdims=0) == ([3], F32)
    assert infer(Op.ReduceMax, [[2, 3, 4]], keepdims=0) == ([1], F32)                                      # all axes -> [1]
    assert infer(Op.ReduceMean, [[2, 3, 4]], axes=[2]) == ([2, 3, 1], F32)
    assert infer(Op.GlobalAveragePool, [[2, 7, 5, 5]]) == ([2, 7, 1, 1], F32)


def test_split_slice_gather_tile_expand_range_shape():
    assert infer(Op.Split, [[2, 3, 12]], n_out=3, opset=11, axis=2, split=[2, 4, 6]) == [([2, 3, 2], F32), ([2, 3, 4], F32), ([2, 3, 6], F32)]
    assert infer(Op.Split, [[2, 3, 12], None], {1: np.array([5, 7], np.int64)}, n_out=2, axis=-1) == [([2, 3, 5], F32), ([2, 3, 7], F32)]
    assert infer(Op.Split, [[2, 6, 12]], n_out=3, axis=1) == [([2, 2, 12], F32)] * 3                       # equal parts
    with pytest.raises(AltiusHipError):
        infer(Op.Split, [[2, 3, 12]], n_out=2, opset=11, axis=2, split=[2, 4])
    x = np.zeros((4, 6, 10))
    i64 = lambda *v: np.array(v, np.int64)
    for starts, ends, axes, steps, want in [
        ((1,), (7,), (2,), (1,), x[:, :, 1:7]), ((0,), (10,), (2,), (3,), x[:, :, 0:10:3]), ((1, 2), (3, 100), (0, 1), (1, 2), x[1:3, 2:100:2]),
        ((-3,), (-1,), (-1,), (1,), x[:, :, -3:-1]), ((5,), (2,), (1,), (1,), x[:, 5:2]),
    ]:
        got = infer(Op.Slice, [list(x.shape), None, None, None, None], {1: i64(*starts), 2: i64(*ends), 3: i64(*axes), 4: i64(*steps)})
        assert got == (list(want.shape), F32)
    assert infer(Op.Slice, [[4, 6, 10], None, None], {1: i64(1, 1), 2: i64(3, 4)}) == ([2, 3, 10], F32)   # axes default to 0..n
    d = np.zeros((5, 6, 7))
    for axis, idx in [(0, np.array(2)), (1, np.array([[0, 3, 5]])), (2, np.array([1, 1])), (-1, np.array(0))]:
        got = infer(Op.Gather, [list(d.shape), None], {1: idx.astype(np.int64)}, axis=axis)
        assert got == (list(np.take(d, idx, axis=axis).shape), F32)
    assert infer(Op.Tile, [[2, 3], None], {1: i64(2, 3)}) == (list(np.tile(np.zeros((2, 3)), (2, 3)).shape), F32)
    assert infer(Op.Expand, [[3, 1], None], {1: i64(2, 1, 6)}) == (list(np.broadcast_shapes((3, 1), (2, 1, 6))), F32)
    assert infer(Op.Expand, [[1, 1, 1, 4], None], {1: i64(1, 1, 5, 4)}, in_types={0: I64}) == ([1, 1, 5, 4], I64)
    for s, l, dlt in [(0, 10, 1), (2, 11, 3), (5, 5, 1), (10, 0, -3), (7, 2, 1)]:
        got = infer(Op.Range, [None, None, None], {0: i64(s).reshape(()), 1: i64(l).reshape(()), 2: i64(dlt).reshape(())})
        assert got == ([len(np.arange(s, l, dlt))], I64)
    assert infer(Op.Shape, [[2, 3, 4, 5]]) == ([4], I64)
    assert infer(Op.Shape, [[2, 3, 4, 5]], opset=15, start=1, end=-1) == ([2], I64)
    c = np.arange(6, dtype=np.int64).reshape(2, 3)
    assert infer(Op.Constant, [], value=c) == ([2, 3], I64)


def test_matmul_and_gemm():
    for a, b in [((3, 4), (4, 5)), ((2, 3, 4), (4, 5)), ((2, 3, 4), (2, 4, 5)), ((1, 6, 3, 4), (1, 6, 4, 5)),
                 ((7, 6, 3, 4), (6, 4, 5)), ((7, 1, 3, 4), (1, 6, 4, 5))]:
        assert infer(Op.MatMul, [list(a), list(b)]) == (list(np.matmul(np.zeros(a), np.zeros(b)).shape), F32)
    with pytest.raises(AltiusHipError) as e:
        infer(Op.MatMul, [[3, 4], [5, 6]])
    assert e.value.code == ERR_SHAPE and "A shape" in e.value.message
    assert infer(Op.Gemm, [[3, 4], [4, 5], [5]]) == ([3, 5], F32)
    assert infer(Op.Gemm, [[4, 3], [5, 4], [3, 5]], transA=1, transB=1) == ([3, 5], F32)
    with pytest.raises(AltiusHipError):
        infer(Op.Gemm, [[3, 4], [5, 4]])


def conv_out(n, k, s, p0, p1, d=1):
    return (n + p0 + p1 - d * (k - 1) - 1) // s + 1


def test_conv_and_maxpool():
    # patch embedding of ViT: 16x16 stride 16
    assert infer(Op.Conv2d, [[8, 3, 224, 224], [768, 3, 16, 16], [768]], kernel_shape=[16, 16], strides=[16, 16]) == ([8, 768, 14, 14], F32)
    assert infer(Op.Conv2d, [[1, 3, 32, 30], [8, 3, 3, 5]], kernel_shape=[3, 5], pads=[1, 2]) == (
        [1, 8, conv_out(32, 3, 1, 1, 1), conv_out(30, 5, 1, 2, 2)], F32)                                # two pads = symmetric
    assert infer(Op.Conv2d, [[1, 3, 32, 30], [8, 3, 3, 3]], kernel_shape=[3, 3], pads=[0, 1, 2, 3], strides=[2, 2], dilations=[2, 1]) == (
        [1, 8, conv_out(32, 3, 2, 0, 2, 2), conv_out(30, 3, 2, 1, 3)], F32)
    # SAME_UPPER: output = ceil(in / stride) (shape.rs:48-61)
    assert infer(Op.Conv2d, [[1, 3, 33, 31], [8, 3, 3, 3]], kernel_shape=[3, 3], strides=[2, 2], auto_pad="SAME_UPPER") == ([1, 8, 17, 16], F32)
    assert infer(Op.MaxPool, [[2, 4, 32, 32]], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1]) == ([2, 4, 16, 16], F32)
    assert infer(Op.MaxPool, [[2, 4, 33, 31]], kernel_shape=[2, 2], strides=[2, 2], auto_pad="SAME_UPPER") == ([2, 4, 17, 16], F32)
    with pytest.raises(AltiusHipError):
        infer(Op.Conv2d, [[1, 3, 4, 4], [8, 3, 7, 7]], kernel_shape=[7, 7])


def test_resize():
    assert infer(Op.Resize, [[1, 3, 8, 8], None, None, None], {1: np.zeros(0, np.float32), 2: np.zeros(0, np.float32),
                                                            3: np.array([1, 3, 20, 24], np.int64)}) == ([1, 3, 20, 24], F32)
    assert infer(Op.Resize, [[1, 3, 8, 9], None, None], {1: np.zeros(0, np.float32), 2: np.array([1, 1, 2, 2.5], np.float32)}) == (
        [1, 3, 16, 22], F32)                                                                                # floor(dim * scale)


def test_unsupported_ops_say_so():
    for op, n in ((Op.Loop, 3), (Op.NonMaxSuppression, 2)):
        with pytest.raises(AltiusHipError) as e:
            infer(op, [[1]] * n)
        assert e.value.code == ERR_SHAPE and "Unsupported op" in e.value.message
