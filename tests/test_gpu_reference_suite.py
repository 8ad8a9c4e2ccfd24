"""The reference's Python operator tests (crates/altius_py/tests/test_ops_*.py), one for one and under their
names, against this backend: each writes the same one-node ONNX model to a file, opens it with
InferenceSession (the reference's entry point, crates/altius_py/altius_py/__init__.py:4-30) and runs it on
U[0,1) inputs.  The reference compares with onnxruntime, which is not installed here: expectations are the
NumPy / closed-form definition of the operator (the CPU oracle for the interpreter's approximated
functions), at the tolerance the reference's test states."""
import os

import numpy as np
import pytest

import onnx_writer as W
import oracle as O
from altius_amd.inference import InferenceSession

pytestmark = pytest.mark.gpu

RNG = np.random.default_rng(1234)


def rand(shape):
    return RNG.random(size=tuple(shape), dtype=np.float32)   # np.random.random_sample(shape).astype(np.float32)


def one_node(tmp_path, op_type, inputs, outputs, initializers=(), opset=13, **attrs):
    """inputs / outputs: (name, elem_type, shape).  Returns an InferenceSession over the saved file."""
    nodes = [W.node(op_type, [i[0] for i in inputs] + [t[0] for t in initializers], [o[0] for o in outputs], **attrs)]
    g = W.graph(nodes, [W.tensor(n, a) for n, a in initializers], [W.value_info(*i) for i in inputs],
                [W.value_info(*o) for o in outputs])
    path = os.path.join(tmp_path, "model.onnx")
    with open(path, "wb") as f:
        f.write(W.model(g, opsets=(("", opset),)))
    return InferenceSession(path)


# ---- test_ops_bin.py ----------------------------------------------------------------------------------
NP_BIN = {"Add": np.add, "Sub": np.subtract, "Mul": np.multiply, "Div": np.divide, "Pow": np.power, "Greater": np.greater}


def op_bin(tmp_path, op_type, shape_x, shape_y=None, shape_z=None, zdtype=W.FLOAT):
    shape_y = shape_y if shape_y else shape_x
    shape_z = shape_z if shape_z else shape_x
    sess = one_node(tmp_path, op_type, [("x", W.FLOAT, shape_x), ("y", W.FLOAT, shape_y)], [("z", zdtype, shape_z)])
    x, y = rand(shape_x), rand(shape_y)
    (actual,) = sess.run(None, {"x": x, "y": y})
    expected = NP_BIN[op_type](x, y)
    assert actual.shape == expected.shape and actual.dtype == expected.dtype
    assert np.allclose(expected, actual)
    if op_type in ("Add", "Sub", "Mul", "Div", "Greater"):      # one IEEE operation per element: exact
        assert np.array_equal(expected, actual)


BIN_CASES = {
    "add_1": ("Add", [1, 2]), "add_2": ("Add", [1, 2, 3, 4, 5, 6, 7]), "add_3": ("Add", [128, 3, 224, 224]),
    "add_4": ("Add", [1, 3, 28, 28], [3, 1, 1]), "add_6": ("Add", [1, 12, 9, 9], [1, 1, 1, 9]),
    "add_7": ("Add", [4, 1, 2], [3, 1], [4, 3, 2]),
    "sub_1": ("Sub", [1, 2]), "sub_2": ("Sub", [1, 2, 3, 4, 5, 6, 7]), "sub_3": ("Sub", [128, 3, 224, 224]),
    "sub_4": ("Sub", [1, 3, 28, 28], [3, 1, 1]), "sub_5": ("Sub", [3, 28, 28], [3, 28, 1]),
    "mul_1": ("Mul", [1, 2]), "mul_2": ("Mul", [1, 2, 3, 4, 5, 6, 7]), "mul_3": ("Mul", [128, 3, 224, 224]),
    "mul_4": ("Mul", [3, 15, 15], [15]),
    "div_1": ("Div", [1, 2]), "div_2": ("Div", [1, 2, 3, 4, 5, 6, 7]), "div_3": ("Div", [128, 3, 224, 224]),
    "div_4": ("Div", [3, 28, 28], [3, 28, 1]), "div_5": ("Div", [3, 28, 28], [1]),
    "pow_1": ("Pow", [1, 2]), "pow_2": ("Pow", [1, 2, 3, 4, 5, 6, 7]), "pow_3": ("Pow", [128, 3, 8, 8]),
    "pow_4": ("Pow", [128, 3, 8, 8], [1]),
}


@pytest.mark.parametrize("name", list(BIN_CASES))
def test_bin(case, tmp_path, name):
    """test_add_1..7, test_sub_1..5, test_mul_1..4, test_div_1..5, test_pow_1..4 (test_ops_bin.py:11-141)."""
    case(f"reference test_{name}")
    op_bin(tmp_path, *BIN_CASES[name])


def test_add_5(case, tmp_path):
    """xfail in the reference (shapes that cannot broadcast abort it): here the failure is an error value."""
    case("reference test_add_5")
    with pytest.raises(Exception) as e:
        op_bin(tmp_path, "Add", [1, 3, 28, 28], [3, 1, 2])
    assert "broadcast" in str(e.value)


def test_greater_1(case, tmp_path):
    """xfail in the reference (its Greater needs a scalar right operand, session.rs:541-562); general here."""
    case("reference test_greater_1")
    op_bin(tmp_path, "Greater", [3, 4, 5], zdtype=W.BOOL)


def test_greater_2(case, tmp_path):
    case("reference test_greater_2")
    op_bin(tmp_path, "Greater", [3, 4, 5], shape_y=[1], zdtype=W.BOOL)


# ---- test_ops_elemwise.py ----------------------------------------------------------------------------
def erf_exact(x):
    import math
    return np.vectorize(math.erf)(x.astype(np.float64))


ELEMWISE = {
    # op -> (expected, kwargs of np.allclose as the reference's test passes them)
    "Identity": (lambda x: x, {}),
    "Relu": (lambda x: np.maximum(x, 0), {}),
    "HardSigmoid": (lambda x: np.clip(0.2 * x + 0.5, 0, 1), {}),
    "LeakyRelu": (lambda x: np.where(x < 0, 0.01 * x, x), {}),
    "Sigmoid": (lambda x: 1 / (1 + np.exp(-x.astype(np.float64))), {}),
    "Clip": (lambda x: x, {}),                          # no bounds given: the identity
    "Sqrt": (np.sqrt, {}),
    "Softmax": (lambda x: np.exp(x.astype(np.float64)) / np.exp(x.astype(np.float64)).sum(-1, keepdims=True), {}),
    "Erf": (erf_exact, {"atol": 1e-1, "rtol": 1e-5}),
}

ELEMWISE_CASES = {
    "identity_1": ("Identity", [1, 2]), "relu_1": ("Relu", [1, 2]), "relu_2": ("Relu", [3, 1, 28, 28]),
    "hardsigmoid_1": ("HardSigmoid", [1, 2]), "hardsigmoid_2": ("HardSigmoid", [3, 1, 28, 28]),
    "leakyrelu_1": ("LeakyRelu", [1, 2]), "leakyrelu_2": ("LeakyRelu", [3, 1, 28, 28]),
    "sigmoid_1": ("Sigmoid", [1, 2]), "sigmoid_2": ("Sigmoid", [3, 1, 28, 28]), "sigmoid_3": ("Sigmoid", [3, 1, 7, 7]),
    "clip_1": ("Clip", [1, 2]), "clip_2": ("Clip", [3, 1, 28, 28]),   # xfail in the reference (no kernel, session.rs:201)
    "sqrt_1": ("Sqrt", [1, 2]), "sqrt_2": ("Sqrt", [3, 1, 28, 28]),
    "softmax_1": ("Softmax", [1, 2, 3]), "softmax_2": ("Softmax", [3, 28, 28]), "softmax_3": ("Softmax", [128, 512, 512]),
    "erf_1": ("Erf", [1, 2, 3]), "erf_2": ("Erf", [3, 28, 28]),
}


@pytest.mark.parametrize("name", list(ELEMWISE_CASES))
def test_elemwise(case, tmp_path, name):
    """test_identity_1 ... test_erf_2 (test_ops_elemwise.py:15-152)."""
    case(f"reference test_{name}")
    op_type, shape = ELEMWISE_CASES[name]
    sess = one_node(tmp_path, op_type, [("x", W.FLOAT, shape)], [("y", W.FLOAT, shape)])
    x = rand(shape)
    (actual,) = sess.run(None, {"x": x})
    fn, tol = ELEMWISE[op_type]
    assert actual.shape == tuple(shape)
    assert np.allclose(fn(x), actual, **tol)


def test_gelu_1(case, tmp_path):
    """test_gelu_1 (test_ops_elemwise.py:155-185): Mul(Mul(x, Add(Erf(Div(x, sqrt 2)), 1)), 0.5) with [1]-shaped
    constants, which InferenceSession rewrites to Gelu; within 1e-1 of the exact function as the reference asks,
    and equal to the interpreter's own Gelu formula bit for bit."""
    case("reference test_gelu_1")
    c = lambda v: np.array([v], np.float32)
    nodes = [W.node("Div", ["x", "sqrt2"], ["d"]), W.node("Erf", ["d"], ["e"]), W.node("Add", ["e", "one"], ["a"]),
             W.node("Mul", ["x", "a"], ["m"]), W.node("Mul", ["m", "half"], ["y"])]
    g = W.graph(nodes, [W.tensor("sqrt2", c(np.sqrt(2.0))), W.tensor("one", c(1.0)), W.tensor("half", c(0.5))],
                [W.value_info("x", W.FLOAT, [1, 2, 3])], [W.value_info("y", W.FLOAT, [1, 2, 3])])
    path = os.path.join(tmp_path, "model.onnx")
    with open(path, "wb") as f:
        f.write(W.model(g, opsets=(("", 12),)))
    sess = InferenceSession(path)
    x = rand([1, 2, 3])
    (actual,) = sess.run(None, {"x": x})
    expected = x * 0.5 * (1 + erf_exact(x / np.sqrt(2.0)))
    assert np.allclose(expected, actual, atol=1e-1, rtol=1e-5)
    assert np.array_equal(actual, O.unary(O.GELU, x))


# ---- test_ops_concat.py, test_ops_gather.py, test_ops_transpose.py, test_ops_where.py ----------------
def test_concat_1(case, tmp_path):
    case("reference test_concat_1")
    sess = one_node(tmp_path, "Concat", [("x", W.FLOAT, [1, 1, 10]), ("y", W.FLOAT, [1, 3, 10])], [("z", W.FLOAT, [1, 4, 10])], axis=1)
    x, y = rand([1, 1, 10]), rand([1, 3, 10])
    (actual,) = sess.run(None, {"x": x, "y": y})
    assert np.array_equal(np.concatenate([x, y], axis=1), actual)


@pytest.mark.parametrize("name,shape_x,indices,shape_z,axis", [("gather_1", [1, 5, 10], 2, [1, 1, 10], 1),
                                                                  ("gather_2", [5, 10], [1, 3], [2, 10], 0)])
def test_gather(case, tmp_path, name, shape_x, indices, shape_z, axis):
    """test_gather_1, test_gather_2 (test_ops_gather.py:11-31); the declared output shapes there are onnx's, the
    computed ones are x.take(indices, axis)."""
    case(f"reference test_{name}")
    shape_y = [] if isinstance(indices, int) else [1, len(indices)]
    sess = one_node(tmp_path, "Gather", [("x", W.FLOAT, shape_x), ("y", W.INT64, shape_y)], [("z", W.FLOAT, shape_z)], axis=axis)
    x = rand(shape_x)
    y = np.array(indices).astype(np.int64).reshape(shape_y)
    (actual,) = sess.run(None, {"x": x, "y": y})
    assert np.array_equal(np.take(x, y, axis=axis), actual)


@pytest.mark.parametrize("name,shape_x,shape_y,perm", [("transpose_1", [50, 12, 64], [12, 64, 50], [1, 2, 0]),
                                                       ("transpose_2", [12, 64], [64, 12], [1, 0]),
                                                       ("transpose_3", [12, 64, 3, 5], [3, 64, 12, 5], [2, 1, 0, 3]),
                                                       ("transpose_4", [50, 12], [50, 12], [0, 1])])
def test_transpose(case, tmp_path, name, shape_x, shape_y, perm):
    case(f"reference test_{name}")
    sess = one_node(tmp_path, "Transpose", [("x", W.FLOAT, shape_x)], [("y", W.FLOAT, shape_y)], perm=perm)
    x = rand(shape_x)
    (actual,) = sess.run(None, {"x": x})
    assert actual.shape == tuple(shape_y) and np.array_equal(x.transpose(perm), actual)


@pytest.mark.parametrize("name,shape_c,shape_x,shape_y", [("where_1", [1, 1, 10, 10], [1, 128, 10, 10], [1]),
                                                          ("where_2", [1, 1, 1, 1], [1, 128, 1, 1], [1])])
def test_where(case, tmp_path, name, shape_c, shape_x, shape_y):
    case(f"reference test_{name}")
    sess = one_node(tmp_path, "Where", [("c", W.BOOL, shape_c), ("x", W.FLOAT, shape_x), ("y", W.FLOAT, shape_y)],
                    [("z", W.FLOAT, shape_x)])
    c = RNG.choice(a=[False, True], size=shape_c)
    x, y = rand(shape_x), rand(shape_y)
    (actual,) = sess.run(None, {"c": c, "x": x, "y": y})
    assert np.array_equal(np.where(c, x, y), actual)


# ---- test_ops_conv.py, test_ops_pool.py, test_ops_resize.py ------------------------------------------
def conv2d_definition(x, w, b, strides, pads, group):
    n, c, h, wd = x.shape
    oc, cg, kh, kw = w.shape
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pads[0], pads[2]), (pads[1], pads[3])))
    oh = (h + pads[0] + pads[2] - kh) // strides[0] + 1
    ow = (wd + pads[1] + pads[3] - kw) // strides[1] + 1
    out = np.zeros((n, oc, oh, ow))
    per = oc // group
    for g in range(group):
        xs = xp[:, g * cg:(g + 1) * cg]
        for fy in range(kh):
            for fx in range(kw):
                patch = xs[:, :, fy:fy + strides[0] * oh:strides[0], fx:fx + strides[1] * ow:strides[1]]
                out[:, g * per:(g + 1) * per] += np.einsum("nchw,oc->nohw", patch, w[g * per:(g + 1) * per, :, fy, fx].astype(np.float64))
    if b is not None:
        out += b.reshape(1, -1, 1, 1)
    return out


@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("name,shape_x,shape_w,shape_y,kw", [
    ("conv2d_1", [1, 3, 224, 224], [16, 3, 3, 3], [1, 16, 112, 112], dict(pads=[1, 1, 1, 1], strides=[2, 2])),
    ("conv2d_2", [1, 16, 112, 112], [16, 1, 3, 3], [1, 16, 112, 112], dict(group=16, pads=[1, 1, 1, 1]))])
def test_conv2d(case, tmp_path, name, shape_x, shape_w, shape_y, kw, bias):
    case(f"reference test_{name} bias={bias}")
    inputs = [("x", W.FLOAT, shape_x), ("w", W.FLOAT, shape_w)] + ([("b", W.FLOAT, [shape_w[0]])] if bias else [])
    sess = one_node(tmp_path, "Conv", inputs, [("y", W.FLOAT, shape_y)], kernel_shape=shape_w[2:], **kw)
    x, w = rand(shape_x), rand(shape_w)
    b = rand([shape_w[0]]) if bias else None
    feed = {"x": x, "w": w, "b": b} if bias else {"x": x, "w": w}
    (actual,) = sess.run(None, feed)
    expected = conv2d_definition(x, w, b, kw.get("strides", [1, 1]), kw["pads"], kw.get("group", 1))
    assert actual.shape == tuple(shape_y) and np.allclose(expected, actual)


def maxpool_definition(x, k, s, p):
    xp = np.pad(x, ((0, 0), (0, 0), (p[0], p[2]), (p[1], p[3])), constant_values=-np.inf)
    oh = (xp.shape[2] - k[0]) // s[0] + 1
    ow = (xp.shape[3] - k[1]) // s[1] + 1
    out = np.full(x.shape[:2] + (oh, ow), -np.inf, np.float32)
    for fy in range(k[0]):
        for fx in range(k[1]):
            out = np.maximum(out, xp[:, :, fy:fy + s[0] * oh:s[0], fx:fx + s[1] * ow:s[1]])
    return out


@pytest.mark.parametrize("name,shape_x,shape_y,kw", [
    ("maxpool_1", [1, 3, 224, 224], [1, 3, 112, 112], dict(kernel_shape=[2, 2], pads=[0, 0, 0, 0], strides=[2, 2], auto_pad="NOTSET")),
    ("maxpool_2", [1, 256, 20, 20], [1, 256, 20, 20], dict(kernel_shape=[5, 5], pads=[2, 2, 2, 2], strides=[1, 1], ceil_mode=0))])
def test_maxpool(case, tmp_path, name, shape_x, shape_y, kw):
    case(f"reference test_{name}")
    sess = one_node(tmp_path, "MaxPool", [("x", W.FLOAT, shape_x)], [("y", W.FLOAT, shape_y)], **kw)
    x = rand(shape_x)
    (actual,) = sess.run(None, {"x": x})
    assert actual.shape == tuple(shape_y) and np.array_equal(maxpool_definition(x, kw["kernel_shape"], kw["strides"], kw["pads"]), actual)


def test_resize_1(case, tmp_path):
    case("reference test_resize_1")
    scales = np.array([1.0, 1.0, 2.0, 2.0], dtype=np.float32)
    sess = one_node(tmp_path, "Resize", [("x", W.FLOAT, [1, 256, 20, 20])], [("y", W.FLOAT, [1, 256, 40, 40])],
                    initializers=[("roi", np.array([], np.float32)), ("scales", scales)],
                    coordinate_transformation_mode="asymmetric", cubic_coeff_a=-0.75, mode="nearest", nearest_mode="floor")
    x = rand([1, 256, 20, 20])
    (actual,) = sess.run(None, {"x": x})
    assert np.array_equal(x.repeat(2, axis=2).repeat(2, axis=3), actual)     # asymmetric + floor with scale 2


# ---- test_ops_gemm.py, test_ops_matmul.py ------------------------------------------------------------
@pytest.mark.parametrize("name,shape_c", [("gemm_1", [15]), ("gemm_2", [5, 15]), ("gemm_3", None)])
def test_gemm(case, tmp_path, name, shape_c):
    case(f"reference test_{name}")
    inputs = [("a", W.FLOAT, [5, 10]), ("b", W.FLOAT, [10, 15])] + ([("c", W.FLOAT, shape_c)] if shape_c else [])
    sess = one_node(tmp_path, "Gemm", inputs, [("y", W.FLOAT, [5, 15])])
    a, b = rand([5, 10]), rand([10, 15])
    feed = {"a": a, "b": b}
    expected = a.astype(np.float64) @ b.astype(np.float64)
    if shape_c:
        feed["c"] = rand(shape_c)
        expected = expected + feed["c"]
    (actual,) = sess.run(None, feed)
    assert np.allclose(expected, actual)


@pytest.mark.parametrize("name,shape_x,shape_y,shape_z", [("matmul_1", [5, 10], [10, 15], [5, 15]), ("matmul_2", [3, 5, 10], [10, 15], [3, 5, 15]),
                                                          ("matmul_3", [3, 5, 10], [3, 10, 15], [3, 5, 15]), ("matmul_4", [1, 5, 10], [10, 15], [1, 5, 15])])
def test_matmul(case, tmp_path, name, shape_x, shape_y, shape_z):
    case(f"reference test_{name}")
    sess = one_node(tmp_path, "MatMul", [("x", W.FLOAT, shape_x), ("y", W.FLOAT, shape_y)], [("z", W.FLOAT, shape_z)])
    x, y = rand(shape_x), rand(shape_y)
    (actual,) = sess.run(None, {"x": x, "y": y})
    assert actual.shape == tuple(shape_z) and np.allclose(np.matmul(x.astype(np.float64), y.astype(np.float64)), actual)


# ---- test_ops_norm.py, test_ops_reduce.py --------------------------------------------------------------
def test_batch_norm_1(case, tmp_path):
    case("reference test_batch_norm_1")
    shape = [1, 20, 10, 10]
    names = ["scale", "bias", "mean", "var"]
    sess = one_node(tmp_path, "BatchNormalization", [("x", W.FLOAT, shape)] + [(n, W.FLOAT, [shape[1]]) for n in names], [("z", W.FLOAT, shape)])
    feed = {"x": rand(shape), **{n: rand([shape[1]]) for n in names}}
    (actual,) = sess.run(None, feed)
    v = lambda n: feed[n].astype(np.float64).reshape(1, -1, 1, 1)
    expected = (feed["x"] - v("mean")) / np.sqrt(v("var") + 1e-5) * v("scale") + v("bias")
    assert np.allclose(expected, actual, rtol=1e-4, atol=1e-5)


def test_layer_norm_1(case, tmp_path):
    case("reference test_layer_norm_1")
    shape, shape_scale = [1, 20, 10], [1, 1, 10]
    sess = one_node(tmp_path, "LayerNormalization", [("x", W.FLOAT, shape), ("scale", W.FLOAT, shape_scale), ("bias", W.FLOAT, shape_scale)],
                    [("z", W.FLOAT, shape)], opset=17)
    x, scale, bias = rand(shape), rand(shape_scale), rand(shape_scale)
    (actual,) = sess.run(None, {"x": x, "scale": scale, "bias": bias})
    xd = x.astype(np.float64)
    expected = (xd - xd.mean(-1, keepdims=True)) / np.sqrt(xd.var(-1, keepdims=True) + 1e-5) * scale + bias
    assert np.allclose(expected, actual, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("name,op_type,shape_x,shape_y,kw", [
    ("reduce_mean_1", "ReduceMean", [1, 50, 70], [1, 50, 1], dict(axes=[-1])),
    ("reduce_mean_2", "ReduceMean", [8, 4, 5, 5], [8, 4, 1, 1], dict(axes=[2, 3])),     # "cpu" backend only in the reference
    ("reduce_max_1", "ReduceMax", [1, 50, 70], [], dict(keepdims=0))])
def test_reduce(case, tmp_path, name, op_type, shape_x, shape_y, kw):
    case(f"reference test_{name}")
    sess = one_node(tmp_path, op_type, [("x", W.FLOAT, shape_x)], [("y", W.FLOAT, shape_y)], opset=13, **kw)
    x = rand(shape_x)
    (actual,) = sess.run(None, {"x": x})
    if op_type == "ReduceMean":
        expected = x.astype(np.float64).mean(tuple(kw["axes"]), keepdims=True)
    else:
        expected = x.max()
    assert np.allclose(expected, actual) and actual.size == np.asarray(expected).size
