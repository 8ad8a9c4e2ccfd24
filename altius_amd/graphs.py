"""The graph fragments of the benchmark configurations, as ONNX exporters emit them.

Used by the tests (fusion passes, session parity) and by bench.py (session-level timing)."""
import numpy as np

from .graph import Model, Op


def layer_norm_chain(m, x, gamma, beta, eps=1e-5):
    """The 9-node chain ONNX exporters emit for LayerNorm (crates/core/src/optimize/layer_norm_fusion.rs:9-16).
    Returns (output value, gamma initializer, beta initializer)."""
    two = m.new_initializer(np.array(2.0, np.float32))
    e = m.new_initializer(np.array(eps, np.float32))
    g = m.new_initializer(gamma)
    b = m.new_initializer(beta)
    v = [m.new_val() for _ in range(9)]
    m.add_node(Op.ReduceMean, [x], [v[0]], axes=[-1], keep_dims=True)
    m.add_node(Op.Sub, [x, v[0]], [v[1]])
    m.add_node(Op.Pow, [v[1], two], [v[2]])
    m.add_node(Op.ReduceMean, [v[2]], [v[3]], axes=[-1], keep_dims=True)
    m.add_node(Op.Add, [v[3], e], [v[4]])
    m.add_node(Op.Sqrt, [v[4]], [v[5]])
    m.add_node(Op.Div, [v[1], v[5]], [v[6]])
    m.add_node(Op.Mul, [v[6], g], [v[7]])
    m.add_node(Op.Add, [v[7], b], [v[8]])
    return v[8], g, b


def erf_gelu_chain(m, x, sqrt2=1.4142135):
    """Div(x, sqrt 2) -> Erf -> Add 1 -> Mul x -> Mul 0.5 (crates/core/src/optimize/gelu_fusion.rs:12-82)."""
    c = m.new_initializer(np.array(sqrt2, np.float32))
    one = m.new_initializer(np.array(1.0, np.float32))
    half = m.new_initializer(np.array(0.5, np.float32))
    v = [m.new_val() for _ in range(5)]
    m.add_node(Op.Div, [x, c], [v[0]])
    m.add_node(Op.Erf, [v[0]], [v[1]])
    m.add_node(Op.Add, [v[1], one], [v[2]])
    m.add_node(Op.Mul, [x, v[2]], [v[3]])
    m.add_node(Op.Mul, [v[3], half], [v[4]])
    return v[4]


def squeeze_excite(m, x, alpha, beta):
    """ReduceMean over H,W (keepdims) -> HardSigmoid -> Mul back onto the NCHW input."""
    s, h, y = m.new_val(), m.new_val(), m.new_val()
    m.add_node(Op.ReduceMean, [x], [s], axes=[2, 3], keep_dims=True)
    m.add_node(Op.HardSigmoid, [s], [h], alpha=float(alpha), beta=float(beta))
    m.add_node(Op.Mul, [x, h], [y])
    return y


def single_input_model(shape, body):
    """A model with one shaped input `x` and one output, the value `body(model, x)` returns."""
    m = Model()
    x = m.new_val_named_and_shaped("x", list(shape))
    out = body(m, x)
    m.add_input(x)
    m.add_output(out)
    return m
