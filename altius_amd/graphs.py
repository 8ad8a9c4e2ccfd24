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


def vit_encoder(batch, layers=12, hidden=768, heads=12, mlp=3072, tokens=197, classes=1000, seed=0):
    """A ViT-B/16-shaped encoder stack the way exporters write it (9-node LayerNorm chains, MatMul + Add, head
    split by Reshape / Transpose, QK^T, Mul by 1/sqrt(d), Softmax, 5-node erf-GELU chains), a final LayerNorm,
    the class token and a Gemm head, with random weights.  Input: embedded tokens [batch, tokens, hidden]."""
    rng = np.random.default_rng(seed)
    w = lambda *shape, scale=0.02: (rng.standard_normal(shape) * scale).astype(np.float32)
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("tokens", [batch, tokens, hidden])
    m.add_input(x)
    d = hidden // heads
    i64 = lambda *v: m.new_initializer(np.array(v, np.int64))

    def node(op, inputs, **attrs):
        out = m.new_val()
        m.add_node(op, inputs, [out], **attrs)
        return out

    def linear(v, n_in, n_out):
        return node(Op.Add, [node(Op.MatMul, [v, m.new_initializer(w(n_in, n_out))]), m.new_initializer(w(n_out))])

    def norm(v):
        return layer_norm_chain(m, v, 1 + w(hidden), w(hidden), eps=1e-6)[0]

    cur = x
    for _ in range(layers):
        qkv = linear(norm(cur), hidden, 3 * hidden)
        parts = [m.new_val() for _ in range(3)]
        m.add_node(Op.Split, [qkv, i64(hidden, hidden, hidden)], parts, axis=2)
        q, k, v = (node(Op.Transpose, [node(Op.Reshape, [p, i64(batch, tokens, heads, d)])], perm=[0, 2, 1, 3]) for p in parts)
        s = node(Op.MatMul, [q, node(Op.Transpose, [k], perm=[0, 1, 3, 2])])
        s = node(Op.Softmax, [node(Op.Mul, [s, m.new_initializer(np.array(d ** -0.5, np.float32))])], axis=-1)
        a = node(Op.Reshape, [node(Op.Transpose, [node(Op.MatMul, [s, v])], perm=[0, 2, 1, 3]), i64(batch, tokens, hidden)])
        cur = node(Op.Add, [cur, linear(a, hidden, hidden)])
        h = erf_gelu_chain(m, linear(norm(cur), hidden, mlp))
        cur = node(Op.Add, [cur, linear(h, mlp, hidden)])
    cls = node(Op.Gather, [norm(cur), m.new_initializer(np.array(0, np.int64))], axis=1)
    logits = node(Op.Gemm, [cls, m.new_initializer(w(classes, hidden)), m.new_initializer(w(classes))], trans_b=True)
    m.add_output(logits)
    return m
