"""Seeded random transformer-shaped graphs through the session, in every configuration.

Each graph strings together the pieces an exported encoder is made of, in random order and with random extra readers:
LayerNormalization (the operator, or the exporter's nine-node chain), linear layers with bias and activation,
residual Adds of any two earlier tensors of one shape, attention blocks in the exporters' variants (K^T through two
Transposes or one, the scale behind the product or on q, masks of five shapes), Softmax, Transposes there and back,
Reshapes to two dimensions around a product, Identity / Unsqueeze / Squeeze aliases.  Intermediate values are graph
outputs at random, which is what forces the session out of its planned shortcuts (a deferred Add, scores that were never
going to be stored, a tensor that was to leave as operand planes).

Checked per graph: the plain session (every node copies, fp32 products, no rewrite: the reference's semantics) against
the graph's definition evaluated in float64 by NumPy; then 18 other sessions against the plain one -- strided views
(bit for bit on the unrewritten graph, graph replay included), products on the bf16 route, the one-kernel attention,
each also behind the reference's rewrites (fuse_layer_norm, fuse_gelu) and behind all rewrites."""
import numpy as np
import pytest

from altius_amd import device as D
from altius_amd.graph import Model, Op, Tensor
from altius_amd.session import HipSessionBuilder

pytestmark = pytest.mark.gpu


def tanh_gelu(x):
    """The function the reference's Gelu computes (crates/session_interpreter/src/fast_math.rs:189-246)."""
    return 0.5 * x * (1 + np.tanh(np.sqrt(2 / np.pi) * (x + 0.044715 * x ** 3)))


def softmax(x):
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


class RandomGraph:
    """A model under construction together with every value's float64 definition."""

    def __init__(self, rng, open_batch=False):
        self.rng = rng
        self.open_batch = open_batch  # the input is declared without a shape and no node spells the batch out
        self.b = int(rng.choice([1, 2, 3, 8]))
        self.t = int(rng.choice([5, 16, 33, 45, 64, 197]))
        self.c = int(rng.choice([64, 128, 192, 256, 384]))
        self.m = Model(opset_version=13)
        self.ref, self.ops = {}, []
        x = self.m.new_val_named("x") if open_batch else self.m.new_val_named_and_shaped("x", [self.b, self.t, self.c])
        self.m.add_input(x)
        self.feed = (rng.standard_normal((self.b, self.t, self.c)) * 0.5).astype(np.float32)
        self.ref[x] = self.feed.astype(np.float64)
        self.input = x
        self.seen = [x]

    # --- building blocks ---------------------------------------------------------------------------------------
    def init(self, array):
        return self.m.new_initializer(np.ascontiguousarray(array))

    def scalar(self, value):
        """A one-value f32 initializer and the float64 of what it holds."""
        v = np.float32(value)
        return self.init(np.array(v, np.float32)), np.float64(v)

    def weights(self, *shape, scale=None):
        a = (self.rng.standard_normal(shape) * (scale if scale else 1.0 / np.sqrt(shape[0]))).astype(np.float32)
        return self.init(a), a.astype(np.float64)

    def node(self, op, inputs, define, n_out=1, **attrs):
        outs = [self.m.new_val() for _ in range(n_out)]
        self.m.add_node(op, inputs, outs, **attrs)
        results = define()
        for o, r in zip(outs, [results] if n_out == 1 else results):
            self.ref[o] = r
        self.ops.append(Op._NAMES[op])
        return outs[0] if n_out == 1 else outs

    def flip(self, p):
        return self.rng.random() < p

    def linear(self, v, cout, bias=True, act=None):
        w, wa = self.weights(self.ref[v].shape[-1], cout)
        y = self.node(Op.MatMul, [v, w], lambda: self.ref[v] @ wa)
        if bias:
            bi, ba = self.weights(cout, scale=0.1)
            y = self.node(Op.Add, [bi, y] if self.flip(0.5) else [y, bi], lambda y=y: self.ref[y] + ba)
        if act == "gelu":
            y = self.node(Op.Gelu, [y], lambda y=y: tanh_gelu(self.ref[y]))
        if act == "relu":
            y = self.node(Op.ReLU, [y], lambda y=y: np.maximum(self.ref[y], 0))
        return y

    def layernorm(self, v, as_operator):
        c = self.ref[v].shape[-1]
        ga = (1.0 + 0.1 * self.rng.standard_normal(c)).astype(np.float32)
        g, ga = self.init(ga), ga.astype(np.float64)
        bt, ba = self.weights(c, scale=0.1)

        def define():
            x = self.ref[v]
            mu = x.mean(-1, keepdims=True)
            var = ((x - mu) ** 2).mean(-1, keepdims=True)
            return (x - mu) / np.sqrt(var + 1e-5) * ga + ba

        if as_operator:
            return self.node(Op.LayerNormalization, [v, g, bt], define, axis=-1, epsilon=1e-5)
        ref = self.ref
        mu = self.node(Op.ReduceMean, [v], lambda: ref[v].mean(-1, keepdims=True), axes=[-1], keepdims=1)
        d = self.node(Op.Sub, [v, mu], lambda: ref[v] - ref[mu])
        two, _ = self.scalar(2.0)
        p = self.node(Op.Pow, [d, two], lambda: ref[d] ** 2)
        var = self.node(Op.ReduceMean, [p], lambda: ref[p].mean(-1, keepdims=True), axes=[-1], keepdims=1)
        eps, eps_v = self.scalar(1e-5)
        ve = self.node(Op.Add, [var, eps], lambda: ref[var] + eps_v)
        sd = self.node(Op.Sqrt, [ve], lambda: np.sqrt(ref[ve]))
        q = self.node(Op.Div, [d, sd], lambda: ref[d] / ref[sd])
        mg = self.node(Op.Mul, [q, g], lambda: ref[q] * ga)
        return self.node(Op.Add, [mg, bt], lambda: ref[mg] + ba)

    def attention(self, v):
        """Returns the block's result and the intermediates that were drawn to be graph outputs as well."""
        ref, rng = self.ref, self.rng
        b, t, c = ref[v].shape
        d = int(rng.choice([64, 64, 32, 16]))
        h = max(1, c // d)
        hd = h * d
        qkv = self.linear(v, 3 * hd, bias=self.flip(0.7))
        sizes = self.init(np.array([hd, hd, hd], np.int64))
        parts = self.node(Op.Split, [qkv, sizes], lambda: [ref[qkv][..., i * hd:(i + 1) * hd] for i in range(3)], 3, axis=2)
        heads = self.init(np.array([0, 0, h, d] if self.open_batch else [b, t, h, d], np.int64))

        def head(p):
            r = self.node(Op.Reshape, [p, heads], lambda: ref[p].reshape(b, t, h, d))
            return self.node(Op.Transpose, [r], lambda: ref[r].transpose(0, 2, 1, 3), perm=[0, 2, 1, 3])

        q, vv = head(parts[0]), head(parts[2])
        extra = [q] if self.flip(0.15) else []
        where_scale = rng.random()
        if where_scale >= 0.7:  # no scale behind the product: q carries it (unscaled scores make a chaotic Softmax)
            qs, qs_v = self.scalar(1 / np.sqrt(d))
            q0 = q
            q = self.node(Op.Mul, [q, qs], lambda: ref[q0] * qs_v)
        if self.flip(0.3):  # K^T straight from the reshaped part
            kr = self.node(Op.Reshape, [parts[1], heads], lambda: ref[parts[1]].reshape(b, t, h, d))
            kt = self.node(Op.Transpose, [kr], lambda: ref[kr].transpose(0, 2, 3, 1), perm=[0, 2, 3, 1])
        else:
            k = head(parts[1])
            kt = self.node(Op.Transpose, [k], lambda: ref[k].transpose(0, 1, 3, 2), perm=[0, 1, 3, 2])
        s = self.node(Op.MatMul, [q, kt], lambda: ref[q] @ ref[kt])
        if where_scale < 0.4:
            sc, sc_v = self.scalar(np.sqrt(d))
            s = self.node(Op.Div, [s, sc], lambda s=s: ref[s] / sc_v)
        elif where_scale < 0.7:
            sc, sc_v = self.scalar(1 / np.sqrt(d))
            s = self.node(Op.Mul, [s, sc], lambda s=s: ref[s] * sc_v)
        if self.flip(0.3):
            shape = [(b, 1, 1, t), (b, 1, 1, t), (1, 1, t, t), (b, 1, t, t), (t,)][int(rng.integers(0, 5))]
            if self.open_batch and len(shape) == 4:
                shape = (1, 1) + shape[2:]
            mask = np.where(rng.random(shape) < 0.2, -10000.0, 0.0).astype(np.float32)
            s = self.node(Op.Add, [s, self.init(mask)], lambda s=s: ref[s] + mask)
        if self.flip(0.1):
            extra.append(s)
        p = self.node(Op.Softmax, [s], lambda: softmax(ref[s]), axis=-1)
        if self.flip(0.1):
            extra.append(p)
        o = self.node(Op.MatMul, [p, vv], lambda: ref[p] @ ref[vv])
        ot = self.node(Op.Transpose, [o], lambda: ref[o].transpose(0, 2, 1, 3), perm=[0, 2, 1, 3])
        if self.flip(0.1):
            extra.append(ot)
        merged = self.init(np.array([0, 0, hd] if self.open_batch else [b, t, hd], np.int64))
        a = self.node(Op.Reshape, [ot, merged], lambda: ref[ot].reshape(b, t, hd))
        return self.linear(a, c, bias=self.flip(0.7)), extra

    # --- the graph -----------------------------------------------------------------------------------------------
    def grow(self):
        """Adds 3 to 9 blocks and declares the outputs; returns them."""
        ref, rng = self.ref, self.rng
        cur, outs = self.input, []
        for _ in range(int(rng.integers(3, 10))):
            r, z = rng.random(), cur
            if r < 0.2:
                cur = self.layernorm(cur, as_operator=self.flip(0.6))
            elif r < 0.4:
                c = ref[cur].shape[-1]
                hidden = int(rng.choice([c, 2 * c, 4 * c]))
                y = self.linear(cur, hidden, bias=self.flip(0.8), act=[None, "gelu", "relu"][int(rng.integers(0, 3))])
                cur = self.linear(y, c, bias=self.flip(0.8)) if hidden != c or self.flip(0.5) else y
            elif r < 0.6:
                cur, extra = self.attention(cur)
                outs += extra
            elif r < 0.8:
                same = [v for v in self.seen if ref[v].shape == ref[cur].shape and v != cur]
                if same:
                    other = same[int(rng.integers(0, len(same)))]
                    a, b = (cur, other) if self.flip(0.5) else (other, cur)
                    cur = self.node(Op.Add, [a, b], lambda a=a, b=b: ref[a] + ref[b])
            elif r < 0.87:
                cur = self.node(Op.Softmax, [cur], lambda: softmax(ref[z]), axis=-1)
            elif r < 0.94:
                sc, sc_v = self.scalar(1.7)
                cur = self.node(Op.Mul, [cur, sc], lambda: ref[z] * sc_v)
            elif r < 0.96:
                tr = self.node(Op.Transpose, [cur], lambda: ref[z].transpose(0, 2, 1), perm=[0, 2, 1])
                cur = self.node(Op.Transpose, [tr], lambda: ref[tr].transpose(0, 2, 1), perm=[0, 2, 1])
            elif r < 0.98:
                b, t, c = ref[z].shape
                flat = self.init(np.array([-1 if self.open_batch else b * t, c], np.int64))
                back = self.init(np.array([-1 if self.open_batch else b, t, c], np.int64))
                f = self.node(Op.Reshape, [cur, flat], lambda: ref[z].reshape(b * t, c))
                y = self.linear(f, c, bias=self.flip(0.5), act=[None, "gelu"][int(rng.integers(0, 2))])
                cur = self.node(Op.Reshape, [y, back], lambda: ref[y].reshape(b, t, c))
            else:
                alias = self.node(Op.Identity, [cur], lambda: ref[z])
                axis0 = self.init(np.array([0], np.int64))
                u = self.node(Op.Unsqueeze, [alias, axis0], lambda: ref[alias][None])
                cur = self.node(Op.Squeeze, [u, axis0], lambda: ref[u][0])
            self.seen.append(cur)
            if self.flip(0.12):
                outs.append(cur)
        outs.append(cur)
        chosen = []
        for o in outs:
            if o not in chosen and o != self.input:
                chosen.append(o)
        for o in chosen:
            self.m.add_output(o)
        return chosen


def run(model, feed, views=False, algorithm=D.GEMM_FP32, attention=False, replay=False):
    builder = HipSessionBuilder(model).with_strided_views(views).with_gemm_algorithm(algorithm)
    if attention:
        builder = builder.with_fused_attention(True)
    if replay:
        builder = builder.with_graph_replay(True)
    session = builder.build()
    try:
        for _ in range(4 if replay else 2):  # a second run reuses pooled blocks; replay starts with the third
            got = [np.array(t) for t in session.run([Tensor.from_numpy(feed)])]
    finally:
        session.close()
    return got


SESSIONS = [
    ("views", dict(views=True), True),
    ("views, graph replay", dict(views=True, replay=True), True),
    ("bf16 route", dict(views=True, algorithm=D.GEMM_BF16X3), False),
    ("bf16 route, one-kernel attention", dict(views=True, algorithm=D.GEMM_BF16X3, attention=True), False),
    ("one-kernel attention", dict(views=True, attention=True), False),
    ("automatic route, one-kernel attention", dict(views=True, algorithm=D.GEMM_AUTO, attention=True), False),
]


def reference_rewrites(m):
    m.fuse_layer_norm()
    m.fuse_gelu()


def all_rewrites(m):
    reference_rewrites(m)
    m.fuse_softmax_prologue()
    m.fuse_matmul_bias()
    m.fuse_transpose_matmul()
    m.fuse_elemwise_ops(extended=True)


REWRITES = [("as built", lambda m: None), ("reference rewrites", reference_rewrites), ("all rewrites", all_rewrites)]


@pytest.mark.parametrize("seed", range(40))
def test_random_encoder_graphs_in_every_session_configuration(case, seed):
    g = RandomGraph(np.random.default_rng(7000 + seed))
    outs = g.grow()
    case(f"random graph {seed}: [{g.b},{g.t},{g.c}], {len(g.ops)} nodes, {len(outs)} outputs: {' '.join(g.ops)}")
    if not g.ops:
        pytest.skip("the draw added no node")
    plain = run(g.m.clone(), g.feed)
    for i, o in enumerate(outs):
        want = g.ref[o]
        tol = 2e-3 * max(1.0, float(np.abs(want).max()))
        np.testing.assert_allclose(plain[i], want, rtol=2e-3, atol=tol, err_msg=f"plain session, output {i}")
    for rewrites, apply in REWRITES:
        model = g.m.clone()
        apply(model)
        for name, options, same_kernels in SESSIONS:
            got = run(model.clone(), g.feed, **options)
            for i in range(len(outs)):
                what = f"{rewrites}, {name}, output {i}"
                if same_kernels and rewrites == "as built":
                    assert got[i].tobytes() == plain[i].tobytes(), what
                else:
                    tol = 1e-3 * max(1.0, float(np.abs(plain[i]).max()))
                    np.testing.assert_allclose(got[i], plain[i], rtol=1e-3, atol=tol, err_msg=what)


@pytest.mark.parametrize("seed", range(12))
def test_one_session_fed_batches_of_changing_size(case, seed):
    """The input is declared without a shape (shapes are then inferred at every run, crates/core/src/analysis/
    shape.rs:704-706) and no node spells the batch out (Reshape targets use 0 and -1): one session of every
    configuration is fed six batches of four sizes in turn, and each result is held to a fresh plain session's on the
    same feed -- what a run leaves behind (pooled blocks, recorded graphs, plans made for another size) must not show."""
    rng = np.random.default_rng(9000 + seed)
    g = RandomGraph(rng, open_batch=True)
    outs = g.grow()
    case(f"random graph {seed}, open batch: [{g.b},{g.t},{g.c}], {len(g.ops)} nodes, {len(outs)} outputs: {' '.join(g.ops)}")
    if not g.ops:
        pytest.skip("the draw added no node")
    batches = [g.b, 1, g.b + 2, g.b, 2, g.b + 2]
    feeds = {b: (rng.standard_normal((b, g.t, g.c)) * 0.5).astype(np.float32) for b in set(batches)}
    plain = {b: run(g.m.clone(), feed) for b, feed in feeds.items()}
    first = run(g.m.clone(), g.feed)
    for i, o in enumerate(outs):
        tol = 2e-3 * max(1.0, float(np.abs(g.ref[o]).max()))
        np.testing.assert_allclose(first[i], g.ref[o], rtol=2e-3, atol=tol, err_msg=f"plain session, output {i}")
    for rewrites, apply in REWRITES:
        model = g.m.clone()
        apply(model)
        for name, options, same_kernels in SESSIONS:
            builder = HipSessionBuilder(model.clone()).with_strided_views(options.get("views", False))
            builder = builder.with_gemm_algorithm(options.get("algorithm", D.GEMM_FP32))
            builder = builder.with_fused_attention(options.get("attention", False)).with_graph_replay(options.get("replay", False))
            session = builder.build()
            try:
                for j, b in enumerate(batches):
                    got = [np.array(t) for t in session.run([Tensor.from_numpy(feeds[b])])]
                    for i in range(len(outs)):
                        what = f"{rewrites}, {name}, run {j} (batch {b}), output {i}"
                        want = plain[b][i]
                        if same_kernels and rewrites == "as built":
                            assert got[i].tobytes() == want.tobytes(), what
                        else:
                            tol = 1e-3 * max(1.0, float(np.abs(want).max()))
                            np.testing.assert_allclose(got[i], want, rtol=1e-3, atol=tol, err_msg=what)
            finally:
                session.close()
