"""Sessions built with_graph_replay(): a run is recorded as a HIP graph the second time a set of
input shapes is seen and replayed afterwards.  Every replay must give the bits of the node-by-node
run, for fresh inputs each time, with other GPU work and synchronisations in between; graphs that
need the host during a run must keep running node by node."""
import numpy as np
import pytest

import oracle as O
from altius_amd import synth
from altius_amd._lib import AltiusHipError
from altius_amd.graph import I64, Model, Op
from altius_amd.graphs import erf_gelu_chain, layer_norm_chain, single_input_model, squeeze_excite
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu


def chain_model(shape, gamma, beta):
    return single_input_model(shape, lambda m, x: layer_norm_chain(m, x, gamma, beta)[0])


def test_replay_matches_eager_for_fresh_inputs(case):
    """The 9-node LayerNorm chain: runs 1 (eager), 2 (recorded, then replayed) and 3..6 (replayed)
    against an eager session on the same bytes; another session works on the GPU between replays."""
    case("graph replay: layernorm chain")
    c = synth.cfg2(batch=2)
    shape = c["x"].shape
    eager = HipSessionBuilder(chain_model(shape, c["gamma"], c["beta"])).build()
    sess = HipSessionBuilder(chain_model(shape, c["gamma"], c["beta"])).with_graph_replay().build()
    other = HipSessionBuilder(single_input_model(shape, lambda m, x: erf_gelu_chain(m, x))).build()
    for i in range(6):
        x = synth.normal(100 + i, shape, std=1.0 + i)
        (want,) = eager.run([x])
        (got,) = sess.run([x])
        assert_bits_equal(got, want, f"run {i}")
        other.run([x])                                   # eager kernels and a synchronisation between replays
        assert sess.graph_replays() == max(0, i)         # run 0 is eager; run 1 records and replays
    allocs = sess.device_allocations()
    (got,) = sess.run([c["x"]])
    assert sess.device_allocations() == allocs           # replays allocate nothing on the device


def test_one_graph_per_input_shape(case):
    """A second batch size is its own signature: eager once, then recorded; the first keeps replaying."""
    case("graph replay: two shapes")
    m = Model()
    x = m.new_val_named("x")                            # no declared shape: inferred from the input at run time
    y = m.new_val()
    m.add_node(Op.Softmax, [x], [y], axis=-1)
    m.add_input(x)
    m.add_output(y)
    sess = HipSessionBuilder(m).with_graph_replay().build()
    eager = HipSessionBuilder(m.clone()).build()
    a = [synth.normal(i, [3, 12, 197, 197], std=0.5) for i in range(3)]
    b = [synth.normal(10 + i, [5, 40], std=2.0) for i in range(3)]
    for i in range(3):
        for x_in in (a[i], b[i]):
            (got,) = sess.run([x_in])
            (want,) = eager.run([x_in])
            assert_bits_equal(got, want, f"softmax {x_in.shape} run {i}")
    # Shapes that are only known at run time are not recorded: all six runs were node by node.
    assert sess.graph_replays() == 0


def test_declared_shapes_with_two_outputs_and_scratch(case):
    """Squeeze-excite plus an all-axes ReduceMax (two-stage through the context's scratch buffer) and
    a second output; the recorded graph writes both outputs on every replay."""
    case("graph replay: two outputs, scratch")
    c = synth.cfg3(batch=4)
    m = Model()
    x = m.new_val_named_and_shaped("se", c["se"].shape)
    y = squeeze_excite(m, x, c["alpha"], c["beta"])
    mx = m.new_val()
    m.add_node(Op.ReduceMax, [y], [mx], axes=[], keep_dims=False)
    m.add_input(x)
    m.add_output(y)
    m.add_output(mx)
    sess = HipSessionBuilder(m).with_graph_replay().build()
    eager = HipSessionBuilder(m.clone()).build()
    for i in range(4):
        x_in = synth.normal(50 + i, c["se"].shape, std=1.0 + 0.5 * i)
        want = eager.run([x_in])
        got = sess.run([x_in])
        assert_bits_equal(got[0], want[0], f"se run {i}")
        assert_bits_equal(got[1], want[1], f"max run {i}")
        assert_bits_equal(got[1], np.array([want[0].max()], np.float32), f"max of output run {i}")
    assert sess.graph_replays() == 3


def test_host_shape_arithmetic_keeps_running_node_by_node(case):
    """Shape -> Gather -> Concat -> Reshape needs tensor contents on the host while the run is built:
    such a graph is never recorded, and says so by its replay count."""
    case("graph replay: refused for host-evaluated nodes")
    m = Model()
    x = m.new_val_named("x")
    shp, b, tgt, y, z = (m.new_val() for _ in range(5))
    m.add_node(Op.Shape, [x], [shp])
    m.add_node(Op.Gather, [shp, m.new_initializer(np.array([0], np.int64))], [b], axis=0)
    m.add_node(Op.Concat, [b, m.new_initializer(np.array([-1], np.int64))], [tgt], axis=0)
    m.add_node(Op.Reshape, [x, tgt], [y])
    m.add_node(Op.ReLU, [y], [z])
    m.add_input(x)
    m.add_output(z)
    sess = HipSessionBuilder(m).with_graph_replay().build()
    for i in range(4):
        x_in = synth.normal(i, [4, 6, 10])
        (got,) = sess.run([x_in])
        assert_bits_equal(got, np.maximum(x_in, 0).reshape(4, 60), f"run {i}")
    assert sess.graph_replays() == 0


def test_gather_index_error_is_reported_on_replay(case):
    """An out-of-range Gather index is found by the kernel (a device flag); a replayed run reports it
    like a node-by-node run, and the session stays usable."""
    case("graph replay: gather flag")
    table = synth.normal(3, [100, 64])
    m = Model()
    idx = m.new_val_named_and_shaped("idx", [4, 5000], I64)     # too large for host arithmetic: runs on the GPU
    y = m.new_val()
    m.add_node(Op.Gather, [m.new_initializer(table), idx], [y], axis=0)
    m.add_input(idx)
    m.add_output(y)
    sess = HipSessionBuilder(m).with_graph_replay().build()
    rng = np.random.default_rng(5)
    good = [rng.integers(-100, 100, size=(4, 5000), dtype=np.int64) for _ in range(4)]
    bad = good[0].copy()
    bad[2, 17] = 100
    for i in range(3):
        (got,) = sess.run([good[i]])
        assert_bits_equal(got, table[good[i]], f"gather run {i}")
    assert sess.graph_replays() == 2
    with pytest.raises(AltiusHipError) as e:
        sess.run([bad])
    assert "Gather" in e.value.message or "index" in e.value.message
    (got,) = sess.run([good[3]])
    assert_bits_equal(got, table[good[3]], "gather after the error")


def test_profiled_session_is_not_recorded(case):
    case("graph replay: profiling wins")
    c = synth.cfg2(batch=1)
    sess = HipSessionBuilder(chain_model(c["x"].shape, c["gamma"], c["beta"])).with_graph_replay().with_profiling_enabled(True).build()
    for _ in range(3):
        sess.run([c["x"]])
    assert sess.graph_replays() == 0 and sess.profile()


def test_replay_of_an_encoder_layer_with_views_attention_and_the_bf16_route(case):
    """A ViT-style encoder layer (two shapes, the second one larger so that the GEMM workspace grows and recorded
    graphs have to be dropped): strided views, the deferred Gelu, the one-kernel attention and the bf16 GEMM route with
    its workspace and cached weight planes, eager against replayed, bit for bit, on fresh inputs."""
    from altius_amd import device as D
    from altius_amd import graphs

    case("graph replay: encoder layer")
    sessions = {}
    for batch in (2, 5):
        m = graphs.vit_encoder(batch, layers=1, tokens=50, classes=10)
        m.fuse_layer_norm(), m.fuse_gelu(), m.fuse_softmax_prologue(), m.fuse_matmul_bias(), m.fuse_transpose_matmul()
        m.fuse_elemwise_ops(extended=True)
        sessions[batch] = (HipSessionBuilder(m.clone()).with_gemm_algorithm(D.GEMM_BF16X3).with_fused_attention().build(),
                           HipSessionBuilder(m).with_gemm_algorithm(D.GEMM_BF16X3).with_fused_attention().with_graph_replay().build())
    for i in range(4):
        for batch, (eager, replayed) in sessions.items():
            x = synth.normal(50 + i, [batch, 50, 768], std=1.0)
            (want,) = eager.run([x])
            (got,) = replayed.run([x])
            assert_bits_equal(got, want, f"batch {batch} run {i}")
            assert eager.copies_avoided() >= 8          # Split, 3 head transposes, first product, Softmax, merge transpose, Gelu
    for eager, replayed in sessions.values():
        assert replayed.graph_replays() >= 2
        eager.close()
        replayed.close()



def test_device_resident_outputs_survive_replays(case, ctx):
    """A recorded graph addresses its intermediates directly.  The blocks they lived in must stay out of the pool
    while the graph exists: outputs of run_device() that the caller holds across replayed run() calls keep their
    bytes.  (The pool hands blocks out last-in first-out, so outputs are freed and held in turn here: that is what
    makes a later output land in a block an earlier run used for an intermediate.)"""
    case("graph replay: run_device outputs held across replays")
    c = synth.cfg2(batch=2)
    shape = c["x"].shape
    sess = HipSessionBuilder(chain_model(shape, c["gamma"], c["beta"])).with_graph_replay().build()
    eager = HipSessionBuilder(chain_model(shape, c["gamma"], c["beta"])).build()
    xs = [synth.normal(300 + i, shape, std=1.0 + i) for i in range(6)]
    for i in range(3):                                    # eager, recorded, replayed
        (got,) = sess.run([xs[i]])
        assert_bits_equal(got, eager.run([xs[i]])[0], f"run {i}")
    assert sess.graph_replays() == 2
    want = [eager.run([xs[3 + i]])[0] for i in range(3)]
    d_in = [ctx.upload(xs[3 + i]) for i in range(3)]
    held = []
    for i in range(12):
        (out,) = sess.run_device([(d_in[i % 3].ptr, shape, np.float32)])
        if i % 2 == 0:
            sess.synchronize()
            out.free()                                    # back to the pool: the next run's blocks come in another order
        else:
            held.append((i % 3, out))
    sess.synchronize()
    for i in range(4):
        (got,) = sess.run([xs[i]])                        # replays: the recorded kernels write their intermediates again
        assert_bits_equal(got, eager.run([xs[i]])[0], f"replay {i}")
    assert sess.graph_replays() == 6
    for n, (i, out) in enumerate(held):
        assert_bits_equal(ctx.download(out, shape), want[i], f"held output {n} after the replays")
        out.free()
    for b in d_in:
        ctx.free(b)
