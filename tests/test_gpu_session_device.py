"""HipSession.run_device: the session on tensors that already live on the GPU (no PCIe inside the
call, no wait for the GPU).  Results must be the bits of run() on the same data; outputs can feed
another session; memory handed out survives the session object."""
import numpy as np
import pytest

from altius_amd import synth
from altius_amd._lib import ERR_ARG, ERR_SHAPE, AltiusHipError
from altius_amd.device import Context
from altius_amd.graph import I64, Model, Op
from altius_amd.graphs import erf_gelu_chain, layer_norm_chain, single_input_model
from altius_amd.session import HipSessionBuilder
from conftest import assert_bits_equal

pytestmark = pytest.mark.gpu


def chain_model(c):
    return single_input_model(c["x"].shape, lambda m, x: layer_norm_chain(m, x, c["gamma"], c["beta"])[0])


def test_device_run_equals_host_run(case, ctx):
    case("run_device: layernorm chain")
    c = synth.cfg2(batch=2)
    sess = HipSessionBuilder(chain_model(c)).build()
    (want,) = sess.run([c["x"]])
    d_x = ctx.upload(c["x"])
    for i in range(3):
        (out,) = sess.run_device([(d_x.ptr, c["x"].shape, np.float32)])
        assert out.shape == want.shape and out.dtype == np.float32 and out.nbytes == want.nbytes
        sess.synchronize()
        assert sess.last_device_ms() > 0
        assert_bits_equal(ctx.download(out, out.shape), want, f"device run {i}")
        if i == 0:
            allocs = sess.device_allocations()
        out.free()
    assert sess.device_allocations() == allocs            # steady state: the pool serves outputs too
    ctx.free(d_x)


def test_a_session_without_its_timing_events_runs_the_same(case, ctx):
    """with_device_timing(False): no pair of events around a run, last_device_ms() reports 0, results and the
    prepared-arguments route unchanged."""
    case("run_device without device timing")
    c = synth.cfg2(batch=2)
    timed = HipSessionBuilder(chain_model(c)).build()
    plain = HipSessionBuilder(chain_model(c)).with_device_timing(False).build()
    (want,) = timed.run([c["x"]])
    (got,) = plain.run([c["x"]])
    assert_bits_equal(got, want, "run() without timing events")
    assert timed.last_device_ms() > 0 and plain.last_device_ms() == 0
    d_x = ctx.upload(c["x"])
    prepared = plain.prepare_device_inputs([(d_x.ptr, c["x"].shape, np.float32)])
    for i in range(3):
        (out,) = plain.run_device_prepared(prepared)
        plain.synchronize()
        assert plain.last_device_ms() == 0
        assert_bits_equal(ctx.download(out, out.shape), want, f"prepared device run {i}")
        out.free()
    ctx.free(d_x)


def test_outputs_feed_another_session_and_outlive_theirs(case, ctx):
    """LayerNorm chain on one session, erf-GELU chain on another, device to device; the first session
    is closed before its output is read or freed."""
    case("run_device: two sessions chained")
    c = synth.cfg2(batch=2)
    ln = HipSessionBuilder(chain_model(c)).build()
    gelu = HipSessionBuilder(single_input_model(c["x"].shape, lambda m, x: erf_gelu_chain(m, x))).build()
    (mid_want,) = ln.run([c["x"]])
    (want,) = gelu.run([mid_want])
    d_x = ctx.upload(c["x"])
    (mid,) = ln.run_device([(d_x.ptr, c["x"].shape, np.float32)])
    ln.synchronize()                                      # the sessions use different streams
    (out,) = gelu.run_device([(mid.ptr, mid.shape, mid.dtype)])
    gelu.synchronize()
    ln.close()
    assert_bits_equal(ctx.download(mid, mid.shape), mid_want, "first session's output after close()")
    assert_bits_equal(ctx.download(out, out.shape), want, "second session's output")
    mid.free()
    out.free()
    ctx.free(d_x)


def test_view_of_an_input_is_the_callers_pointer(case, ctx):
    case("run_device: aliasing output, two outputs, integer input")
    x = synth.normal(4, [6, 10, 8])
    idx = np.array([[5, 0, -1], [2, 2, 3]], np.int64)
    m = Model()
    vx = m.new_val_named_and_shaped("x", x.shape)
    vi = m.new_val_named_and_shaped("idx", idx.shape, I64)
    flat, picked = m.new_val(), m.new_val()
    m.add_node(Op.Reshape, [vx, m.new_initializer(np.array([6, 80], np.int64))], [flat])
    m.add_node(Op.Gather, [vx, vi], [picked], axis=0)
    m.add_input(vx)
    m.add_input(vi)
    m.add_output(flat)
    m.add_output(picked)
    sess = HipSessionBuilder(m).build()
    d_x, d_i = ctx.upload(x), ctx.upload(idx)
    flat_out, picked_out = sess.run_device([(d_x.ptr, x.shape, np.float32), (d_i.ptr, idx.shape, np.int64)])
    sess.synchronize()
    assert flat_out.ptr == d_x.ptr and flat_out.shape == (6, 80)
    assert picked_out.shape == (2, 3, 10, 8)
    assert_bits_equal(ctx.download(picked_out, picked_out.shape), x[idx], "gather on device inputs")
    flat_out.free()                                       # not the pool's memory: the caller's buffer is untouched
    assert_bits_equal(ctx.download(d_x, x.shape), x, "input after freeing its view")
    picked_out.free()

    # An out-of-range index is found by the kernel and reported when the caller synchronises.
    bad = idx.copy()
    bad[1, 1] = 6
    d_bad = ctx.upload(bad)
    outs = sess.run_device([(d_x.ptr, x.shape, np.float32), (d_bad.ptr, bad.shape, np.int64)])
    with pytest.raises(AltiusHipError) as e:
        sess.synchronize()
    assert e.value.code == ERR_ARG and "Gather" in e.value.message
    for o in outs:
        o.free()
    (_, again) = sess.run([x, idx])                        # the session is still usable, host path too
    assert_bits_equal(again, x[idx], "host run after a device-side error")
    for b in (d_x, d_i, d_bad):
        ctx.free(b)


def test_run_device_argument_errors(case, ctx):
    case("run_device: errors")
    c = synth.cfg2(batch=1)
    sess = HipSessionBuilder(chain_model(c)).build()
    with pytest.raises(AltiusHipError) as e:
        sess.run_device([])
    assert e.value.code == ERR_ARG
    with pytest.raises(AltiusHipError) as e:
        sess.run_device([(0, c["x"].shape, np.float32)])
    assert e.value.code == ERR_ARG and "device pointer" in e.value.message
    # A tensor that is not of the declared shape or element type is refused before any kernel is sized by
    # the shapes derived from the declaration.
    d = ctx.upload(np.zeros([3, 768], np.float32))
    for shape, dtype in (((3, 768), np.float32), (c["x"].shape, np.int32)):
        with pytest.raises(AltiusHipError) as e:
            sess.run_device([(d.ptr, shape, dtype)])
        assert e.value.code == ERR_SHAPE and "declares" in e.value.message
    with pytest.raises(AltiusHipError) as e:
        sess.run([np.zeros([3, 768], np.float32)])
    assert e.value.code == ERR_SHAPE
    sess.synchronize()
    ctx.free(d)
