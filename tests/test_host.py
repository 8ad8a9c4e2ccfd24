"""Host-side logic behind the C ABI, no GPU needed: the library loads and exports every
symbol the header declares, broadcasting index math, graph IR, topological order, execution
plan, shape inference and the fusion passes.  Expectations come from the reference's own unit
tests and from the documented behaviour of its functions (cited per test)."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest

from altius_amd import _lib
from altius_amd import device as D
from altius_amd._lib import ERR_ARG, ERR_OOM, ERR_SHAPE, AltiusHipError
from altius_amd.graph import F32, I64, Model, Op, Tensor, host_pool_stats, host_pool_trim
from altius_amd.graphs import erf_gelu_chain, layer_norm_chain

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "altius_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(ahip_[a-z0-9_]+)\s*\(", header))
    assert len(names) >= 60
    L = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(L, n)]
    assert not missing, f"declared but not exported: {missing}"


def test_no_cpu_fallback_when_library_is_missing(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libaltius_hip.so"))
    with pytest.raises(ImportError):
        _lib.lib()


def test_in_kernel_k_cut_is_allowed_only_on_a_round_robin_placement():
    """The bf16 GEMM combines the slices of a tile inside one XCD's L2 only if the probe launch showed blocks 0..7
    on eight different XCDs, every block i where block i % 8 ran, and a CU count that is a multiple of eight;
    anything else switches the cut off.  Where the turn starts does not matter (on the part it starts where the
    queue's previous launch stopped)."""
    ids = np.arange(4096, dtype=np.uint32)
    rr = ids % 8
    assert D.xcd_round_robin_holds(256, rr)
    assert D.xcd_round_robin_holds(64, rr[:16])
    for start in range(1, 8):
        assert D.xcd_round_robin_holds(256, (ids + start) % 8), start     # the turn may start at any XCD
    assert D.xcd_round_robin_holds(256, np.array([3, 1, 4, 0, 5, 7, 2, 6], np.uint32)[ids % 8])  # any fixed order of the eight
    assert not D.xcd_round_robin_holds(256, rr[:8])          # one round of eight says nothing
    assert not D.xcd_round_robin_holds(256, [])
    for cus in (0, 4, 7, 250, 255, 257, 300, -8):             # not eight equal XCDs
        assert not D.xcd_round_robin_holds(cus, rr), cus
    one_off = rr.copy()
    one_off[4095] = 0                                         # a single misplaced block, the last one
    assert not D.xcd_round_robin_holds(256, one_off)
    one_off = rr.copy()
    one_off[9] = 2
    assert not D.xcd_round_robin_holds(256, one_off)
    assert not D.xcd_round_robin_holds(256, np.zeros(4096, np.uint32))   # one XCD for everything
    assert not D.xcd_round_robin_holds(256, ids // 512)                  # contiguous runs per XCD
    assert not D.xcd_round_robin_holds(256, ids % 4)                     # four XCDs
    assert not D.xcd_round_robin_holds(256, ids % 16)                    # ids no eight-XCD part has
    drift = (ids + ids // 1000) % 8                                      # the turn slips by one every 1000 blocks
    assert not D.xcd_round_robin_holds(256, drift)
    never_ran = rr.copy()
    never_ran[100] = 0xFFFFFFFF                               # the probe's fill value: that block wrote nothing
    assert not D.xcd_round_robin_holds(256, never_ran)
    never_ran = rr.copy()
    never_ran[3] = 0xFFFFFFFF
    assert not D.xcd_round_robin_holds(256, never_ran)


def test_broadcast_reference_unit_tests():
    """crates/core/src/fixed_dim.rs:192-245."""
    assert D.broadcast_shape([1], [1]) == [1]
    assert D.broadcast_shape([1], [4, 1]) == [4, 1]
    assert D.broadcast_shape([4, 1], [1]) == [4, 1]
    with pytest.raises(AltiusHipError) as e:
        D.broadcast_shape([10, 20, 30], [10, 20])
    assert e.value.code == ERR_SHAPE
    assert D.broadcast_shape([1, 3, 3], [5, 1, 3, 3]) == [5, 1, 3, 3]
    assert D.broadcast_shape([1, 3, 1], [5, 3, 10]) == [5, 3, 10]
    assert D.broadcast_shape([1, 3, 4, 4], [3, 1, 1]) == [1, 3, 4, 4]
    assert D.broadcast_shape([], []) == []


@pytest.mark.parametrize("a,b", [
    ([1, 3, 28, 28], [3, 1, 1]), ([1, 12, 9, 9], [1, 1, 1, 9]), ([4, 1, 2], [3, 1]), ([3, 28, 28], [3, 28, 1]),
    ([3, 15, 15], [15]), ([3, 28, 28], [1]), ([1, 197, 768], [768]), ([256, 12, 197, 197], [256, 1, 1, 197]),
    ([32, 197, 768], [32, 197, 1]), ([32, 576, 7, 7], [32, 576, 1, 1]), ([5, 1, 7, 1, 3], [1, 6, 1, 2, 3]), ([2, 3], []),
])
def test_strides_agree_with_oracle_and_numpy(oracle, a, b):
    """Tensor::strides_for_broadcasting (crates/core/src/tensor.rs:369-406): integer, must be exact."""
    out = D.broadcast_shape(a, b)
    assert tuple(out) == np.broadcast_shapes(tuple(a), tuple(b))
    for src in (a, b):
        assert D.strides_for_broadcasting(src, out) == oracle.strides_for_broadcasting(src, out)
    assert D.strides_for_broadcasting([256, 1, 1, 197], [256, 12, 197, 197]) == [197, 0, 0, 1]
    with pytest.raises(AltiusHipError):
        D.strides_for_broadcasting([3, 1, 2], [1, 3, 28, 28])


def chain_model():
    """x -> Relu -> Sigmoid -> (Add with x) -> out, plus a side branch that is a second output."""
    m = Model()
    x = m.new_val_named_and_shaped("x", [2, 3])
    a, b, c, d = (m.new_val_named(n) for n in "abcd")
    n_add = m.add_node(Op.Add, [b, x], [c], name="add")     # added first: order must come from the data flow
    n_relu = m.add_node(Op.ReLU, [x], [a], name="relu")
    n_sig = m.add_node(Op.Sigmoid, [a], [b], name="sigmoid")
    n_sqrt = m.add_node(Op.Sqrt, [a], [d], name="sqrt")
    m.add_input(x)
    m.add_output(c)
    m.add_output(d)
    return m, (x, a, b, c, d), (n_add, n_relu, n_sig, n_sqrt)


def test_graph_round_trip_and_named_lookup():
    m, (x, a, b, c, d), (n_add, n_relu, n_sig, n_sqrt) = chain_model()
    assert m.inputs == [x] and m.outputs == [c, d]
    assert m.lookup_named_value("b") == b and m.lookup_named_value("nope") is None
    node = m.node(n_add)
    assert node["op_name"] == "Add" and node["inputs"] == [b, x] and node["outputs"] == [c]
    assert [_lib.lib().ahip_op_name(i).decode() for i in (Op.ReLU, Op.LayerNormalization, Op.FusedElemwise)] == [
        "ReLU", "LayerNormalization", "FusedElemwise"]  # Op::name (crates/core/src/op.rs:324-376)


def test_topological_order_and_execution_plan():
    """create_execution_plan (crates/session/src/plan.rs:14-58): each value is freed after its last
    reader; graph outputs are never freed."""
    m, (x, a, b, c, d), (n_add, n_relu, n_sig, n_sqrt) = chain_model()
    order = m.topo_sort_nodes()
    assert sorted(order) == sorted([n_add, n_relu, n_sig, n_sqrt])
    pos = {n: i for i, n in enumerate(order)}
    assert pos[n_relu] < pos[n_sig] < pos[n_add] and pos[n_relu] < pos[n_sqrt]
    plan = m.execution_plan()
    assert [n for n, _ in plan] == order
    frees = {n: f for n, f in plan}
    last_reader_of_a = n_sig if pos[n_sig] > pos[n_sqrt] else n_sqrt
    assert frees[last_reader_of_a] == [a]
    assert frees[n_add] == [b]
    assert all(v not in (c, d, x) for f in frees.values() for v in f)


def test_shape_inference():
    """crates/core/src/analysis/shape.rs:89-94, 354-411, 590-611."""
    m = Model(opset_version=13)
    x = m.new_val_named_and_shaped("x", [4, 12, 197, 197])
    mask = m.new_val_named_and_shaped("mask", [4, 1, 1, 197])
    y = m.new_val_named_and_shaped("y", [4, 768, 197])
    s, p, r1, r2, r3, r4 = (m.new_val() for _ in range(6))
    m.add_node(Op.Add, [x, mask], [s])
    m.add_node(Op.Softmax, [s], [p], axis=-1)
    m.add_node(Op.ReduceMax, [y], [r1], axes=[1], keep_dims=False)
    m.add_node(Op.ReduceMax, [y], [r2], axes=[], keep_dims=False)
    m.add_node(Op.ReduceMean, [y], [r3], axes=[-1], keep_dims=True)
    m.add_node(Op.ReduceMean, [y], [r4], axes=[], keep_dims=True)
    for v in (x, mask, y):
        m.add_input(v)
    assert m.infer_value_shape(s) == ([4, 12, 197, 197], F32)
    assert m.infer_value_shape(p) == ([4, 12, 197, 197], F32)
    assert m.infer_value_shape(r1) == ([4, 197], F32)
    assert m.infer_value_shape(r2) == ([1], F32)            # full reduction without keepdims -> [1]
    assert m.infer_value_shape(r3) == ([4, 768, 1], F32)
    assert m.infer_value_shape(r4) == ([4, 768, 197], F32)  # ReduceMean without axes reduces nothing


def test_shape_inference_errors_are_values_not_aborts():
    m = Model()
    a = m.new_val_named_and_shaped("a", [1, 3, 28, 28])
    b = m.new_val_named_and_shaped("b", [3, 1, 2])
    c = m.new_val()
    m.add_node(Op.Add, [a, b], [c])
    m.add_input(a)
    m.add_input(b)
    with pytest.raises(AltiusHipError) as e:  # the reference unwrap()s None here and panics
        m.infer_value_shape(c)
    assert e.value.code == ERR_SHAPE and "broadcast" in e.value.message

    m = Model()
    a = m.new_val_named_and_shaped("a", [None, 3])  # dynamic dimension: "Must be fixed dimension" (shape.rs:675)
    c = m.new_val()
    m.add_node(Op.ReLU, [a], [c])
    m.add_input(a)
    with pytest.raises(AltiusHipError) as e:
        m.infer_value_shape(c)
    assert e.value.code == ERR_SHAPE

    m = Model()
    a = m.new_val_named("a")  # no declared shape: nodes are skipped, inferred at run time (shape.rs:704-706)
    c = m.new_val()
    m.add_node(Op.ReLU, [a], [c])
    m.add_input(a)
    with pytest.raises(AltiusHipError) as e:
        m.infer_value_shape(c)
    assert e.value.code == ERR_ARG

    m = Model(opset_version=18)  # ReduceMax asserts opset <= 13 (shape.rs:355)
    a = m.new_val_named_and_shaped("a", [2, 3])
    c = m.new_val()
    m.add_node(Op.ReduceMax, [a], [c], axes=[1])
    m.add_input(a)
    with pytest.raises(AltiusHipError):
        m.infer_value_shape(c)

    m = Model()
    a = m.new_val_named_and_shaped("a", [2, 3])
    c = m.new_val()
    m.add_node(Op.MatMul, [a, a], [c])  # outside this backend
    m.add_input(a)
    with pytest.raises(AltiusHipError) as e:
        m.infer_value_shape(c)
    assert "MatMul" in e.value.message


def test_fuse_layer_norm():
    m = Model()
    x = m.new_val_named_and_shaped("x", [2, 5, 8])
    out, g, b = layer_norm_chain(m, x, np.ones(8, np.float32), np.zeros(8, np.float32), eps=1e-6)
    tail = m.new_val()
    m.add_node(Op.ReLU, [out], [tail])
    m.add_input(x)
    m.add_output(tail)
    assert len(m.nodes()) == 10
    assert m.fuse_layer_norm() == 1
    nodes = m.nodes()
    assert [n["op_name"] for n in nodes] == ["LayerNormalization", "ReLU"]
    ln = nodes[0]
    assert ln["inputs"] == [x, g, b] and ln["axis"] == -1 and ln["stash_type"] == 1
    assert ln["epsilon"] == np.float32(1e-6)               # taken from the Add's initializer (:128)
    assert nodes[1]["inputs"] == ln["outputs"]             # the chain's reader now reads the fused node
    assert m.fuse_layer_norm() == 0

    # the chain's result as a graph output: the output is rewired (layer_norm_fusion.rs:141-145)
    m = Model()
    x = m.new_val_named_and_shaped("x", [2, 8])
    out, _, _ = layer_norm_chain(m, x, np.ones(8, np.float32), np.zeros(8, np.float32))
    m.add_input(x)
    m.add_output(out)
    assert m.fuse_layer_norm() == 1
    (ln,) = m.nodes()
    assert m.outputs == ln["outputs"]

    # a chain that stops early is left alone
    m = Model()
    x = m.new_val_named_and_shaped("x", [2, 8])
    a, b2 = m.new_val(), m.new_val()
    m.add_node(Op.ReduceMean, [x], [a], axes=[-1])
    m.add_node(Op.Sub, [x, a], [b2])
    m.add_input(x)
    m.add_output(b2)
    assert m.fuse_layer_norm() == 0 and len(m.nodes()) == 2


def test_fused_chains_back_to_back_read_each_other():
    """Two patterns where the second starts at the value the first ends in (the matches are collected before any of
    them is rewritten, layer_norm_fusion.rs:24-139, gelu_fusion.rs:12-74): the second fused node must read the first
    one's new output, also where that value is a graph output as well."""
    for middle_is_output in (False, True):
        m = Model()
        x = m.new_val_named_and_shaped("x", [2, 8])
        a, _, _ = layer_norm_chain(m, x, np.ones(8, np.float32), np.zeros(8, np.float32))
        b, _, _ = layer_norm_chain(m, a, np.ones(8, np.float32), np.zeros(8, np.float32))
        m.add_input(x)
        if middle_is_output:
            m.add_output(a)
        m.add_output(b)
        assert m.fuse_layer_norm() == 2
        first, second = m.nodes()
        assert first["inputs"][0] == x and second["inputs"][0] == first["outputs"][0]
        assert m.outputs == ([first["outputs"][0]] if middle_is_output else []) + second["outputs"]
        m.infer_value_shape(m.outputs[-1])  # every value has a producer

        m = Model()
        x = m.new_val_named_and_shaped("x", [1, 2, 3])
        a = erf_gelu_chain(m, x)
        b = erf_gelu_chain(m, a)
        m.add_input(x)
        if middle_is_output:
            m.add_output(a)
        m.add_output(b)
        assert m.fuse_gelu() == 2
        first, second = m.nodes()
        assert first["inputs"] == [x] and second["inputs"] == first["outputs"]
        assert m.outputs == ([first["outputs"][0]] if middle_is_output else []) + second["outputs"]


def test_fuse_gelu():
    """crates/core/src/optimize/gelu_fusion.rs:12-82."""
    m = Model()
    x = m.new_val_named_and_shaped("x", [1, 2, 3])
    out = erf_gelu_chain(m, x)
    m.add_input(x)
    m.add_output(out)
    assert m.fuse_gelu() == 1
    (g,) = m.nodes()
    assert g["op_name"] == "Gelu" and g["inputs"] == [x] and m.outputs == g["outputs"]

    m = Model()  # a divisor that is not sqrt(2) within 1e-5: no fusion (:18-24)
    x = m.new_val_named_and_shaped("x", [1, 2, 3])
    out = erf_gelu_chain(m, x, sqrt2=1.5)
    m.add_input(x)
    m.add_output(out)
    assert m.fuse_gelu() == 0 and len(m.nodes()) == 5


def test_fuse_fast_gelu():
    """crates/core/src/optimize/fast_gelu_fusion.rs:5-190: the tanh form with x produced by a node."""
    m = Model()
    x0 = m.new_val_named_and_shaped("x0", [2, 4])
    x = m.new_val()
    m.add_node(Op.ReLU, [x0], [x])
    three = m.new_initializer(np.array(3.0, np.float32))
    c1 = m.new_initializer(np.array(0.044715, np.float32))
    c2 = m.new_initializer(np.array(0.7978845608, np.float32))
    one = m.new_initializer(np.array(1.0, np.float32))
    half = m.new_initializer(np.array(0.5, np.float32))
    v = [m.new_val() for _ in range(8)]
    m.add_node(Op.Pow, [x, three], [v[0]])
    m.add_node(Op.Mul, [v[0], c1], [v[1]])
    m.add_node(Op.Add, [x, v[1]], [v[2]])
    m.add_node(Op.Mul, [v[2], c2], [v[3]])
    m.add_node(Op.Tanh, [v[3]], [v[4]])
    m.add_node(Op.Add, [v[4], one], [v[5]])
    m.add_node(Op.Mul, [x, half], [v[6]])
    m.add_node(Op.Mul, [v[6], v[5]], [v[7]])
    tail = m.new_val()
    m.add_node(Op.Sqrt, [v[7]], [tail])
    m.add_input(x0)
    m.add_output(tail)
    assert m.fuse_fast_gelu() == 1
    names = [n["op_name"] for n in m.nodes()]
    assert names == ["ReLU", "Gelu", "Sqrt"]
    gelu = m.nodes()[1]
    assert gelu["inputs"] == [x] and m.nodes()[2]["inputs"] == gelu["outputs"]


def test_eliminate_identity():
    """crates/core/src/optimize/identity_elim.rs:5-45: readers are rewired; an Identity feeding a graph
    output stays."""
    m = Model()
    x = m.new_val_named_and_shaped("x", [3])
    a, b, c = m.new_val(), m.new_val(), m.new_val()
    m.add_node(Op.Identity, [x], [a])
    m.add_node(Op.ReLU, [a], [b])
    m.add_node(Op.Identity, [b], [c])
    m.add_input(x)
    m.add_output(c)
    assert m.eliminate_identity() == 1
    nodes = m.nodes()
    assert [n["op_name"] for n in nodes] == ["ReLU", "Identity"] and nodes[0]["inputs"] == [x]


def test_extents_whose_product_does_not_fit_are_refused():
    """usize arithmetic wraps in the reference's release build (tensor.rs:116-132 multiplies the extents); here a
    product past 2^60 saturates, so the allocation sized from it fails instead of succeeding at the wrapped size
    (2^33 x 2^33 elements would wrap to 4)."""
    for dims in ([1 << 40, 1 << 40], [1 << 33, 1 << 33], [1 << 62, 4], [3, 1 << 31, 1 << 31]):
        with pytest.raises(AltiusHipError) as e:
            Tensor.zeros(dims)
        assert e.value.code == ERR_OOM, dims
    assert Tensor.zeros([0, 1 << 62, 1 << 62]).dims == [0, 1 << 62, 1 << 62]  # an empty tensor is empty whatever its other extents
    m = Model()
    x = m.new_val_named_and_shaped("x", [1 << 33, 1 << 33])
    y = m.new_val()
    m.add_node(Op.ReLU, [x], [y])
    m.add_input(x)
    assert m.infer_value_shape(y)[0] == [1 << 33, 1 << 33]  # shapes are only numbers until something is allocated


OUT_OF_MEMORY_INSIDE_THE_LIBRARY = """
import resource, sys
from altius_amd.graph import Model, Op
from altius_amd._lib import AltiusHipError, ERR_OOM
m = Model()
cur = m.new_val_named_and_shaped("x", [4])
m.add_input(cur)
for _ in range(60000):
    nxt = m.new_val()
    m.add_node(Op.ReLU, [cur], [nxt])
    cur = nxt
m.add_output(cur)
size = next(int(line.split()[1]) * 1024 for line in open("/proc/self/status") if line.startswith("VmSize"))
resource.setrlimit(resource.RLIMIT_AS, (size + (24 << 20), size + (24 << 20)))
try:
    copies = [m.clone() for _ in range(2000)]
except AltiusHipError as e:
    print("code", e.code, e.message)
    sys.exit(0 if e.code == ERR_OOM else 4)
except MemoryError:
    print("the interpreter ran out first")
    sys.exit(3)
sys.exit(5)
"""


def test_running_out_of_memory_inside_the_library_is_an_error_code():
    """No exception may unwind through the C boundary (the reference panics; a C++ exception escaping an extern "C"
    function ends the caller's process).  A child process copies a 60 000-node model under an address-space limit a
    few MB above what it already uses: the copy constructor's allocation fails inside ahip_model_clone, and the call
    must return AHIP_ERR_OOM with the process alive."""
    r = subprocess.run([sys.executable, "-c", OUT_OF_MEMORY_INSIDE_THE_LIBRARY], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, (r.returncode, r.stdout[-300:], r.stderr[-300:])
    assert "out of host memory" in r.stdout


def test_argument_errors():
    m = Model()
    x = m.new_val()
    L = _lib.lib()
    assert L.ahip_model_add_input(m.handle, 999) == ERR_ARG
    assert L.ahip_model_add_node(m.handle, 999, None, None, 0, None, 0, None, None) == ERR_ARG
    bad = (ctypes.c_int64 * 1)(42)
    assert L.ahip_model_add_node(m.handle, Op.ReLU, None, None, 1, bad, 0, None, None) == ERR_ARG
    assert b"unknown input" in L.ahip_last_error(None)
    with pytest.raises(AltiusHipError):  # initializer whose byte count does not match its shape
        check_dims = (ctypes.c_int64 * 1)(4)
        data = np.zeros(3, np.float32)
        _lib.check(L.ahip_model_add_initializer(m.handle, x, F32, 1, check_dims, data.ctypes.data, data.nbytes))
    assert L.ahip_session_builder_new(None, None) == ERR_ARG
    assert L.ahip_tensor_new(7, 0, None, None, 0, None) == ERR_ARG
    # device entry points refuse a null context before touching the runtime
    assert L.ahip_module_load(None, None, 0, None) == ERR_ARG
    assert L.ahip_launch(None, None, b"k", None, None, 0, None) == ERR_ARG
    assert b"null context" in L.ahip_last_error(None)


def test_host_tensor_round_trip():
    for arr in (np.arange(24, dtype=np.float32).reshape(2, 3, 4), np.array(5, np.int64), np.zeros((0, 3), np.float32)):
        t = Tensor.from_numpy(arr)
        assert t.dims == list(arr.shape)
        back = t.numpy()
        assert back.dtype == arr.dtype and np.array_equal(back, arr)
    assert Tensor.from_numpy(np.array([1, 2], np.int64)).elem_ty == I64


def test_host_tensor_views_and_pool_without_a_device():
    """Large tensors ask the pinned pool first; the pool's counters never go backwards and the
    bytes are the same whichever memory holds them.  view() aliases the tensor's own storage."""
    before = host_pool_stats()
    a = np.arange(1 << 18, dtype=np.float32).reshape(512, 512)      # 1 MiB: above the pool's threshold
    t = Tensor.from_numpy(a)
    v = t.view()
    assert v.shape == (512, 512) and np.array_equal(v, a)
    v[0, 0] = 42.0                                                  # Tensor::data_mut
    assert t.numpy()[0, 0] == 42.0 and a[0, 0] == 0.0               # the tensor holds a copy of `a`
    z = Tensor.zeros([3, 5])
    assert z.dims == [3, 5] and not z.view().any()
    z.view()[:] = 7
    assert np.all(z.numpy() == 7)
    live = host_pool_stats()[0]
    del v, t
    after = host_pool_stats()
    assert after[0] <= live and after[2] >= before[2] and after[3] >= before[3]
    host_pool_trim()
    assert host_pool_stats()[1] == 0
    keep = Tensor.from_numpy(a).view()                              # the view keeps its tensor alive
    import gc
    gc.collect()
    assert np.array_equal(keep, a)


def _ln_chain_model(shape=(2, 5, 8)):
    m = Model()
    x = m.new_val_named_and_shaped("x", list(shape))
    out, g, b = layer_norm_chain(m, x, np.ones(shape[-1], np.float32), np.zeros(shape[-1], np.float32))
    m.add_input(x)
    m.add_output(out)
    return m, x, out, g, b


def test_fuse_elemwise_ops_reference_rule():
    """crates/core/src/optimize/elemwise_fusion.rs:12-138 on the exporter's LayerNorm chain: Add(eps) -> Sqrt
    fuse (Sqrt is unary and reads the Add), Mul(gamma) -> Add(beta) fuse (second operands of equal shape);
    Sub feeds two readers, Pow feeds a ReduceMean, Div's second operand [2,5,1] differs from gamma's [8]."""
    m, x, out, g, b = _ln_chain_model()
    assert m.fuse_elemwise_ops() == 2
    nodes = m.nodes()
    assert [n["op_name"] for n in nodes] == ["ReduceMean", "Sub", "Pow", "ReduceMean", "FusedElemwise", "Div", "FusedElemwise"]
    assert m.fused_chain(nodes[4]["id"]) == ["Add", "Sqrt"] and m.fused_chain(nodes[6]["id"]) == ["Mul", "Add"]
    # inputs of the fused node = the chain's outside operands in order of first use (:95-112), output = the last node's
    assert nodes[6]["inputs"] == [nodes[5]["outputs"][0], g, b] and nodes[6]["outputs"] == [out] == m.outputs
    assert len(nodes[4]["inputs"]) == 2 and nodes[5]["inputs"][1] == nodes[4]["outputs"][0]
    assert m.infer_value_shape(out) == ([2, 5, 8], F32)     # shape.rs:616-650 walks the chain
    assert m.fuse_elemwise_ops() == 0                        # FusedElemwise itself is not element-wise (op.rs:387-412)

    # a unary node ends a chain: the node after it would need a binary predecessor (:44)
    m = Model()
    x = m.new_val_named_and_shaped("x", [4, 4])
    v = [m.new_val() for _ in range(3)]
    m.add_node(Op.Add, [x, x], [v[0]])
    m.add_node(Op.Sqrt, [v[0]], [v[1]])
    m.add_node(Op.ReLU, [v[1]], [v[2]])
    m.add_input(x)
    m.add_output(v[2])
    assert m.fuse_elemwise_ops() == 1
    assert [n["op_name"] for n in m.nodes()] == ["FusedElemwise", "ReLU"]

    # the approximated functions are not element-wise for the reference (op.rs:400-409): nothing to fuse
    m = Model()
    x = m.new_val_named_and_shaped("x", [3, 7])
    out = erf_gelu_chain(m, x)
    m.add_input(x)
    m.add_output(out)
    assert m.fuse_elemwise_ops() == 0 and len(m.nodes()) == 5


def test_fuse_elemwise_ops_extended_rule():
    m = Model()
    x = m.new_val_named_and_shaped("x", [3, 7])
    out = erf_gelu_chain(m, x)
    m.add_input(x)
    m.add_output(out)
    assert m.fuse_elemwise_ops(extended=True) == 1
    (n,) = m.nodes()
    assert m.fused_chain(n["id"]) == ["Div", "Erf", "Add", "Mul", "Mul"]
    assert n["inputs"][0] == x and len(n["inputs"]) == 4 and n["outputs"] == m.outputs   # x, sqrt 2, 1, 0.5: x only once
    assert m.infer_value_shape(out) == ([3, 7], F32)
    assert [p[0] for p in m.execution_plan()] == [n["id"]]

    # The LayerNorm chain: Add(eps) -> Sqrt -> Div(d, .) -> Mul(gamma) -> Add(beta) is one chain, the square root
    # being the SECOND operand of the Div; its [2,5,1] intermediates are computed at the output's extent.
    m, x, out, g, b = _ln_chain_model()
    assert m.fuse_elemwise_ops(extended=True) == 1
    nodes = m.nodes()
    assert [n["op_name"] for n in nodes] == ["ReduceMean", "Sub", "Pow", "ReduceMean", "FusedElemwise"]
    assert m.fused_chain(nodes[4]["id"]) == ["Add", "Sqrt", "Div", "Mul", "Add"]
    assert nodes[4]["inputs"][0] == nodes[3]["outputs"][0] and nodes[4]["inputs"][2:] == [nodes[1]["outputs"][0], g, b]
    assert m.infer_value_shape(out) == ([2, 5, 8], F32)

    # a value that is also a graph output ends its chain; an integer tensor is never fused
    m = Model()
    x = m.new_val_named_and_shaped("x", [4])
    i = m.new_val_named_and_shaped("i", [4], I64)
    a, b2, c, d = (m.new_val() for _ in range(4))
    m.add_node(Op.Sqrt, [x], [a])
    m.add_node(Op.ReLU, [a], [b2])
    m.add_node(Op.Tanh, [b2], [c])
    m.add_node(Op.Add, [i, i], [d])
    m.add_input(x)
    m.add_input(i)
    for o in (a, c, d):
        m.add_output(o)
    assert m.fuse_elemwise_ops(extended=True) == 1
    assert sorted(n["op_name"] for n in m.nodes()) == ["Add", "FusedElemwise", "Sqrt"]

    # chains are cut at 16 steps and at 6 distinct outside operands
    m = Model()
    x = m.new_val_named_and_shaped("x", [8])
    cur = x
    for _ in range(20):
        nxt = m.new_val()
        m.add_node(Op.ReLU, [cur], [nxt])
        cur = nxt
    m.add_input(x)
    m.add_output(cur)
    assert m.fuse_elemwise_ops(extended=True) == 2
    assert [len(m.fused_chain(n["id"])) for n in m.nodes()] == [16, 4]
    m = Model()
    x = m.new_val_named_and_shaped("x", [8])
    cur = x
    for k in range(9):
        nxt = m.new_val()
        m.add_node(Op.Add, [cur, m.new_initializer(np.full(8, k, np.float32))], [nxt])
        cur = nxt
    m.add_input(x)
    m.add_output(cur)
    assert m.fuse_elemwise_ops(extended=True) == 2
    assert [len(n["inputs"]) for n in m.nodes()] == [6, 5]   # x + 5 constants, then the first result + 4 constants

    with pytest.raises(AltiusHipError) as e:                  # shape inference fails -> ShapeError, as in the reference
        m = Model()
        p, q, r = m.new_val_named_and_shaped("p", [2, 3]), m.new_val_named_and_shaped("q", [4]), m.new_val()
        m.add_node(Op.Add, [p, q], [r])
        m.add_input(p)
        m.add_input(q)
        m.add_output(r)
        m.fuse_elemwise_ops()
    assert e.value.code == ERR_SHAPE


def _attention_tail(x_shape, mask_shape, scale_kind="Div", mask_first=False, swap_scale=False):
    m = Model()
    x = m.new_val_named_and_shaped("scores", list(x_shape))
    cur = x
    c = None
    if scale_kind:
        c = m.new_initializer(np.array(8.0, np.float32))
        nxt = m.new_val()
        m.add_node(Op.Div if scale_kind == "Div" else Op.Mul, [c, cur] if swap_scale else [cur, c], [nxt])
        cur = nxt
    mask = None
    if mask_shape is not None:
        mask = m.new_val_named_and_shaped("mask", list(mask_shape))
        nxt = m.new_val()
        m.add_node(Op.Add, [mask, cur] if mask_first else [cur, mask], [nxt])
        cur = nxt
        m.add_input(mask)
    p = m.new_val_named("p")
    m.add_node(Op.Softmax, [cur], [p], axis=-1)
    m.add_input(x)
    m.add_output(p)
    return m, x, c, mask


def test_fuse_softmax_prologue():
    def attr(m, node, name):
        v = ctypes.c_int64()
        _lib.check(m.L.ahip_node_get_attr_int(m.handle, node["id"], name.encode(), ctypes.byref(v)))
        return v.value

    m, x, c, mask = _attention_tail([2, 4, 9, 9], [2, 1, 1, 9])
    assert m.fuse_softmax_prologue() == 1
    (sm,) = m.nodes()
    assert sm["op_name"] == "Softmax" and sm["inputs"] == [x, c, mask] and sm["outputs"] == m.outputs
    assert attr(m, sm, "prologue_scale") == 2 and attr(m, sm, "prologue_mask") == 1
    assert m.infer_value_shape(m.outputs[0]) == ([2, 4, 9, 9], F32)
    assert m.fuse_softmax_prologue() == 0

    m, x, c, mask = _attention_tail([2, 4, 9, 9], [9], scale_kind="Mul", mask_first=True, swap_scale=True)   # c * x, mask + .
    assert m.fuse_softmax_prologue() == 1
    (sm,) = m.nodes()
    assert sm["inputs"] == [x, c, mask] and attr(m, sm, "prologue_scale") == 1

    m, x, c, mask = _attention_tail([2, 4, 9, 9], None, scale_kind="Mul")                                    # scale only
    assert m.fuse_softmax_prologue() == 1 and m.nodes()[0]["inputs"] == [x, c]
    m, x, c, mask = _attention_tail([2, 4, 9, 9], [1, 1, 1, 9], scale_kind=None)                             # mask only
    assert m.fuse_softmax_prologue() == 1 and m.nodes()[0]["inputs"] == [x, mask]

    # left alone: c / x is not a scale; a mask that varies along a middle axis; a mask that grows the scores;
    # an intermediate that is also a graph output
    m, *_ = _attention_tail([2, 4, 9, 9], None, scale_kind="Div", swap_scale=True)
    assert m.fuse_softmax_prologue() == 0 and len(m.nodes()) == 2
    m, *_ = _attention_tail([2, 4, 9, 9], [2, 4, 1, 9], scale_kind=None)
    assert m.fuse_softmax_prologue() == 0
    m, *_ = _attention_tail([1, 4, 9, 9], [2, 1, 1, 9], scale_kind=None)
    assert m.fuse_softmax_prologue() == 0
    m, x, c, mask = _attention_tail([2, 4, 9, 9], None, scale_kind="Mul")
    m.add_output(m.nodes()[0]["outputs"][0])
    assert m.fuse_softmax_prologue() == 0


def test_fuse_matmul_bias():
    def build(x_shape, w_shape, b_shape, bias_first=False, extra_reader=False):
        m = Model()
        x = m.new_val_named_and_shaped("x", x_shape)
        w = m.new_initializer(np.zeros(w_shape, np.float32))
        b = m.new_initializer(np.zeros(b_shape, np.float32))
        p, y = m.new_val(), m.new_val_named("y")
        m.add_node(Op.MatMul, [x, w], [p])
        m.add_node(Op.Add, [b, p] if bias_first else [p, b], [y])
        m.add_input(x)
        m.add_output(y)
        if extra_reader:
            z = m.new_val()
            m.add_node(Op.ReLU, [p], [z])
            m.add_output(z)
        return m, x, w, b, y

    for x_shape, w_shape, b_shape, first in (([5, 10], [10, 15], [15], False), ([3, 5, 10], [10, 15], [1, 15], True),
                                             ([2, 3, 5, 10], [2, 3, 10, 15], [1, 1, 1, 15], False)):
        m, x, w, b, y = build(x_shape, w_shape, b_shape, first)
        assert m.fuse_matmul_bias() == 1
        (mm,) = m.nodes()
        assert mm["op_name"] == "MatMul" and mm["inputs"] == [x, w, b] and mm["outputs"] == [y] == m.outputs
        assert m.infer_value_shape(y)[0] == x_shape[:-1] + [15]
        assert m.fuse_matmul_bias() == 0
    # left alone: a bias that is not one value per column, a product with a second reader
    assert build([5, 10], [10, 15], [5, 1])[0].fuse_matmul_bias() == 0
    assert build([5, 10], [10, 15], [5, 15])[0].fuse_matmul_bias() == 0
    assert build([5, 10], [10, 15], [15], extra_reader=True)[0].fuse_matmul_bias() == 0


def test_fuse_transpose_matmul():
    """crates/core/src/optimize/transpose_fusion.rs:33-62: perms [1,0], [0,2,1], [0,1,3,2] on either operand."""
    def attr(m, node, name):
        v = ctypes.c_int64()
        _lib.check(m.L.ahip_node_get_attr_int(m.handle, node["id"], name.encode(), ctypes.byref(v)))
        return v.value

    m = Model()
    q = m.new_val_named_and_shaped("q", [2, 3, 7, 4])
    k = m.new_val_named_and_shaped("k", [2, 3, 7, 4])
    kt, s, other = m.new_val(), m.new_val_named("s"), m.new_val_named("other")
    m.add_node(Op.Transpose, [k], [kt], perm=[0, 1, 3, 2])
    m.add_node(Op.MatMul, [q, kt], [s])
    m.add_input(q)
    m.add_input(k)
    m.add_output(s)
    keep = m.clone()
    assert m.fuse_transpose_matmul() == 1
    (mm,) = m.nodes()
    assert mm["op_name"] == "MatMul" and mm["inputs"] == [q, k] and attr(m, mm, "transB") == 1 and attr(m, mm, "transA") == 0
    assert m.infer_value_shape(s) == ([2, 3, 7, 7], F32)
    assert m.fuse_transpose_matmul() == 0

    # a Transpose with a second reader stays for it; a permutation that moves other axes is not folded
    t2 = keep.new_val()
    keep.add_node(Op.ReLU, [kt], [t2])
    keep.add_output(t2)
    assert keep.fuse_transpose_matmul() == 1
    assert sorted(n["op_name"] for n in keep.nodes()) == ["MatMul", "ReLU", "Transpose"]
    m = Model()
    a = m.new_val_named_and_shaped("a", [5, 2, 6])
    at, w, y = m.new_val(), m.new_initializer(np.zeros([2, 5, 3], np.float32)), m.new_val()
    m.add_node(Op.Transpose, [a], [at], perm=[1, 2, 0])
    m.add_node(Op.MatMul, [at, w], [y])
    m.add_input(a)
    m.add_output(y)
    assert m.fuse_transpose_matmul() == 0
    # both operands, rank 2
    m = Model()
    a, b = m.new_val_named_and_shaped("a", [6, 5]), m.new_val_named_and_shaped("b", [4, 6])
    at, bt, y = m.new_val(), m.new_val(), m.new_val()
    m.add_node(Op.Transpose, [a], [at], perm=[1, 0])
    m.add_node(Op.Transpose, [b], [bt], perm=[1, 0])
    m.add_node(Op.MatMul, [at, bt], [y])
    m.add_input(a)
    m.add_input(b)
    m.add_output(y)
    assert m.fuse_transpose_matmul() == 1 and len(m.nodes()) == 1
    assert m.infer_value_shape(y) == ([5, 4], F32)
