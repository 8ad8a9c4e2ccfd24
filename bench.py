#!/usr/bin/env python3
"""Benchmark of the interpreter tensor kernels on one MI355X.

Workload (BASELINE.json configs[4], the configuration the >= 70 %-of-HBM target is quoted on):
one "step" is one pass of the four kernels over device-resident fp32 inputs

    Add      scores[256,12,197,197] + mask[256,1,1,197]
    Softmax  over the last axis of that sum
    ReduceMax over axis 1 of [256,768,197]
    Div      [256,197,768] / scalar

`value` is the whole step's algorithmic bytes (every tensor read or written once) divided by
the step time, in GB/s: W warm-up steps and K timed ones after the step has kept the GPU busy
for --settle-ms; `value_after_idle` is the same W + K steps straight after the uploads, which
leave the GPU idle for seconds (for a few milliseconds after an idle period the part runs
slower).  Per-kernel times are measured with HIP events on the stream the kernels run on (mean,
median and minimum over at least 100 launches after a warm-up of 20 launches and at least 25 ms,
and once more inside the running step); `roofline` describes the slowest kernel of the step.  Beside the
step the line carries every other operator of the path on the step's [256,197,768] array
(`listed_ops`), Softmax / LayerNormalization / ReduceMean by row length (`row_sweep`), the same operators on
shapes away from the configs' own (`shape_sweep`) and the
kernels and graphs of configs[0..3] (`other_configs`).  The CPU baseline is the oracle (a C++
restatement of the reference interpreter's kernels) timed on this machine's host cores on the same
workload, with 16 threads and with 1, allocating its outputs per call as the reference does and
writing into existing ones.

Prints one JSON line of less than 6000 characters on stdout, last: the headline, `roofline` and `cpu_baseline` in full and
every table as rows of numbers under a `cols` legend.  stderr carries one short line per section; --verbose prints the
tables there, --full-json PATH writes every figure to a file.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E


VERBOSE = False


def log(*a):
    """The wide tables: stderr, only with --verbose."""
    if VERBOSE:
        print(*a, file=sys.stderr, flush=True)


def note(*a):
    """One short progress line per section: stderr, always (a few hundred characters over the whole run)."""
    print(*a, file=sys.stderr, flush=True)


LINE_LIMIT = 6000  # the JSON line on stdout stays below this many characters


def _strip(name):
    return name.replace(", ", ",").replace(" -> ", ">").replace(" ", "")


def compact_line(result, limit=LINE_LIMIT):
    """The one line for stdout: the headline fields, `config`, `roofline` and `cpu_baseline` in full, and every table
    of the run as rows of numbers under a `cols` legend (us = mean HIP-event time per launch, pct = algorithmic bytes
    / us as a percentage of 8 TB/s).  Tables are dropped, last first, if the line would pass `limit`, and named
    under `dropped`; the full record goes to the file --full-json names."""
    head = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
            "dtype", "data", "config", "value_after_idle", "ms_per_step_after_idle", "settle_ms")
    line = {k: result[k] for k in head if k in result}
    if "roofline" in result:
        line["roofline"] = result["roofline"]
    if "cpu_baseline" in result:
        keep = ("value", "unit", "cores", "kind", "sample", "single_thread_value", "value_existing_outputs",
                "single_thread_value_existing_outputs", "us_per_kernel_scaled", "us_per_kernel_scaled_1_thread")
        line["cpu_baseline"] = {k: v for k, v in result["cpu_baseline"].items() if k in keep}
    tables = []
    if result.get("per_kernel"):
        tables.append(("per_kernel", {"cols": ["kernel", "bytes", "us", "us_median", "pct", "us_in_step"],
                                      "rows": [[_strip(r["kernel"]), r["bytes"], r["us"], r["us_median"], r["pct_hbm_peak"], r.get("us_interleaved")]
                                               for r in result["per_kernel"]]}))
    if result.get("listed_ops"):
        tables.append(("listed_ops", {"cols": ["kernel", "us", "pct"],
                                      "rows": [[_strip(r["kernel"]), r["us"], r["pct_hbm_peak"]] for r in result["listed_ops"]]}))
    if result.get("other_configs"):
        oc = result["other_configs"]
        tables.append(("other_configs", {
            "cols": ["kernel", "us", "pct", "cpu_us_16_threads", "cpu_us_1_thread"],
            "rows": [[_strip(r["kernel"]), r["us"], r["pct_hbm_peak"], r.get("cpu_us_16_threads"), r.get("cpu_us_1_thread")] for r in oc["kernels"]],
            "graph_cols": ["graph", "kernels_us", "kernels_us_graph_replay", "run_device_us", "run_device_enqueue_us", "run_ms_with_pcie"],
            "graphs": [[r["graph"], r["kernels_us"], r["kernels_us_graph_replay"], r["run_device_us"], r.get("run_device_enqueue_us"), r["run_ms_with_pcie"]]
                       for r in oc["graphs"]]}))
    if result.get("row_sweep"):
        names = [k for k in result["row_sweep"][0] if k != "row_length"]
        tables.append(("row_sweep", {"cols": ["row_length"] + [n + "_pct" for n in names],
                                     "rows": [[e["row_length"]] + [e[n]["pct_hbm_peak"] for n in names] for e in result["row_sweep"]]}))
    if result.get("shape_sweep"):
        # operators that share a shape share a row: [shape, pct of each operator of the group]
        groups = {}
        for r in result["shape_sweep"]:
            op, _, shape = r["kernel"].partition(" ")
            g = groups.setdefault("Transpose" if op == "Transpose" else "middle_axis" if "axis=1" in op else "odd_rows" if "(-1)" in op else "other",
                                  {"ops": [], "shapes": {}})
            if op not in g["ops"]:
                g["ops"].append(op)
            g["shapes"].setdefault(_strip(shape), {})[op] = r["pct_hbm_peak"]
        tables.append(("shape_sweep", {name: {"cols": ["shape"] + [o + "_pct" for o in g["ops"]],
                                              "rows": [[sh] + [v.get(o) for o in g["ops"]] for sh, v in g["shapes"].items()]}
                                       for name, g in groups.items()}))
    for k in ("vit", "next_rows", "timeline", "calibration"):
        if k in result:
            tables.append((k, result[k]))
    for name, t in tables:
        line[name] = t
    dropped = []
    while len(json.dumps(line, separators=(",", ":"))) >= limit and tables:
        name, _ = tables.pop()
        del line[name]
        dropped.append(name)
        line["dropped"] = dropped
    return json.dumps(line, separators=(",", ":"))


def ensure_built():
    from altius_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from altius_amd import build

        note("libaltius_hip.so missing: building")
        build.build()


class Op:
    """One kernel launch on fixed device buffers, with its algorithmic byte count."""

    def __init__(self, name, nbytes, launchers, cpu=None):
        self.name = name
        self.nbytes = nbytes
        self.launchers = launchers  # one closure per rotated buffer set
        self.cpu = cpu              # cpu(threads): the same operator on the CPU oracle (test infrastructure, timed beside)
        self.i = 0

    def launch(self):
        self.launchers[self.i % len(self.launchers)]()
        self.i += 1


def build_cfg4(ctx, D, synth, batch, rotate_bytes):
    """Uploads configs[4] at the given batch and returns the four ops of a step."""
    from altius_amd._lib import check

    c = synth.cfg4(batch=batch)
    ops = []

    def copies(nbytes_per_set):
        return max(1, min(4, int(np.ceil(rotate_bytes / max(nbytes_per_set, 1)))))

    # Add (mask)
    scores, mask = c["scores"], c["mask"]
    out_dims = list(scores.shape)
    a_str = D.strides_for_broadcasting(scores.shape, out_dims)
    b_str = D.strides_for_broadcasting(mask.shape, out_dims)
    d_scores = ctx.upload(scores)
    d_mask = ctx.upload(mask)
    d_sum = ctx.alloc(scores.nbytes)
    add_bytes = 2 * scores.nbytes + mask.nbytes
    ops.append(Op("Add(mask) [%d,12,197,197]+[%d,1,1,197]" % (batch, batch), add_bytes,
                  [lambda: ctx.binary_raw(D.ADD, d_sum.ptr, d_scores.ptr, d_mask.ptr, out_dims, a_str, b_str)]))

    # Softmax on the sum
    d_prob = ctx.alloc(scores.nbytes)
    rows = scores.size // 197
    ops.append(Op("Softmax(-1) [%d,12,197,197]" % batch, 2 * scores.nbytes,
                  [lambda: ctx.softmax_raw(d_prob.ptr, d_sum.ptr, rows, 197)]))
    # The two of them as one kernel (what fuse_softmax_prologue makes of Add(mask) -> Softmax): same bits, the
    # intermediate sum never written.  Timed beside the step, not part of it.
    fused = [Op("Add(mask)+Softmax in one kernel [%d,12,197,197]" % batch, 2 * scores.nbytes + mask.nbytes,
                [lambda: check(ctx.L.ahip_softmax_lastaxis_prologue(ctx.handle, d_prob.ptr, d_scores.ptr, rows, 197, 0, 1.0,
                                                                     d_mask.ptr, 12 * 197), ctx.handle)])]

    # ReduceMax over axis 1; inputs rotated so that repeated launches do not hit the Infinity Cache
    x = c["rmax_in"]
    rmax_bytes = x.nbytes + batch * 197 * 4
    d_out = ctx.alloc(batch * 197 * 4)
    ins = [ctx.upload(x) for _ in range(copies(rmax_bytes))]
    ops.append(Op("ReduceMax(axis=1) [%d,768,197]" % batch, rmax_bytes,
                  [(lambda p=b.ptr: ctx.reduce_raw(D.REDUCE_MAX, d_out.ptr, p, batch, 768, 197)) for b in ins]))

    # Div by a scalar
    y = c["div_in"]
    d_scalar = ctx.upload(np.array([c["div_scalar"]], np.float32))
    div_bytes = 2 * y.nbytes + 4
    n_sets = copies(div_bytes)
    ins = [ctx.upload(y) for _ in range(n_sets)]
    outs = [ctx.alloc(y.nbytes) for _ in range(n_sets)]
    dims = list(y.shape)
    ys = D.strides_for_broadcasting(y.shape, dims)
    ss = D.strides_for_broadcasting([], dims)
    ops.append(Op("Div(scalar) [%d,197,768]" % batch, div_bytes,
                  [(lambda i=i: ctx.binary_raw(D.DIV, outs[i].ptr, ins[i].ptr, d_scalar.ptr, dims, ys, ss))
                   for i in range(n_sets)]))
    return ops, fused, c


def build_listed_ops(ctx, D, c, batch, rotate_bytes=900e6):
    """Every operator of the path at configs[4]-sized tensors: the operators the step itself does not hold
    (Sub, Mul, Pow, the unary ones, ReduceMean, LayerNormalization) on the step's own arrays, so that each has a
    bandwidth figure at the size where bandwidth is what bounds it.  Buffers rotate past the 256 MB cache."""
    ops = []
    y = c["div_in"]                                   # [batch,197,768] ~ N(0,1)
    dims = list(y.shape)
    rows_n = batch * 197
    k = max(2, min(4, int(np.ceil(rotate_bytes / (2 * y.nbytes)))))
    xs = [ctx.upload(y) for _ in range(k)]
    pos = [ctx.upload(np.abs(y) + np.float32(0.5)) for _ in range(k)]
    outs = [ctx.alloc(y.nbytes) for _ in range(k)]
    small = [ctx.alloc(rows_n * 4) for _ in range(k)]
    rng = np.random.default_rng(11)
    col = ctx.upload((1.5 + rng.random((batch, 197, 1))).astype(np.float32))       # per-row operand (mean, std)
    vec = ctx.upload((1.0 + 0.02 * rng.standard_normal(768)).astype(np.float32))   # gamma-like operand
    vec2 = ctx.upload((0.02 * rng.standard_normal(768)).astype(np.float32))
    two = ctx.upload(np.array([2.0], np.float32))
    ys = D.strides_for_broadcasting(dims, dims)

    def binary(name, op, other, other_shape, src=xs):
        os_ = D.strides_for_broadcasting(other_shape, dims)
        nbytes = 2 * y.nbytes + 4 * int(np.prod(other_shape, dtype=np.int64))
        ops.append(Op(name, nbytes, [(lambda i=i: ctx.binary_raw(op, outs[i].ptr, src[i].ptr, other.ptr, dims, ys, os_))
                                     for i in range(k)]))

    def unary(name, op, src=xs, alpha=0.0, beta=0.0):
        ops.append(Op(name, 2 * y.nbytes, [(lambda i=i: ctx.unary_raw(op, outs[i].ptr, src[i].ptr, y.size, alpha, beta))
                                           for i in range(k)]))

    shape = "[%d,197,768]" % batch
    binary("Sub %s-[%d,197,1]" % (shape, batch), D.SUB, col, [batch, 197, 1])
    binary("Mul %s*[768]" % shape, D.MUL, vec, [768])
    binary("Div %s/[%d,197,1]" % (shape, batch), D.DIV, col, [batch, 197, 1])
    binary("Pow(.,2) %s" % shape, D.POW, two, [])
    unary("Sqrt %s" % shape, D.SQRT, src=pos)
    unary("Erf %s" % shape, D.ERF)
    unary("Gelu %s" % shape, D.GELU)
    unary("Sigmoid %s" % shape, D.SIGMOID)
    unary("HardSigmoid %s" % shape, D.HARDSIGMOID, alpha=1.0 / 6.0, beta=0.5)
    unary("Relu %s" % shape, D.RELU)
    ops.append(Op("ReduceMean(-1) %s" % shape, y.nbytes + rows_n * 4,
                  [(lambda i=i: ctx.reduce_raw(D.REDUCE_MEAN, small[i].ptr, xs[i].ptr, rows_n, 768, 1)) for i in range(k)]))
    ops.append(Op("Softmax(-1) %s" % shape, 2 * y.nbytes,
                  [(lambda i=i: ctx.softmax_raw(outs[i].ptr, xs[i].ptr, rows_n, 768)) for i in range(k)]))
    ops.append(Op("LayerNormalization(-1) %s" % shape, 2 * y.nbytes + 2 * 768 * 4,
                  [(lambda i=i: ctx.layernorm_raw(outs[i].ptr, xs[i].ptr, vec.ptr, vec2.ptr, rows_n, 768, 1e-5)) for i in range(k)]))
    return ops


ROW_SWEEP_ELEMS = 96 << 20   # 403 MB in, 403 MB out: every launch misses the 256 MB cache
ROW_SWEEP_LENGTHS = (49, 64, 100, 128, 197, 256, 384, 512, 768, 1000, 1024, 1280, 2048, 3072, 4096, 5120, 8192, 12288, 16384)


def build_row_sweep(ctx, D, lengths=ROW_SWEEP_LENGTHS, elems=ROW_SWEEP_ELEMS):
    """The three row operators of the path on one ~400 MB array cut into rows of every length between a 7 x 7
    feature map and a 16 K hidden size.  One input and one output buffer serve all lengths."""
    rng = np.random.default_rng(21)
    d_in = ctx.upload(rng.standard_normal(elems, dtype=np.float32))
    d_out = ctx.alloc(elems * 4)
    longest = max(lengths)
    d_g = ctx.upload((1.0 + 0.02 * rng.standard_normal(longest)).astype(np.float32))
    d_b = ctx.upload((0.02 * rng.standard_normal(longest)).astype(np.float32))
    for length in lengths:
        rows = elems // length
        n = rows * length
        yield length, [
            Op("Softmax", 2 * n * 4, [lambda rows=rows, length=length: ctx.softmax_raw(d_out.ptr, d_in.ptr, rows, length)]),
            Op("LayerNormalization", 2 * n * 4 + 2 * length * 4,
               [lambda rows=rows, length=length: ctx.layernorm_raw(d_out.ptr, d_in.ptr, d_g.ptr, d_b.ptr, rows, length, 1e-5)]),
            Op("ReduceMean", n * 4 + rows * 4,
               [lambda rows=rows, length=length: ctx.reduce_raw(D.REDUCE_MEAN, d_out.ptr, d_in.ptr, rows, length, 1)]),
        ]
    for b in (d_in, d_out, d_g, d_b):
        ctx.free(b)


def run_row_sweep(ctx, D, args, lengths):
    sweep = []
    log("Softmax / LayerNormalization / ReduceMean over the last axis, %d M elements, by row length (%% of 8 TB/s):" % (ROW_SWEEP_ELEMS >> 20))
    for length, ops_l in build_row_sweep(ctx, D, lengths):
        entry = {"row_length": length}
        for o in ops_l:
            t = time_kernel(ctx, o, args.kernel_iters, args.kernel_warmup, args.kernel_settle_ms)
            r = t.row(o.nbytes)
            entry[o.name] = {"bytes": o.nbytes, "us": r["us"], "us_median": r["us_median"], "us_min": r["us_min"], "GBps": r["GBps"],
                             "pct_hbm_peak": r["pct_hbm_peak"]}
        sweep.append(entry)
        log("  rows of %6d: %s" % (length, "   ".join("%s %6.1f us %5.1f %%" % (k, v["us"], v["pct_hbm_peak"])
                                                        for k, v in entry.items() if k != "row_length")))
    return sweep


SHAPE_SWEEP_ELEMS = 96 << 20
SHAPE_SWEEP_MIDDLE = ((197, 768), (49, 1024), (12, 4096), (1024, 8), (2, 65536), (196, 3), (7, 7))   # (reduced, inner) extents
SHAPE_SWEEP_ODD_ROWS = (1025, 2049, 5001, 9999, 50257)
SHAPE_SWEEP_TRANSPOSES = (([64, 256, 56, 56], [0, 2, 3, 1]), ([8192, 8192], [1, 0]), ([8196, 8196], [1, 0]), ([256, 197, 768], [0, 2, 1]), ([50257, 768], [1, 0]),
                          ([768, 50257], [1, 0]))


def build_shape_sweep(ctx, D, elems=SHAPE_SWEEP_ELEMS):
    """The listed operators on shapes away from the configs' own: reductions over a middle axis, rows that are not whole
    float4s (lengths above 1024, a vocabulary), a broadcast vector of three values, transposes that change the
    innermost axis.  One ~400 MB input, cut to each shape."""
    from altius_amd._lib import check, i64_array
    rng = np.random.default_rng(22)
    d_in = ctx.upload(rng.standard_normal(elems, dtype=np.float32))
    d_out = ctx.alloc(elems * 4)
    d_g = ctx.upload((1.0 + 0.02 * rng.standard_normal(65536)).astype(np.float32))
    d_b = ctx.upload((0.02 * rng.standard_normal(65536)).astype(np.float32))
    ops = []
    for red, inner in SHAPE_SWEEP_MIDDLE:
        outer = elems // (red * inner)
        for kind, name in ((D.REDUCE_MEAN, "ReduceMean"), (D.REDUCE_MAX, "ReduceMax")):
            ops.append(Op("%s(axis=1) [%d,%d,%d]" % (name, outer, red, inner), (outer * red * inner + outer * inner) * 4,
                          [lambda k=kind, o=outer, r=red, i=inner: ctx.reduce_raw(k, d_out.ptr, d_in.ptr, o, r, i)]))
    for length in SHAPE_SWEEP_ODD_ROWS:
        rows = elems // length
        n = rows * length
        ops.append(Op("Softmax(-1) [%d,%d]" % (rows, length), 2 * n * 4, [lambda r=rows, l=length: ctx.softmax_raw(d_out.ptr, d_in.ptr, r, l)]))
        ops.append(Op("LayerNormalization(-1) [%d,%d]" % (rows, length), 2 * n * 4 + 2 * length * 4,
                      [lambda r=rows, l=length: ctx.layernorm_raw(d_out.ptr, d_in.ptr, d_g.ptr, d_b.ptr, r, l, 1e-5)]))
        ops.append(Op("ReduceMean(-1) [%d,%d]" % (rows, length), (n + rows) * 4, [lambda r=rows, l=length: ctx.reduce_raw(D.REDUCE_MEAN, d_out.ptr, d_in.ptr, r, l, 1)]))
    rgb = [4096, 4096, 3]
    ops.append(Op("Sub [4096,4096,3] - [3]", (2 * 4096 * 4096 * 3 + 3) * 4,
                  [lambda: ctx.binary_raw(D.SUB, d_out.ptr, d_in.ptr, d_g.ptr, rgb, D.strides_for_broadcasting(rgb, rgb), D.strides_for_broadcasting([3], rgb))]))
    for shape, perm in SHAPE_SWEEP_TRANSPOSES:
        n = int(np.prod(shape))
        ops.append(Op("Transpose %s -> %s" % (shape, tuple(perm)), 2 * n * 4,
                      [lambda sh=shape, pm=perm: check(ctx.L.ahip_transpose(ctx.handle, d_out.ptr, d_in.ptr, 4, len(sh), i64_array(sh), i64_array(pm)), ctx.handle)]))
    for o in ops:
        yield o
    for b in (d_in, d_out, d_g, d_b):
        ctx.free(b)


def build_other_configs(ctx, D, synth, rotate_bytes=600e6, max_sets=48):
    """Kernels of configs[0..3] at their BASELINE.json shapes (parity-test shapes, reported as a table
    only).  Buffers are rotated over enough copies that repeated launches miss the 256 MB cache.  Each
    operator also carries the same call on the CPU oracle, timed beside it by the caller."""
    import oracle as O

    ops = []

    def sets(nbytes):
        return max(1, min(max_sets, int(np.ceil(rotate_bytes / max(nbytes, 1)))))

    def binary(name, op, a, b):
        out_dims = D.broadcast_shape(a.shape, b.shape)
        n = int(np.prod(out_dims))
        nbytes = a.nbytes + b.nbytes + 4 * n
        a_str, b_str = D.strides_for_broadcasting(a.shape, out_dims), D.strides_for_broadcasting(b.shape, out_dims)
        k = sets(nbytes)
        da = [ctx.upload(a) for _ in range(k)]
        db = ctx.upload(b) if b.nbytes < (1 << 20) else None
        dbs = [db] * k if db else [ctx.upload(b) for _ in range(k)]
        do = [ctx.alloc(4 * n) for _ in range(k)]
        ops.append(Op(name, nbytes, [(lambda i=i: ctx.binary_raw(op, do[i].ptr, da[i].ptr, dbs[i].ptr, out_dims, a_str, b_str))
                                     for i in range(k)], cpu=lambda threads: O.binary(op, a, b, threads=threads)))

    def unary(name, op, x, alpha=0.0, beta=0.0):
        k = sets(2 * x.nbytes)
        dx = [ctx.upload(x) for _ in range(k)]
        do = [ctx.alloc(x.nbytes) for _ in range(k)]
        ops.append(Op(name, 2 * x.nbytes, [(lambda i=i: ctx.unary_raw(op, do[i].ptr, dx[i].ptr, x.size, alpha, beta))
                                           for i in range(k)], cpu=lambda threads: O.unary(op, x, alpha, beta, threads=threads)))

    def softmax(name, x):
        k = sets(2 * x.nbytes)
        dx = [ctx.upload(x) for _ in range(k)]
        do = [ctx.alloc(x.nbytes) for _ in range(k)]
        rows, length = x.size // x.shape[-1], x.shape[-1]
        ops.append(Op(name, 2 * x.nbytes, [(lambda i=i: ctx.softmax_raw(do[i].ptr, dx[i].ptr, rows, length)) for i in range(k)],
                      cpu=lambda threads: O.softmax(x, threads=threads)))

    def layer_norm(name, x, gamma, beta, eps):
        nbytes = 2 * x.nbytes + gamma.nbytes + beta.nbytes
        k = sets(nbytes)
        dx = [ctx.upload(x) for _ in range(k)]
        do = [ctx.alloc(x.nbytes) for _ in range(k)]
        dg, db = ctx.upload(gamma), ctx.upload(beta)
        rows, length = x.size // x.shape[-1], x.shape[-1]
        ops.append(Op(name, nbytes, [(lambda i=i: ctx.layernorm_raw(do[i].ptr, dx[i].ptr, dg.ptr, db.ptr, rows, length, eps))
                                     for i in range(k)], cpu=lambda threads: O.layer_norm(x, gamma, beta, eps, threads=threads)))

    def reduce(name, kind, x, outer, red, inner, axes):
        nbytes = x.nbytes + 4 * outer * inner
        k = sets(nbytes)
        dx = [ctx.upload(x) for _ in range(k)]
        do = [ctx.alloc(4 * outer * inner) for _ in range(k)]
        ops.append(Op(name, nbytes, [(lambda i=i: ctx.reduce_raw(kind, do[i].ptr, dx[i].ptr, outer, red, inner))
                                     for i in range(k)], cpu=lambda threads: O.reduce(kind, x, axes, True)))  # single-threaded in the reference

    # the floor under every figure of this table: a kernel with next to nothing to do
    unary("floor Relu [64]", D.RELU, np.zeros(64, np.float32))
    c0 = synth.cfg0()
    binary("cfg0 Add [1,197,768]+[768]", D.ADD, c0["a"], c0["b"])
    c1 = synth.cfg1()
    softmax("cfg1 Softmax [8,12,197,197]", c1["scores"])
    layer_norm("cfg1 LayerNorm [8,197,768]", c1["x"], c1["gamma"], c1["beta"], float(c1["eps"]))
    c2 = synth.cfg2()
    x = c2["x"]
    mean = np.zeros((32, 197, 1), np.float32)
    layer_norm("cfg2 LayerNorm (fused) [32,197,768]", x, c2["gamma"], c2["beta"], float(c2["eps"]))
    reduce("cfg2 ReduceMean(-1) [32,197,768]", D.REDUCE_MEAN, x, 32 * 197, 768, 1, [-1])
    binary("cfg2 Sub [32,197,768]-[32,197,1]", D.SUB, x, mean)
    binary("cfg2 Pow(.,2) [32,197,768]", D.POW, x, np.array(2.0, np.float32))
    binary("cfg2 Div [32,197,768]/[32,197,1]", D.DIV, x, mean + np.float32(1.5))
    binary("cfg2 Mul gamma [32,197,768]*[768]", D.MUL, x, c2["gamma"])
    c3 = synth.cfg3()
    unary("cfg3 Gelu [32,197,3072]", D.GELU, c3["x"])
    unary("cfg3 Erf [32,197,3072]", D.ERF, c3["x"])
    binary("cfg3 Mul [32,197,3072]*[32,197,3072]", D.MUL, c3["x"], c3["x"])
    se = c3["se"]
    reduce("cfg3 ReduceMean(H,W) [32,576,7,7]", D.REDUCE_MEAN, se, 32 * 576, 49, 1, [2, 3])
    unary("cfg3 HardSigmoid [32,576,1,1]", D.HARDSIGMOID, np.zeros((32, 576, 1, 1), np.float32), 1.0 / 6.0, 0.5)
    binary("cfg3 Mul [32,576,7,7]*[32,576,1,1]", D.MUL, se, np.ones((32, 576, 1, 1), np.float32))
    return ops


def session_table(synth, dev_ctx):
    """Whole `run()` calls on host tensors (upload, kernels, download) for the graph-level configurations,
    with the device-only share from the session's own per-op events."""
    from altius_amd import graphs
    from altius_amd.graph import Tensor
    from altius_amd.session import HipSessionBuilder

    rows = []

    def measure(name, model, x, alg_bytes):
        t_in = Tensor.from_numpy(x)              # the caller's host tensor, as the reference's run() takes it
        row = {"graph": name, "algorithmic_bytes": alg_bytes}
        # Node by node, then with the run recorded as a HIP graph and replayed (one launch per run).
        for key, replay in (("kernels_us", False), ("kernels_us_graph_replay", True)):
            sess = HipSessionBuilder(model.clone()).with_graph_replay(replay).build()
            best_run, best_dev = float("inf"), float("inf")
            for _ in range(7):
                outs = sess.run([t_in], copy=False)
                best_run = min(best_run, sess.last_run_ms())
                best_dev = min(best_dev, sess.last_device_ms())
                del outs                         # output tensors dropped, as a caller would after use
            if replay:
                assert sess.graph_replays() == 6, sess.graph_replays()
            row[key] = round(best_dev * 1e3, 1)
            row["run_ms_with_pcie" + ("_graph_replay" if replay else "")] = round(best_run, 3)
            sess.close()
        row["kernels_GBps"] = round(alg_bytes / (min(row["kernels_us"], row["kernels_us_graph_replay"]) * 1e-6) / 1e9, 1)
        # The same graph on a tensor that already lives on the GPU: wall time of the C ABI's run_device + synchronize
        # (arguments built once, no event pair around the run), no PCIe; and the host's share of it, the enqueue.
        sess = HipSessionBuilder(model.clone()).with_device_timing(False).build()
        d_x = dev_ctx.upload(x)
        prepared = sess.prepare_device_inputs([(d_x.ptr, x.shape, x.dtype)])
        best, best_enqueue = float("inf"), float("inf")
        for _ in range(30):
            t0 = time.perf_counter()
            outs = sess.run_device_prepared(prepared)
            sess.synchronize()
            best = min(best, time.perf_counter() - t0)
            best_enqueue = min(best_enqueue, sess.last_run_ms())
            for o in outs:
                o.free()
        dev_ctx.free(d_x)
        sess.close()
        row["run_device_enqueue_us"] = round(best_enqueue * 1e3, 1)
        row["run_device_us"] = round(best * 1e6, 1)
        rows.append(row)

    c2 = synth.cfg2()
    X, r = c2["x"].nbytes, 32 * 197 * 4
    chain = graphs.single_input_model(c2["x"].shape, lambda m, x: graphs.layer_norm_chain(
        m, x, c2["gamma"], c2["beta"], float(c2["eps"]))[0])
    fused = chain.clone()
    fused.fuse_layer_norm()
    measure("cfg2 LayerNorm chain, 9 nodes", chain, c2["x"], 12 * X + 8 * r + 2 * 768 * 4 + 8)
    measure("cfg2 after fuse_layer_norm, 1 node", fused, c2["x"], 2 * X + 2 * 768 * 4)
    ew = chain.clone()
    ew.fuse_elemwise_ops(extended=True)        # ReduceMean, Sub, Pow, ReduceMean, FusedElemwise[Add,Sqrt,Div,Mul,Add]
    measure("cfg2 chain after fuse_elemwise_ops, 5 nodes", ew, c2["x"], 8 * X + 4 * r + 2 * 768 * 4 + 8)
    c3 = synth.cfg3()
    X = c3["x"].nbytes
    chain = graphs.single_input_model(c3["x"].shape, lambda m, x: graphs.erf_gelu_chain(m, x, float(c3["sqrt2"])))
    fused = chain.clone()
    fused.fuse_gelu()
    measure("cfg3 erf-GELU chain, 5 nodes", chain, c3["x"], 11 * X + 12)
    measure("cfg3 after fuse_gelu, 1 node", fused, c3["x"], 2 * X)
    ew = chain.clone()
    ew.fuse_elemwise_ops(extended=True)        # one FusedElemwise with the bits of the 5-node chain
    measure("cfg3 chain after fuse_elemwise_ops, 1 node", ew, c3["x"], 2 * X + 12)
    se = c3["se"]
    model = graphs.single_input_model(se.shape, lambda m, x: graphs.squeeze_excite(m, x, c3["alpha"], c3["beta"]))
    measure("cfg3 squeeze-excite, 3 nodes", model, se, 3 * se.nbytes + 4 * 32 * 576 * 4)
    return rows


def vit_table(batch, layers=12):
    """Whole-model device time (kernels only, input already uploaded by run()) of a ViT-B/16-shaped encoder for
    three versions of the same graph, with the per-operator split of each from a profiled run."""
    from altius_amd import device as D, graphs
    from altius_amd.graph import Tensor
    from altius_amd.session import HipSessionBuilder

    base = graphs.vit_encoder(batch, layers=layers)
    x = Tensor.from_numpy(np.random.default_rng(1).standard_normal((batch, 197, 768)).astype(np.float32))
    versions = []
    versions.append(("as exported", base))
    ref = base.clone()
    ref.fuse_layer_norm(), ref.fuse_gelu(), ref.fuse_fast_gelu(), ref.eliminate_identity()
    versions.append(("reference rewrites (fuse_layer_norm, fuse_gelu)", ref))
    ours = ref.clone()
    ours.fuse_softmax_prologue(), ours.fuse_matmul_bias(), ours.fuse_transpose_matmul(), ours.fuse_elemwise_ops(extended=True)
    versions.append(("+ softmax prologue, matmul bias / transposes, element-wise chains", ours))
    versions.append(("+ large products on the bf16 matrix cores (three planes per operand)", ours))
    versions.append(("+ strided views, one-kernel attention, Gelu and residual Add done by the products around them", ours))
    rows = []
    for i, (name, model) in enumerate(versions):
        algo = D.GEMM_AUTO if i >= 3 else D.GEMM_FP32
        views = i >= 4
        sess = HipSessionBuilder(model).with_gemm_algorithm(algo).with_strided_views(views).with_fused_attention(views).build()
        best = float("inf")
        for _ in range(4):
            outs = sess.run([x], copy=False)
            best = min(best, sess.last_device_ms())
            del outs
        sess.close()
        prof = HipSessionBuilder(model).with_gemm_algorithm(algo).with_strided_views(views).with_fused_attention(views).with_profiling_enabled(True).build()
        for _ in range(2):
            outs = prof.run([x], copy=False)
            del outs
        split = {k: round(v, 3) for k, v in sorted(prof.profile().items(), key=lambda kv: -kv[1])}
        prof.close()
        rows.append({"graph": name, "nodes": len(model.nodes()), "device_ms": round(best, 3), "per_op_ms": split})
    return rows


def build_next_rows(ctx, D, batch=256):
    """The operators either side of the hot path (data movement, MatMul) at ViT-B/16 shapes for the given
    batch: (name, bytes, flops, launcher).  Device buffers are left uninitialised where contents do not matter."""
    from altius_amd._lib import check, i64_array

    L, h = ctx.L, ctx.handle
    rows = []
    T, H, NH, DH = 197, 768, 12, 64

    def transpose(name, shape, perm):
        n = int(np.prod(shape))
        a, b = ctx.alloc(n * 4), ctx.alloc(n * 4)
        rows.append((name, 8 * n, 0, lambda: check(L.ahip_transpose(h, b.ptr, a.ptr, 4, len(shape), i64_array(shape), i64_array(perm)), h)))

    transpose("Transpose split heads [%d,197,12,64]->(0,2,1,3)" % batch, (batch, T, NH, DH), (0, 2, 1, 3))
    transpose("Transpose K^T [%d,12,197,64]->(0,1,3,2)" % batch, (batch, NH, T, DH), (0, 1, 3, 2))
    n = batch * T * 3 * H
    qkv = ctx.alloc(n * 4)
    parts = [ctx.alloc(n * 4 // 3) for _ in range(3)]

    def split():
        for i, o in enumerate(parts):
            check(L.ahip_copy_strided(h, o.ptr, qkv.ptr + H * 4 * i, 4, 2, i64_array([batch * T, H]), i64_array([H, 1]),
                                      i64_array([3 * H, 1])), h)

    rows.append(("Split qkv [%d,197,2304] -> 3 x 768" % batch, 8 * n, 0, split))
    V, S = 50257, batch * 128
    table, out = ctx.alloc(V * H * 4), ctx.alloc(S * H * 4)
    ids = ctx.upload(np.random.default_rng(0).integers(0, V, size=S).astype(np.int64))
    rows.append(("Gather [50257,768] x %d ids" % S, 2 * S * H * 4 + S * 8, 0,
                 lambda: check(L.ahip_gather(h, out.ptr, table.ptr, ids.ptr, 8, 4, 1, V, S, H), h)))

    rng = np.random.default_rng(5)

    def gemm(name, b, m, n_, k, a_bs, b_bs, algorithms=(("fp32 MFMA", D.GEMM_FP32),), trans_b=False):
        # random operands: constant ones toggle fewer bits in the matrix cores and run at a higher clock
        a = ctx.upload(rng.standard_normal(((b if a_bs else 1) * m, k), dtype=np.float32))
        w = ctx.upload(rng.standard_normal(((b if b_bs else 1) * k, n_), dtype=np.float32) * np.float32(0.03))
        c = ctx.alloc(b * m * n_ * 4)
        nbytes = 4 * ((b if a_bs else 1) * m * k + (b if b_bs else 1) * k * n_ + b * m * n_)
        for label, algo in algorithms:
            if algo == D.GEMM_BF16X3:
                ctx.gemm_register_constant(w)  # as a session does for its weights: their planes are made once

            def launch(algo=algo):
                ctx.gemm_set_algorithm(algo)
                ctx.gemm_raw(c.ptr, a.ptr, w.ptr, None, b, m, n_, k, trans_b=trans_b, a_bs=a_bs, b_bs=b_bs, c_bs=m * n_)
                ctx.gemm_set_algorithm(D.GEMM_DEFAULT)

            rows.append(("%s (%s)" % (name, label), nbytes, 2.0 * b * m * n_ * k, launch))

    M = batch * T
    both = (("fp32 MFMA", D.GEMM_FP32), ("bf16 x 3 incl. split of A", D.GEMM_BF16X3))
    gemm("MatMul qkv [%d,768]x[768,2304]" % M, 1, M, 3 * H, H, 0, 0, both)
    gemm("MatMul proj [%d,768]x[768,768]" % M, 1, M, H, H, 0, 0, both)
    gemm("MatMul fc1 [%d,768]x[768,3072]" % M, 1, M, 4 * H, H, 0, 0, both)
    gemm("MatMul fc2 [%d,3072]x[3072,768]" % M, 1, M, H, 4 * H, 0, 0, both)
    # the MLP's second product with the Gelu in front of it applied while its operand is split (f(A) never stored)
    ga = ctx.upload(rng.standard_normal((M, 4 * H), dtype=np.float32))
    gw = ctx.upload(rng.standard_normal((4 * H, H), dtype=np.float32) * np.float32(0.03))
    gc = ctx.alloc(M * H * 4)
    ctx.gemm_register_constant(gw)

    def gelu_fc2():
        ctx.gemm_set_algorithm(D.GEMM_BF16X3)
        check(L.ahip_gemm_activated(h, D.GELU, gc.ptr, ga.ptr, gw.ptr, None, M, H, 4 * H, 0, 0, 4 * H, H, H, 0, 0, 1.0, 0.0), h)
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)

    rows.append(("MatMul Gelu(A) x B, fc2 [%d,3072]x[3072,768] (bf16 x 3 incl. Gelu and split of A)" % M, 4 * (M * 4 * H + 4 * H * H + M * H),
                 2.0 * M * H * 4 * H, gelu_fc2))
    gemm("MatMul QK^T %d x [197,64]x[64,197]" % (batch * NH), batch * NH, T, T, DH, T * DH, DH * T)
    # the same product with K where it lies, [197,64] per head, as a session that plans views hands it over (the operand has
    # the same number of values either way round, so the upload above serves)
    gemm("MatMul QK^T %d x [197,64]x[197,64]^T, K in place" % (batch * NH), batch * NH, T, T, DH, T * DH, DH * T, trans_b=True)
    gemm("MatMul PV %d x [197,197]x[197,64]" % (batch * NH), batch * NH, T, DH, T, T * T, T * DH)
    # QK^T -> scale -> Softmax -> PV in one kernel, heads read in place from the [b, t, 3 h d] result of the qkv product
    # and written as [b, t, h d]
    import ctypes
    qkv3 = ctx.upload(rng.standard_normal((batch * T, 3 * H), dtype=np.float32))
    att = ctx.alloc(batch * T * H * 4)
    S2 = ctypes.c_size_t * 2
    ld = 3 * H
    def attention(algo):
        ctx.gemm_set_algorithm(algo)
        check(L.ahip_attention(h, att.ptr, qkv3.ptr, qkv3.ptr + H * 4, qkv3.ptr + 2 * H * 4, batch, NH, T, T, DH, ld, ld, ld, H,
                               S2(T * ld, DH), S2(T * ld, DH), S2(T * ld, DH), S2(T * H, DH), 1, 0.125, None, 0), h)
        ctx.gemm_set_algorithm(D.GEMM_DEFAULT)

    for label, algo in (("fp32 MFMA", D.GEMM_FP32), ("bf16 x 3", D.GEMM_BF16X3)):
        rows.append(("Attention %d x Softmax(QK^T/8)V [197,64], one kernel (%s)" % (batch * NH, label), 4 * batch * T * 4 * H,
                     2.0 * batch * NH * (2 * T * T * DH), lambda algo=algo: attention(algo)))
    return rows


def calibration_op(ctx, D):
    """A copy-shaped kernel of known traffic (Relu over 477 MB in, 477 MB out) used to scale the
    FETCH_SIZE / WRITE_SIZE counters of a profiling run."""
    n = 256 * 12 * 197 * 197
    d_in = ctx.alloc(n * 4)
    d_out = ctx.alloc(n * 4)
    ctx.memset(d_in, 0x3f)
    return Op("Relu(copy calibration) [%d]" % n, 2 * n * 4,
              [lambda: ctx.unary_raw(D.RELU, d_out.ptr, d_in.ptr, n)])


TRAFFIC_FILE = "profiles/hbm_traffic.json"


def measured_traffic(kernel_name):
    """HBM bytes per launch of a kernel as derived from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this program
    (profiles/hbm_traffic.json, written from those runs; counters cannot be read from inside the timed run), or None."""
    path = os.path.join(ROOT, TRAFFIC_FILE)
    if not os.path.exists(path):
        return None
    with open(path) as f:
        table = json.load(f)
    for key, entry in table.get("kernels", {}).items():
        if kernel_name.startswith(key):
            return entry.get("traffic_bytes")
    return None


class Timing:
    """Launch durations of one kernel in ms: mean over all timed launches (what `roofline.achieved` uses),
    median and minimum over the samples (one sample = the average of a short group of back-to-back launches)."""

    def __init__(self, samples_ms, group):
        self.samples = sorted(samples_ms)
        self.group = group
        self.launches = len(samples_ms) * group
        self.mean = sum(samples_ms) / len(samples_ms)
        self.median = float(np.median(samples_ms))
        self.min = self.samples[0]

    def row(self, nbytes):
        """The figures every table of the report carries, rounded."""
        gbps = nbytes / (self.mean * 1e-3) / 1e9
        return {"us": round(self.mean * 1e3, 2), "us_median": round(self.median * 1e3, 2), "us_min": round(self.min * 1e3, 2),
                "launches": self.launches, "GBps": round(gbps, 1), "pct_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 1),
                "pct_hbm_peak_median": round(100.0 * nbytes / (self.median * 1e-3) / 1e9 / HBM_PEAK_GBPS, 1)}


SETTLE_MS = 25.0  # warm-up of a kernel lasts at least this long


def time_kernel(ctx, op, iters=100, warmup=20, settle_ms=SETTLE_MS):
    """`warmup` untimed launches, and as many more as it takes to keep the GPU on this kernel for `settle_ms`; then at
    least `iters` timed ones with a HIP event on the kernels' stream between consecutive samples.  A sample is a group
    of back-to-back launches lasting about 0.25 ms (one launch for the longest kernels, dozens for the few-microsecond
    ones), so that the event between samples does not weigh on the figure.
    Why the warm-up goes by time: after an idle period, or when the load changes, the part runs the next 3 to 25 ms of
    kernels several percent slower (a 150 us Softmax: up to 180 us between its 15th and its 100th launch, then 152 us
    for as long as it is kept busy) while its power management settles; 20 launches of a long kernel end inside that
    window and 100 timed ones cover it."""
    for _ in range(warmup):
        op.launch()
    probe = [ctx.event(), ctx.event()]
    ctx.sync()
    ctx.record(probe[0])
    for _ in range(5):
        op.launch()
    ctx.record(probe[1])
    est_ms = ctx.elapsed_ms(probe[0], probe[1]) / 5
    for e in probe:
        ctx.destroy_event(e)
    for _ in range(min(20000, max(0, int(settle_ms / max(est_ms, 1e-4)) - warmup - 5))):
        op.launch()
    group = max(1, min(64, int(round(0.25 / max(est_ms, 1e-4)))))
    n = max(25, (iters + group - 1) // group)
    events = [ctx.event() for _ in range(n + 1)]
    ctx.sync()
    ctx.record(events[0])
    for i in range(n):
        for _ in range(group):
            op.launch()
        ctx.record(events[i + 1])
    ctx.sync()
    samples = [ctx.elapsed_ms(events[i], events[i + 1]) / group for i in range(n)]
    for e in events:
        ctx.destroy_event(e)
    return Timing(samples, group)


def launch_timeline(ctx, op, n):
    """Duration of each of n consecutive launches (a HIP event after every launch): shows how long after an idle
    period the kernel takes to reach the time it then keeps."""
    events = [ctx.event() for _ in range(n + 1)]
    ctx.sync()
    ctx.record(events[0])
    for i in range(n):
        op.launch()
        ctx.record(events[i + 1])
    ctx.sync()
    us = [ctx.elapsed_ms(events[i], events[i + 1]) * 1e3 for i in range(n)]
    for e in events:
        ctx.destroy_event(e)
    return us


def time_interleaved(ctx, ops, steps, warmup):
    """The step's kernels in step order, an event between every two launches: the duration of each kernel while the
    others run around it (sustained mixed load), as opposed to the same kernel launched back to back."""
    for _ in range(warmup):
        for o in ops:
            o.launch()
    events = [[ctx.event() for _ in range(len(ops) + 1)] for _ in range(steps)]
    ctx.sync()
    for s in range(steps):
        ctx.record(events[s][0])
        for i, o in enumerate(ops):
            o.launch()
            ctx.record(events[s][i + 1])
    ctx.sync()
    out = []
    for i in range(len(ops)):
        out.append(Timing([ctx.elapsed_ms(events[s][i], events[s][i + 1]) for s in range(steps)], 1))
    for row in events:
        for e in row:
            ctx.destroy_event(e)
    return out


def cpu_baseline(synth, batch_full, sample_batch, threads, arrays=None):
    """Times the oracle on the same step (the whole batch, or a reduced one).  Every operator is timed twice: writing
    into a fresh output array per call, which is what the reference's run_node does (session.rs:95-110: one allocation
    per node output, whose pages fault in while the kernel writes), and writing into an output that already exists.
    Returns GB/s of the step (fresh outputs, the reference's behaviour), per-op seconds of both variants."""
    import oracle as O

    O.lib()
    c = arrays if arrays is not None and sample_batch == batch_full else synth.cfg4(batch=sample_batch)
    fresh, reused = {}, {}
    total_bytes = 0

    def best_of(fn, reps=3):
        best = float("inf")
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            best = min(best, time.perf_counter() - t0)
        return best

    def timed(name, nbytes, fn, out_shape):
        nonlocal total_bytes
        fresh[name] = best_of(lambda: fn(np.empty(out_shape, np.float32)))
        out = np.zeros(out_shape, np.float32)    # exists and is mapped
        reused[name] = best_of(lambda: fn(out))
        total_bytes += nbytes
        return out

    scores, mask = c["scores"], c["mask"]
    z = timed("Add", 2 * scores.nbytes + mask.nbytes, lambda out: O.binary(O.ADD, scores, mask, threads=threads, out=out), scores.shape)
    timed("Softmax", 2 * scores.nbytes, lambda out: O.softmax(z, threads=threads, out=out), scores.shape)
    x = c["rmax_in"]
    timed("ReduceMax", x.nbytes + sample_batch * 197 * 4, lambda out: O.reduce(O.REDUCE_MAX, x, [1], False, out=out), (sample_batch, 197))
    y = c["div_in"]
    s = np.array(c["div_scalar"], np.float32)
    timed("Div", 2 * y.nbytes + 4, lambda out: O.binary(O.DIV, y, s, threads=threads, out=out), y.shape)
    return total_bytes / sum(fresh.values()) / 1e9, fresh, total_bytes / sum(reused.values()) / 1e9, reused


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=256, help="batch of configs[4] (256 = the named workload)")
    ap.add_argument("--kernel-iters", type=int, default=100, help="timed launches per kernel for the per-kernel timing")
    ap.add_argument("--kernel-warmup", type=int, default=20, help="untimed launches per kernel ahead of them (and as many more as %g ms take)" % SETTLE_MS)
    ap.add_argument("--kernel-settle-ms", type=float, default=SETTLE_MS,
                    help="least duration of a kernel's warm-up (0 for counter passes of a profiler, where every launch is slow)")
    ap.add_argument("--settle-ms", type=float, default=250.0,
                    help="the step is run for this long, untimed, before the W warm-up steps and the K timed ones that make 'value' "
                         "(the K steps straight after the uploads are reported beside it as 'value_after_idle')")
    ap.add_argument("--cpu-sample-batch", type=int, default=0,
                    help="batch of the CPU baseline sample (0: the whole batch, about 2 s of CPU time)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", type=str, default="", help="run only kernels whose name contains this text (profiling)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run a copy-shaped Relu of known size (scales rocprof byte counters)")
    ap.add_argument("--no-listed-ops", action="store_true",
                    help="skip the table of the path's other operators at configs[4]-sized tensors ('listed_ops' in the JSON)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the kernels and graphs of configs[0..3] (table on stderr, 'other_configs' in the JSON: us, GB/s and "
                         "the CPU oracle's us at 16 threads and at 1 thread beside each)")
    ap.add_argument("--all-configs", action="store_true", help="accepted for compatibility: configs[0..3] are part of the default run")
    ap.add_argument("--no-row-sweep", action="store_true",
                    help="skip Softmax / LayerNormalization / ReduceMean by row length ('row_sweep' in the JSON)")
    ap.add_argument("--streaming-threshold-mib", type=int, default=-1,
                    help="tensors of at least this many MiB use non-temporal accesses (default: the library's own threshold)")
    ap.add_argument("--sweep-lengths", type=str, default="", help="comma-separated row lengths for the sweep (default: 49 ... 16384)")
    ap.add_argument("--sweep-only", action="store_true", help="run the row sweep and nothing else (profiling)")
    ap.add_argument("--section", type=str, default="", choices=("", "row_sweep", "shape_sweep", "other_configs"),
                    help="run this table and nothing else, behind the calibration kernel if --calibrate is given (profiling); "
                         "prints the table's full records as one JSON line")
    ap.add_argument("--timeline", type=int, default=0, metavar="N",
                    help="print the duration of each of N consecutive launches of every kernel of the step, the first kernel after "
                         "the uploads and one second of idle, and exit ('timeline' in the JSON)")
    ap.add_argument("--next-rows", action="store_true",
                    help="also time the data-movement and MatMul kernels at ViT-B/16 shapes ('next_rows' in the JSON)")
    ap.add_argument("--vit", type=int, default=0, metavar="BATCH",
                    help="also run a ViT-B/16-shaped encoder (12 layers, exporter-style graph, random weights) at this batch: "
                         "device time per forward as exported, after the reference's rewrites, and after this backend's ('vit' in the JSON)")
    ap.add_argument("--verbose", action="store_true", help="print the tables of every section on stderr (default: one short line per section)")
    ap.add_argument("--full-json", type=str, default="", metavar="PATH",
                    help="also write the full record (every figure of every table, as one JSON document) to this file")
    args = ap.parse_args()
    global VERBOSE
    VERBOSE = args.verbose

    if args.gpus != 1:
        note("bench.py: this build runs on one GPU only (every operator on the path is independent along the batch "
            "axis, so more GPUs would each run the same kernels on a slice of the batch, without communication); "
            "run with --gpus 1")
        sys.exit(2)

    ensure_built()
    from altius_amd import device as D
    from altius_amd import synth

    ctx = D.Context(0)
    if args.streaming_threshold_mib >= 0:
        ctx.set_streaming_threshold(args.streaming_threshold_mib << 20)
    sweep_lengths = tuple(int(v) for v in args.sweep_lengths.split(",") if v) or ROW_SWEEP_LENGTHS
    if args.sweep_only:
        args.section = "row_sweep"
    if args.section:
        out = {}
        if args.calibrate:  # first, so that a profile of this run finds the copy kernel of known size ahead of the table
            cal = calibration_op(ctx, D)
            out["calibration"] = dict({"kernel": cal.name, "bytes": cal.nbytes}, **time_kernel(ctx, cal, args.kernel_iters, args.kernel_warmup, args.kernel_settle_ms).row(cal.nbytes))
            log("%-44s %14d %9.1f us %6.1f %%" % (cal.name, cal.nbytes, out["calibration"]["us"], out["calibration"]["pct_hbm_peak"]))
        if args.section == "row_sweep":
            out["row_sweep"] = run_row_sweep(ctx, D, args, sweep_lengths)
        else:
            build = build_shape_sweep(ctx, D) if args.section == "shape_sweep" else build_other_configs(ctx, D, synth)
            rows = []
            mark = ctx.alloc(256)
            for o in build:
                if args.only and args.only.lower() not in o.name.lower():
                    continue
                ctx.memset(mark, 0)  # a fill kernel between two tables' rows: a profile of this run can tell them apart
                t = time_kernel(ctx, o, args.kernel_iters, args.kernel_warmup, args.kernel_settle_ms)
                rows.append(dict({"kernel": o.name, "bytes": o.nbytes}, **t.row(o.nbytes)))
                log("%-52s %14d %9.2f us %8.1f GB/s %6.1f %%" % (o.name, o.nbytes, rows[-1]["us"], rows[-1]["GBps"], rows[-1]["pct_hbm_peak"]))
            out[args.section] = rows
        print(json.dumps(out), flush=True)
        ctx.close()
        return
    ops, fused_ops, cfg4_arrays = build_cfg4(ctx, D, synth, args.batch, rotate_bytes=600e6)
    if args.only:
        ops = [o for o in ops if args.only.lower() in o.name.lower()]
        fused_ops = [o for o in fused_ops if args.only.lower() in o.name.lower()]
    # timed per kernel, not part of the step
    extra_ops = fused_ops + ([calibration_op(ctx, D)] if args.calibrate else [])
    ctx.sync()

    if args.timeline:
        out = {"timeline": []}
        time.sleep(1.0)
        for o in [ops[1], ops[0], ops[1]] if len(ops) > 1 else ops:
            us = launch_timeline(ctx, o, args.timeline)
            tenths = [sum(us[i:i + 10]) / len(us[i:i + 10]) for i in range(0, len(us), 10)]
            out["timeline"].append({"kernel": o.name, "us_mean_of_each_10_launches": [round(v, 1) for v in tenths]})
            log("%-44s %s" % (o.name, " ".join("%.0f" % v for v in tenths)))
        print(json.dumps(out), flush=True)
        ctx.close()
        return

    # --- whole step: W warm-up steps, then exactly K timed steps --------------------------------
    def timed_steps():
        for _ in range(args.warmup):
            for o in ops:
                o.launch()
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            for o in ops:
                o.launch()
        ctx.sync()
        return (time.perf_counter() - t0) / args.steps

    # Once straight after the uploads (the GPU has been idle for seconds: the first 3 to 25 ms of kernels run inside
    # the window in which the part's power management settles), and once for the record after the step has kept the
    # GPU busy for --settle-ms: the sustained rate, which is what a job of more than a few steps sees.
    step_s_after_idle = timed_steps()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < args.settle_ms:
        for _ in range(8):
            for o in ops:
                o.launch()
        ctx.sync()
    step_s = timed_steps()
    step_bytes = sum(o.nbytes for o in ops)
    value = step_bytes / step_s / 1e9

    # --- per kernel, HIP events on the kernels' stream -----------------------------------------
    rows = []
    for o in ops + extra_ops:
        t = time_kernel(ctx, o, args.kernel_iters, args.kernel_warmup, args.kernel_settle_ms)
        rows.append(dict({"kernel": o.name, "bytes": o.nbytes}, **t.row(o.nbytes)))
    # ... and each of the step's kernels while the others run around it
    if len(ops) > 1:
        for r, t in zip(rows, time_interleaved(ctx, ops, max(args.steps, 25), args.warmup)):
            r["us_interleaved"] = round(t.mean * 1e3, 2)
            r["us_interleaved_median"] = round(t.median * 1e3, 2)
            r["pct_hbm_peak_interleaved"] = round(100.0 * r["bytes"] / (t.mean * 1e-3) / 1e9 / HBM_PEAK_GBPS, 1)
    log("%-44s %14s %9s %9s %9s %9s %8s %12s" % ("kernel", "alg. bytes", "us mean", "us median", "us min", "GB/s", "% peak", "us in step"))
    for r in rows:
        log("%-44s %14d %9.1f %9.1f %9.1f %9.1f %8.1f %12s" % (r["kernel"], r["bytes"], r["us"], r["us_median"], r["us_min"], r["GBps"],
                                                            r["pct_hbm_peak"], "%.1f" % r["us_interleaved"] if "us_interleaved" in r else "-"))
    dom = max(rows[:len(ops)], key=lambda r: r["us"])
    note("step %.4f ms, %.1f GB/s; per kernel: %s" % (step_s * 1e3, value, "; ".join(
        "%s %.1f us %.1f %%" % (r["kernel"].split(" ")[0], r["us"], r["pct_hbm_peak"]) for r in rows)))

    result = {
        "metric": "per-op HBM GB/s and % of MI355X peak; us/call vs CPU interpreter",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "value_after_idle": round(step_bytes / step_s_after_idle / 1e9, 1),
        "ms_per_step_after_idle": round(step_s_after_idle * 1e3, 4),
        "settle_ms": args.settle_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[4]: Add(mask)+Softmax on [%d,12,197,197], ReduceMax(axis=1) on [%d,768,197], "
                        "Div(scalar) on [%d,197,768]; one step = the four kernels once" % ((args.batch,) * 3),
            "batch": args.batch,
            "step_bytes": step_bytes,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": dom["kernel"],
            "achieved": round(dom["GBps"], 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dom["GBps"] / HBM_PEAK_GBPS, 4),
            "traffic": measured_traffic(dom["kernel"]),
            "traffic_source": TRAFFIC_FILE + ": rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command scaled by a copy kernel of known "
                              "size; read from that file, not measured in this run",
            "us_per_launch": round(dom["us"], 2),
            "us_per_launch_median": dom["us_median"],
            "us_per_launch_min": dom["us_min"],
            "us_per_launch_in_step": dom.get("us_interleaved"),
            "frac_in_step": round(dom["bytes"] / (dom["us_interleaved"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4) if "us_interleaved" in dom else None,
            "launches": dom["launches"],
            "algorithmic_bytes": dom["bytes"],
        },
        "timing": "value: the step run untimed for settle_ms, then W warm-up steps, then K timed steps (value_after_idle: W + K steps "
                  "straight after the uploads, while the part's power management is still settling). "
                  "per kernel: %d warm-up launches and as many more as %g ms take, then >= %d launches with a HIP event between "
                  "samples on the kernels' stream; us = mean, us_median, us_min; us_interleaved = the same kernel inside the step "
                  "(an event between every two kernels of the step)" % (args.kernel_warmup, args.kernel_settle_ms, args.kernel_iters),
        "per_kernel": rows,
    }

    if not args.only and not args.no_listed_ops:
        listed = []
        log("every operator of the path at configs[4]-sized tensors:")
        for o in build_listed_ops(ctx, D, cfg4_arrays, args.batch):
            t = time_kernel(ctx, o, args.kernel_iters, args.kernel_warmup, args.kernel_settle_ms)
            r = dict({"kernel": o.name, "bytes": o.nbytes}, **t.row(o.nbytes))
            listed.append(r)
            log("%-44s %14d %9.1f %9.1f %9.1f %9.1f %8.1f" % (o.name, o.nbytes, r["us"], r["us_median"], r["us_min"], r["GBps"], r["pct_hbm_peak"]))
        result["listed_ops"] = listed
        note("listed_ops: %d kernels, %.1f to %.1f %% of 8 TB/s" % (len(listed), min(r["pct_hbm_peak"] for r in listed), max(r["pct_hbm_peak"] for r in listed)))

    if not args.only and not args.no_row_sweep:
        result["row_sweep"] = run_row_sweep(ctx, D, args, sweep_lengths)
        shapes = []
        log("the same operators on other shapes (a middle axis, rows that are not whole float4s, innermost-axis transposes):")
        for o in build_shape_sweep(ctx, D):
            t = time_kernel(ctx, o, min(args.kernel_iters, 40), min(args.kernel_warmup, 10), args.kernel_settle_ms)
            r = dict({"kernel": o.name, "bytes": o.nbytes}, **t.row(o.nbytes))
            shapes.append(r)
            log("%-52s %14d %9.1f us %8.1f GB/s %6.1f %%" % (o.name, o.nbytes, r["us"], r["GBps"], r["pct_hbm_peak"]))
        result["shape_sweep"] = shapes
        note("row_sweep: %d row lengths; shape_sweep: %d kernels, lowest %s" % (
            len(result["row_sweep"]), len(shapes), ", ".join("%s %.1f %%" % (r["kernel"], r["pct_hbm_peak"]) for r in sorted(shapes, key=lambda r: r["pct_hbm_peak"])[:3])))

    if not args.only and not args.no_other_configs:
        others = []
        log("%-44s %14s %10s %10s %10s %8s %14s %14s" % ("kernel", "alg. bytes", "us mean", "us median", "GB/s", "% peak", "CPU 16 thr us", "CPU 1 thr us"))
        for o in build_other_configs(ctx, D, synth):
            t = time_kernel(ctx, o, args.kernel_iters, args.kernel_warmup, args.kernel_settle_ms)
            row = dict({"kernel": o.name, "bytes": o.nbytes}, **t.row(o.nbytes))
            cpu_us = {}
            if not args.no_cpu and o.cpu:
                for threads in (16, 1):               # the CPU oracle on the host cores, best of 2 calls
                    best = float("inf")
                    for _ in range(2):
                        t0 = time.perf_counter()
                        o.cpu(threads)
                        best = min(best, time.perf_counter() - t0)
                    cpu_us[threads] = best * 1e6
                row["cpu_us_16_threads"], row["cpu_us_1_thread"] = round(cpu_us[16], 1), round(cpu_us[1], 1)
            others.append(row)
            log("%-44s %14d %10.2f %10.2f %10.1f %8.1f %14s %14s" % (o.name, o.nbytes, row["us"], row["us_median"], row["GBps"], row["pct_hbm_peak"],
                                                                     "%.1f" % cpu_us[16] if cpu_us else "-", "%.1f" % cpu_us[1] if cpu_us else "-"))
        graphs_rows = session_table(synth, ctx)
        for r in graphs_rows:
            log("%-36s kernels %7.1f us, as one HIP graph %7.1f us (%7.1f GB/s)  run_device() + synchronize() wall %7.1f us (enqueue %5.1f us)  run() incl. PCIe %7.3f ms"
                % (r["graph"], r["kernels_us"], r["kernels_us_graph_replay"], r["kernels_GBps"], r["run_device_us"], r["run_device_enqueue_us"],
                   r["run_ms_with_pcie"]))
        result["other_configs"] = {"kernels": others, "graphs": graphs_rows}
        note("other_configs: %d kernels, %d graphs" % (len(others), len(graphs_rows)))

    if args.vit:
        vit_rows = vit_table(args.vit)
        for r in vit_rows:
            top = ", ".join("%s %.2f" % kv for kv in list(r["per_op_ms"].items())[:8])
            log("ViT-B/16 encoder, batch %d, %-58s %4d nodes %9.3f ms   (%s)" % (args.vit, r["graph"], r["nodes"], r["device_ms"], top))
        result["vit"] = {"batch": args.vit, "layers": 12, "rows": vit_rows}

    if args.next_rows:
        MFMA_F32_PEAK = 157.3  # TFLOP/s, dense fp32 matrix cores
        nxt = []
        for name, nbytes, flops, fn in build_next_rows(ctx, D, args.batch):
            o = Op(name, nbytes, [fn])
            ms = time_kernel(ctx, o, max(10, args.kernel_iters // 2), 3, args.kernel_settle_ms).mean
            row = {"kernel": name, "us": round(ms * 1e3, 1), "bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1)}
            if flops:
                # six bf16 MFMAs per fp32 product: the bf16 peak (2500 TFLOP/s dense) over six
                peak = 2500.0 / 6 if "bf16 x 3" in name else MFMA_F32_PEAK
                row.update({"bound": "mfma", "TFLOPs": round(flops / ms / 1e9, 1), "peak_TFLOPs": round(peak, 1),
                            "frac_of_peak": round(flops / ms / 1e9 / peak, 3)})
                log("%-64s %10.1f us %8.1f TFLOP/s (%4.1f %% of %.1f)" % (name, ms * 1e3, flops / ms / 1e9,
                                                                         100 * flops / ms / 1e9 / peak, peak))
            else:
                row.update({"bound": "hbm", "frac_of_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 3)})
                log("%-48s %10.1f us %8.1f GB/s    (%4.1f %% of 8000)" % (name, ms * 1e3, nbytes / ms / 1e6,
                                                                        100 * nbytes / ms / 1e6 / HBM_PEAK_GBPS))
            nxt.append(row)
        result["next_rows"] = nxt

    if not args.no_cpu:
        threads = min(16, os.cpu_count() or 1)
        sample = args.cpu_sample_batch or args.batch
        gbps_n, t_n, gbps_n_re, t_n_re = cpu_baseline(synth, args.batch, sample, threads, cfg4_arrays)
        gbps_1, t_1, gbps_1_re, t_1_re = cpu_baseline(synth, args.batch, sample, 1, cfg4_arrays)
        scale = args.batch / sample
        note("CPU oracle, batch %d sample (x%.0f for the full step), fresh output per call as the reference allocates it: "
            "%d threads %.2f GB/s, 1 thread %.2f GB/s; into existing outputs: %.2f and %.2f GB/s"
            % (sample, scale, threads, gbps_n, gbps_1, gbps_n_re, gbps_1_re))
        for k in t_n:
            log("  %-10s %d threads %9.1f us (existing output %9.1f)   1 thread %9.1f us (existing output %9.1f)  (scaled to batch %d)"
                % (k, threads, t_n[k] * scale * 1e6, t_n_re[k] * scale * 1e6, t_1[k] * scale * 1e6, t_1_re[k] * scale * 1e6, args.batch))
        us = lambda t: {k: round(v * scale * 1e6, 1) for k, v in t.items()}
        result["cpu_baseline"] = {
            "value": round(gbps_n, 2),
            "unit": "GB/s",
            "cores": threads,
            "kind": "port",
            "sample": "same four kernels at batch %d of %d (1/%d of the step), best of 3 runs, each output allocated per call "
                      "as the reference's run_node does; 1 thread: %.2f GB/s; writing into existing outputs instead: %.2f GB/s "
                      "(%d threads), %.2f GB/s (1 thread)" % (sample, args.batch, int(scale), gbps_1, gbps_n_re, threads, gbps_1_re),
            "single_thread_value": round(gbps_1, 2),
            "value_existing_outputs": round(gbps_n_re, 2),
            "single_thread_value_existing_outputs": round(gbps_1_re, 2),
            "us_per_kernel_scaled": us(t_n),
            "us_per_kernel_scaled_existing_outputs": us(t_n_re),
            "us_per_kernel_scaled_1_thread": us(t_1),
            "us_per_kernel_scaled_1_thread_existing_outputs": us(t_1_re),
            "build": "g++ -O3 -march=x86-64-v3 -ffp-contract=off (oracle/Makefile)",
        }

    ctx.close()
    if args.full_json:
        os.makedirs(os.path.dirname(os.path.abspath(args.full_json)), exist_ok=True)
        with open(args.full_json, "w") as f:
            json.dump(result, f)
    sys.stderr.flush()
    print(compact_line(result), flush=True)


if __name__ == "__main__":
    main()
