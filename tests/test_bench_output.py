"""The line bench.py prints: one JSON document of less than 6000 characters that always carries the headline, `roofline`
and `cpu_baseline`, whatever the tables beside them hold.  Runs without a GPU on canned timings."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def _timing(nbytes, us):
    t = bench.Timing([us * 1e-3 * f for f in (0.98, 1.0, 1.03)], 4)
    return t.row(nbytes)


def canned_result(batch=256, us=12345.67):
    """Every section of a default run, with the names the default run gives its kernels and wide figures."""
    n = batch * 12 * 197 * 197 * 4
    step = ["Add(mask) [%d,12,197,197]+[%d,1,1,197]" % (batch, batch), "Softmax(-1) [%d,12,197,197]" % batch,
            "ReduceMax(axis=1) [%d,768,197]" % batch, "Div(scalar) [%d,197,768]" % batch,
            "Add(mask)+Softmax in one kernel [%d,12,197,197]" % batch]
    rows = []
    for name in step:
        r = dict({"kernel": name, "bytes": 2 * n}, **_timing(2 * n, us))
        r.update({"us_interleaved": us, "us_interleaved_median": us, "pct_hbm_peak_interleaved": 77.7})
        rows.append(r)
    shape = "[%d,197,768]" % batch
    listed_names = ["Sub %s-[%d,197,1]" % (shape, batch), "Mul %s*[768]" % shape, "Div %s/[%d,197,1]" % (shape, batch), "Pow(.,2) %s" % shape,
                    "Sqrt %s" % shape, "Erf %s" % shape, "Gelu %s" % shape, "Sigmoid %s" % shape, "HardSigmoid %s" % shape, "Relu %s" % shape,
                    "ReduceMean(-1) %s" % shape, "Softmax(-1) %s" % shape, "LayerNormalization(-1) %s" % shape]
    listed = [dict({"kernel": k, "bytes": n}, **_timing(n, us)) for k in listed_names]
    sweep = []
    for length in bench.ROW_SWEEP_LENGTHS:
        e = {"row_length": length}
        for k in ("Softmax", "LayerNormalization", "ReduceMean"):
            r = _timing(n, us)
            e[k] = {"bytes": n, "us": r["us"], "us_median": r["us_median"], "us_min": r["us_min"], "GBps": r["GBps"], "pct_hbm_peak": r["pct_hbm_peak"]}
        sweep.append(e)
    elems = bench.SHAPE_SWEEP_ELEMS
    shape_names = []
    for red, inner in bench.SHAPE_SWEEP_MIDDLE:
        for k in ("ReduceMean", "ReduceMax"):
            shape_names.append("%s(axis=1) [%d,%d,%d]" % (k, elems // (red * inner), red, inner))
    for length in bench.SHAPE_SWEEP_ODD_ROWS:
        for k in ("Softmax", "LayerNormalization", "ReduceMean"):
            shape_names.append("%s(-1) [%d,%d]" % (k, elems // length, length))
    shape_names.append("Sub [4096,4096,3] - [3]")
    for sh, perm in bench.SHAPE_SWEEP_TRANSPOSES:
        shape_names.append("Transpose %s -> %s" % (sh, tuple(perm)))
    shapes = [dict({"kernel": k, "bytes": n}, **_timing(n, us)) for k in shape_names]
    other_names = ["floor Relu [64]", "cfg0 Add [1,197,768]+[768]", "cfg1 Softmax [8,12,197,197]", "cfg1 LayerNorm [8,197,768]",
                   "cfg2 LayerNorm (fused) [32,197,768]", "cfg2 ReduceMean(-1) [32,197,768]", "cfg2 Sub [32,197,768]-[32,197,1]",
                   "cfg2 Pow(.,2) [32,197,768]", "cfg2 Div [32,197,768]/[32,197,1]", "cfg2 Mul gamma [32,197,768]*[768]",
                   "cfg3 Gelu [32,197,3072]", "cfg3 Erf [32,197,3072]", "cfg3 Mul [32,197,3072]*[32,197,3072]",
                   "cfg3 ReduceMean(H,W) [32,576,7,7]", "cfg3 HardSigmoid [32,576,1,1]", "cfg3 Mul [32,576,7,7]*[32,576,1,1]"]
    others = [dict({"kernel": k, "bytes": n, "cpu_us_16_threads": 123456.7, "cpu_us_1_thread": 1234567.8}, **_timing(n, us)) for k in other_names]
    graph_names = ["cfg2 LayerNorm chain, 9 nodes", "cfg2 after fuse_layer_norm, 1 node", "cfg2 chain after fuse_elemwise_ops, 5 nodes",
                   "cfg3 erf-GELU chain, 5 nodes", "cfg3 after fuse_gelu, 1 node", "cfg3 chain after fuse_elemwise_ops, 1 node",
                   "cfg3 squeeze-excite, 3 nodes"]
    graphs = [{"graph": g, "algorithmic_bytes": n, "kernels_us": 1234.5, "run_ms_with_pcie": 12.345, "kernels_us_graph_replay": 1234.5,
               "run_ms_with_pcie_graph_replay": 12.345, "kernels_GBps": 4283.6, "run_device_us": 1234.5, "run_device_enqueue_us": 123.4} for g in graph_names]
    per = {"Add": 32184.7, "Softmax": 12438.1, "ReduceMax": 82546.8, "Div": 10542.4}
    return {
        "metric": "per-op HBM GB/s and % of MI355X peak; us/call vs CPU interpreter", "value": 6421.3, "unit": "GB/s", "n_gpus": 1,
        "steps": 20, "warmup": 5, "ms_per_step": 0.3694, "value_after_idle": 6321.3, "ms_per_step_after_idle": 0.3794, "settle_ms": 250.0,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[4]: Add(mask)+Softmax on [%d,12,197,197], ReduceMax(axis=1) on [%d,768,197], "
                               "Div(scalar) on [%d,197,768]; one step = the four kernels once" % ((batch,) * 3),
                   "batch": batch, "step_bytes": 2372725740},
        "roofline": {"bound": "hbm", "kernel": step[1], "achieved": 6198.1, "peak": 8000.0, "unit": "GB/s", "frac": 0.7748, "traffic": 953461007,
                     "traffic_source": "x" * 190, "us_per_launch": 153.88, "us_per_launch_median": 153.5, "us_per_launch_min": 150.02,
                     "us_per_launch_in_step": 153.38, "frac_in_step": 0.7773, "launches": 100, "algorithmic_bytes": 953769984},
        "timing": "x" * 470, "per_kernel": rows, "listed_ops": listed, "row_sweep": sweep, "shape_sweep": shapes,
        "other_configs": {"kernels": others, "graphs": graphs},
        "cpu_baseline": {"value": 17.23, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "x" * 260, "single_thread_value": 9.14,
                         "value_existing_outputs": 20.38, "single_thread_value_existing_outputs": 10.5, "us_per_kernel_scaled": per,
                         "us_per_kernel_scaled_existing_outputs": per, "us_per_kernel_scaled_1_thread": per,
                         "us_per_kernel_scaled_1_thread_existing_outputs": per, "build": "g++ -O3 -march=x86-64-v3 -ffp-contract=off (oracle/Makefile)"},
    }


def test_default_line_fits_and_keeps_every_section():
    line = bench.compact_line(canned_result())
    assert len(line) < 6000, len(line)
    assert "\n" not in line
    out = json.loads(line)
    assert "dropped" not in out
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype",
                "data", "config", "roofline", "cpu_baseline", "per_kernel", "listed_ops", "row_sweep", "shape_sweep", "other_configs"):
        assert key in out, key
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "us_per_launch", "us_per_launch_in_step"):
        assert key in out["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in out["cpu_baseline"], key
    assert len(out["per_kernel"]["rows"]) == 5 and len(out["per_kernel"]["cols"]) == len(out["per_kernel"]["rows"][0])
    assert len(out["listed_ops"]["rows"]) == 13
    assert len(out["row_sweep"]["rows"]) == len(bench.ROW_SWEEP_LENGTHS) and len(out["row_sweep"]["cols"]) == 4
    assert len(out["other_configs"]["rows"]) == 16 and len(out["other_configs"]["graphs"]) == 7
    n_shapes = sum(len(g["rows"]) * (len(g["cols"]) - 1) for g in out["shape_sweep"].values())
    assert n_shapes == 2 * len(bench.SHAPE_SWEEP_MIDDLE) + 3 * len(bench.SHAPE_SWEEP_ODD_ROWS) + 1 + len(bench.SHAPE_SWEEP_TRANSPOSES)


def test_oversized_tables_are_dropped_not_the_headline():
    r = canned_result()
    r["shape_sweep"] = r["shape_sweep"] * 8
    r["listed_ops"] = r["listed_ops"] * 20
    line = bench.compact_line(r)
    assert len(line) < 6000
    out = json.loads(line)
    assert out["dropped"]
    for key in ("value", "ms_per_step", "config", "roofline", "cpu_baseline"):
        assert key in out
    assert out["roofline"]["frac"] == 0.7748 and out["cpu_baseline"]["value"] == 17.23


def test_no_optional_sections():
    r = canned_result()
    for k in ("listed_ops", "row_sweep", "shape_sweep", "other_configs", "cpu_baseline"):
        del r[k]
    out = json.loads(bench.compact_line(r))
    assert "roofline" in out and "per_kernel" in out and "cpu_baseline" not in out
