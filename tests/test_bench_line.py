"""The one JSON line bench.py prints must stay short enough to survive a log tail: built here from canned
numbers (as many ops as the full run measures, long plan strings, a long CPU sample text) and measured."""
import json
import sys
from pathlib import Path

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

import bench  # noqa: E402  (imports numpy and ctypes only; nothing touches a device)


def canned_ops(n_extra=60):
    keys = list(bench.SUMMARY_KEYS) + ["C2.layernorm"]
    keys += ["ref.sum(%s)" % a for a in ("0", "1", "2", "0,1", "0,2", "1,2", "0,1,2")]
    keys += [f"ref.softmax{n}({a})" for n in (256, 512) for a in range(3)]
    keys += [None] * n_extra
    ops = []
    for i, k in enumerate(keys):
        fields = {"key": k, "config": "f32 [1016800,33] (short odd rows) " + "x" * 40, "op": "log_softmax(axis=1)",
                  "dtype": "f32", "algorithmic_bytes": 268468224 + i, "rows": 8192,
                  "plan": "rowreg-lds-shift rows=4096 cols=30522 vec=4 tpr=512 rpb=1 nchunk=28 ostride=1 max_blocks=1024"}
        ops.append(bench.op_record(fields, [46.0 + 0.01 * j for j in range(bench.GROUPS)]))
    return ops


def canned_line(ops):
    cpu = {"value": 93.21, "unit": "GB/s", "cores": 16, "kind": "port", "rows_per_s": 2.6e6,
           "sample": "400 passes of the full f32 [8192,4096] layernorm (median 3.1 ms/pass, 2642580 rows/s)",
           "port_max_abs_err_vs_f64_oracle": 2e-5}
    extra = {"plan": "rowreg rows=8192 cols=4096 vec=4 tpr=256 rpb=1 nchunk=4 ostride=1 max_blocks=768",
             "kernel": "void hpt::row_reg_kernel<2, float, 4, 4, 1, false, false, false>(hpt::NormArgs)",
             "profile_matches_plan": True, "profiler_kernel_us": 46.14, "traffic": 268784095}
    return bench.summary_line(20, 5, 0.00095, 0.93, 268468224, 8192, 4, extra, cpu, ops)


def test_line_is_short_and_complete():
    ops = canned_ops()
    line = canned_line(ops)
    text = bench.encode_line(line)
    assert len(text.encode()) < bench.MAX_LINE_BYTES
    assert "\n" not in text
    back = json.loads(text)
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in back, k
    assert back["config"]["workload"].startswith("LayerNorm")
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "kernel_us", "plan"):
        assert k in back["roofline"], k
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in back["cpu_baseline"], k
    assert len(back["configs_pct_of_hbm_peak"]) <= bench.MAX_SUMMARY_OPS
    assert len(back["reference_shapes_pct_of_hbm_peak"]) == 13
    assert "ops" not in back and back["ops_measured"] == len(ops)
    # frac is achieved / peak, achieved is bytes over the event time
    r = back["roofline"]
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert abs(r["achieved"] - 268468224 / (0.93e-3 / 20) / 1e9) < 1.0


def test_line_length_does_not_grow_with_the_number_of_ops():
    a = len(bench.encode_line(canned_line(canned_ops(10))))
    b = len(bench.encode_line(canned_line(canned_ops(500))))
    assert abs(a - b) <= 4      # only the digits of `ops_measured`


def test_line_without_cpu_leg_and_without_other_ops():
    line = bench.summary_line(20, 5, 0.001, 0.95, 268468224, 8192, 4, {"plan": "p"}, None, [])
    text = bench.encode_line(line)
    back = json.loads(text)
    assert back["cpu_baseline"] is None and back["ops_file"] is None
    assert back["configs_pct_of_hbm_peak"] == {}
