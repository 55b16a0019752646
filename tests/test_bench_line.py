"""The last stdout line of bench.py must be one strict-JSON line small enough for a log
tail to hold it whole, with the headline, `roofline` and `cpu_baseline` intact, whatever
the size of the per-op tables behind it."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def canned(n_configs=12, n_ops=25, label_len=40):
    ops = [{"op": "op%02d " % i + "x" * (label_len - 5), "bytes": 268435456, "sets": 9, "rotation_bytes": 9 * 268435456,
            "ms_median": 0.04321, "ms_best": 0.04301, "gbps": 6214.3, "frac_of_peak": 0.77678, "gelem_s": 388.1,
            "ms_median_replay": 0.0426, "frac_replay": 0.7872} for i in range(n_ops)]
    return {
        "metric": bench.METRIC, "value": 6088.3, "unit": "GB/s", "n_gpus": 1, "steps": 50, "warmup": 5, "ms_per_step": 0.0882,
        "value_replay": 6186.7, "ms_per_step_python_host": 0.09031, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": bench.WORKLOAD_TEXT["c2"], "rotation": "r" * 90, "bytes_per_step": 536969216,
                   "launches_per_step": 3, "frac_of_hbm_peak": 0.761, "gelem_per_s": 570.67},
        "roofline": {"bound": "hbm", "kernel": "k" * 90, "achieved": 6214.3, "peak": 8000.0, "unit": "GB/s", "frac": 0.7768,
                     "bytes_per_launch": 268468224, "avg_launch_ms": 0.0432, "median_launch_ms": 0.04321, "method": "m" * 90,
                     "traffic": 268469633, "frac_replay": 0.7872, "avg_launch_ms_replay": 0.04263},
        "cpu_baseline": {"value": 26.109, "unit": "GB/s", "cores": 1, "kind": "port", "sample": "s" * 220, "ms_per_step": 20.566},
        "per_config": {"cfg%02d" % c: {"workload": "w" * 100, "ops": ops} for c in range(n_configs)},
        "host_io": {"bytes": 1 << 28, "unit": "GB/s", "ingest_staged": 50.1},
        "host_cost": {"unit": "us per operation", "empty_launch": 1.54, "launcher_add": 3.0, "add_alloc_free": 3.27, "sum_alloc_free": 3.89},
    }


HEADLINE = ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
            "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline")


def strict_loads(line):
    def refuse(tok):
        raise ValueError("not strict JSON: " + tok)
    return json.loads(line, parse_constant=refuse)


def test_final_line_is_small_and_strict():
    out = canned(n_configs=10, n_ops=10, label_len=24)
    line = bench.final_line(out, "gpurun_out/bench_full.json")
    assert "\n" not in line
    assert len(line) <= bench.FINAL_LINE_MAX
    got = strict_loads(line)
    for k in HEADLINE:
        assert got[k] == out[k], k
    assert got["full_results"] == "gpurun_out/bench_full.json"
    # the per-op map: one number per op
    assert set(got["per_config"]) == set(out["per_config"])
    one = got["per_config"]["cfg00"]
    assert len(one) == 10 and all(isinstance(v, float) for v in one.values())
    assert "host_io" not in got and "host_cost" not in got
    assert got["host_cost_us"]["launcher_add"] == 3.0


def test_final_line_drops_the_map_before_the_headline():
    out = canned(n_configs=12, n_ops=25, label_len=60)   # a per-op map that alone is over the limit
    line = bench.final_line(out, None)
    assert len(line) <= bench.FINAL_LINE_MAX
    got = strict_loads(line)
    assert "per_config" not in got and got["per_config_omitted"]
    for k in HEADLINE:
        assert got[k] == out[k], k


def test_full_table_goes_to_a_file(tmp_path):
    out = canned(2, 3)
    path = bench.write_full(out, str(tmp_path / "sub" / "full.json"))
    assert path is not None
    with open(tmp_path / "sub" / "full.json") as f:
        assert json.load(f) == out


def test_real_labels_fit():
    """The op labels the bench really uses, with plausible numbers: the compact line must
    hold the whole per-op map (nothing dropped) for the default run."""
    import inspect
    import re
    src = inspect.getsource(bench)
    labels = set(re.findall(r'\("([^"\n]{1,60})",\s*lambda', src))
    assert len(labels) > 50, "op labels not found in bench.py; adapt this test to its table format"
    out = canned(1, 1)
    out["per_config"] = {"all": {"workload": "", "ops": [{"op": l, "frac_of_peak": 0.77777} for l in sorted(labels)]}}
    line = bench.final_line(out, "gpurun_out/bench_full.json")
    assert "per_config_omitted" not in strict_loads(line)
