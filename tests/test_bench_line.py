"""bench.py's output contract, checked without a GPU: the LAST line of stdout is one compact, strict JSON object
(headline + roofline + cpu_baseline + a short targets block), the per-shape tables go on earlier lines."""
import json
import math

import pytest

import bench


def stub_result():
    return {
        "metric": bench.METRIC, "value": 212.345, "unit": "TFLOP/s", "n_gpus": 1, "steps": 200, "warmup": 20,
        "ms_per_step": 0.015234, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic", "samples_per_s": 33609876.5,
        "config": {"workload": "linear_1024x1024_fp16_FW+WG+IG_batched_N512", "in": 1024, "out": 1024, "batch": 512,
                   "accumulate": "f32", "layout": "W[out][in], X[batch][in]"},
        "roofline": {"bound": "mfma", "achieved": 204.1, "peak": 2500.0, "unit": "TFLOP/s", "frac": 0.08164,
                     "traffic": 13270000.0, "kernel": "k" * 160, "flops_per_launch": 1610612736.0,
                     "launches_per_step": 2, "avg_launch_us": 7.891, "traffic_note": "n" * 120,
                     "event_ms_per_step": 0.015782},
        "host_staged": {"ms_per_step": 1.2345, "TFLOP/s": 2.609, "note": "n" * 90},
        "cpu_baseline": {"value": 0.004213, "unit": "TFLOP/s", "cores": 8, "kind": "port", "sample": "s" * 130},
    }


def stub_detail():
    rows = []
    for _, names, field in bench.TARGET_ROWS:
        for n in names:
            rows.append({"workload": n + (" N=128, 92 launches" if n.startswith("resnet20") else ""), "dtype": "fp16",
                         "us": 123.45, "TFLOP/s": 987.654, "GB/s": 5432.1, "bound_TFLOP/s": 2500.0,
                         "frac_of_bound": 0.3951, "samples/s": 161234.5})
    # and a long tail of rows that the headline does not quote
    rows += [{"workload": "conv2d %d->%d 56x56 k3 p1 FW N=128" % (i, i), "dtype": "fp16", "us": 1.0 + i,
              "TFLOP/s": 1.0, "GB/s": 2.0, "bound_TFLOP/s": 2500.0, "frac_of_bound": 0.1} for i in range(120)]
    return rows


def test_last_line_is_compact_strict_json():
    cpu = [{"workload": "linear 1024x1024 FW N=1", "dtype": "fp32", "us": 400.0, "TFLOP/s": 0.005, "threads": 8,
            "kind": "port", "sample": "one call, median of 21"}] * 20
    lines = bench.compose_output(stub_result(), cpu, stub_detail())
    assert all("\n" not in l for l in lines)
    last = lines[-1]
    assert len(last) < bench.MAX_LAST_LINE <= 4096

    def reject(c):
        raise ValueError("non-finite constant " + c)
    head = json.loads(last, parse_constant=reject)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "dtype", "config", "roofline",
                "cpu_baseline", "targets", "higher_is_better", "scaling", "vs_baseline", "data"):
        assert key in head, key
    assert "detail" not in head and "cpu_baseline_detail" not in head
    assert len(head["targets"]) <= 10
    assert all(v is not None for vals in head["targets"].values() for v in (vals if isinstance(vals, list) else [vals]))
    assert head["targets"]["resnet20_fp16_N128_step_samples/s"] == 161234.5
    for k in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert k in head["roofline"]
    for k in ("value", "unit", "cores", "kind", "sample"):
        assert k in head["cpu_baseline"]
    # every earlier line is a one-row object of one of the two tables
    kinds = [next(iter(json.loads(l, parse_constant=reject))) for l in lines[:-1]]
    assert kinds.count("cpu_baseline_detail") == 20 and kinds.count("detail") == len(stub_detail())


def test_headline_without_tables_and_non_finite_numbers():
    lines = bench.compose_output(stub_result(), [], [])
    assert len(lines) == 1 and "targets" not in json.loads(lines[0])
    bad = stub_result()
    bad["value"] = math.nan
    with pytest.raises(ValueError):
        bench.compose_output(bad, [], [])
    long = stub_result()
    long["roofline"]["kernel"] = "k" * 5000
    with pytest.raises(RuntimeError):
        bench.compose_output(long, [], [])
