"""The line bench.py prints must survive whoever runs it keeping only the tail of its standard output: one JSON object of
well under 8000 bytes whatever the number of family cases, with the headline, roofline and CPU baseline in it.  No GPU."""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

import bench  # noqa: E402


def _headline():
    return {
        "metric": "achieved HBM GB/s (algorithmic bytes) of the legacy op path: pairwise add + pairwise multiply + broadcast add row",
        "value": 6230.8, "unit": "GB/s", "n_gpus": 1, "steps": 50, "warmup": 5, "ms_per_step": 0.3447, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: pairwise add+multiply, broadcast add row; float32 [65536,1024] c-order, seed 7",
                   "elements_per_step": 201326592, "bytes_per_step": 2147487744},
        "elements_per_sec": 584140698905.5, "pct_of_peak": 77.89,
        "kernels": {n: {"ms": 0.1251, "GB/s": 6435.7, "frac": 0.8045} for n in ("pairwise_add", "pairwise_multiply", "broadcast_add_row")},
        "roofline": {"bound": "hbm", "kernel": "ewVecKernel (pairwise Add, fp32, 16-byte vectors)", "achieved": 6435.7, "peak": 8000.0,
                     "unit": "GB/s", "frac": 0.8045, "traffic": 805326634, "bytes_per_launch": 805306368, "avg_launch_ms": 0.1251},
        "cpu_baseline": {"value": 273.68, "unit": "GB/s", "cores": 16, "kind": "reference",
                         "sample": "1509 full passes of the same step (all 3 calls on the full [65536,1024] operands), median; "
                                   "7.8 ms per step, 2.57e+10 elements/s", "elements_per_sec": 25657063764.2},
    }


def _rows(count):
    return [{"case": "family_case_name_%02d" % i, "family": "transform", "ms": 0.1234, "GB/s": 6543.2, "frac": 0.81234,
             "elements_per_sec": 5.4e11, "bound": "hbm", "traffic": 805326634, "cpu_ms": 12.345,
             "note": "notes, counters and CPU times stay out of the printed line"} for i in range(count)]


def test_result_line_is_one_short_json_object():
    rows = _rows(75)  # more cases than the benchmark has
    line = bench.result_line(_headline(), rows)
    assert "\n" not in line and len(line) < 4096
    parsed = json.loads(line)
    for key in ("metric", "value", "unit", "ms_per_step", "steps", "warmup", "dtype", "config", "roofline", "cpu_baseline"):
        assert key in parsed, key
    assert parsed["roofline"]["frac"] == 0.8045 and parsed["cpu_baseline"]["kind"] == "reference"
    assert len(parsed["families"]) == 75
    assert parsed["families"]["family_case_name_03"] == [0.1234, 0.812]
    assert len(bench.result_line(_headline(), None)) < 2048


def test_result_line_refuses_to_outgrow_the_tail():
    try:
        bench.result_line(_headline(), _rows(400))
    except RuntimeError as e:
        assert "limit" in str(e)
    else:
        raise AssertionError("a line of 400 cases was printed")


def test_full_rows_go_to_a_file(tmp_path):
    path = str(tmp_path / "sub" / "families.json")
    bench.write_family_rows(path, _headline(), _rows(3))
    with open(path) as f:
        data = json.load(f)
    assert data["headline"]["value"] == 6230.8 and len(data["families"]) == 3 and "note" in data["families"][0]
