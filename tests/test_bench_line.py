"""The bench's last stdout line must stay small enough for a reader that keeps only the tail of stdout."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _record(n_mfma_rows, sample_len):
    return {
        "metric": "m", "value": 3200.0, "unit": "GB/s", "n_gpus": 1, "steps": 200, "warmup": 50, "ms_per_step": 0.1,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "w" * 300, "launches_per_step": 12},
        "roofline": {"bound": "hbm", "achieved": 3200.0, "peak": 8000.0, "unit": "GB/s", "frac": 0.4, "traffic": 1},
        "roofline_mfma": [dict(kernel="k" * 30, K=4096, N=28672, M=4096, flops_per_launch=9.6e11, avg_ns=800000,
                               peak_TFLOPs=2500.0, frac=0.48, vendor_ns=640000) for _ in range(n_mfma_rows)],
        "cpu_baseline": {"value": 0.3, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * sample_len},
        "extra": {f"section{i}": [dict(a=1.0, b=2.0)] * 200 for i in range(10)},
    }


def test_final_line_is_compact_and_round_trips():
    b = _bench()
    for rows, sample in ((8, 400), (8, 5000), (200, 400)):
        line = b.final_line(_record(rows, sample))
        assert len(line) <= b.MAX_LINE_BYTES <= 8192 and "\n" not in line
        d = json.loads(line)
        assert "extra" not in d
        assert d["roofline"]["frac"] == 0.4 and d["cpu_baseline"]["cores"] == 16 and d["value"] == 3200.0


def test_extra_goes_to_a_side_file(tmp_path):
    b = _bench()
    p = tmp_path / "x" / "extra.json"
    b.write_extra({"prefill": [dict(K=1)]}, str(p))
    assert json.loads(p.read_text()) == {"prefill": [{"K": 1}]}
