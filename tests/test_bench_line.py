"""The benchmark's last stdout line must stay short: a harness that keeps only a tail of a few KB of
stdout has to find the whole record (metric, value, roofline, cpu_baseline) in it."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("qm_bench", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _row(bound, n):
    return {"workload": "w" * 60, "us_per_step": 123.456789 + n, "us_per_step_graph": 120.123456 + n,
            "algorithmic_bytes": 593202640 + n, "algorithmic_flops": 17196646400 + n, "bound": bound,
            "cpu_oracle": {"seconds": 1.0, "sample": "x" * 200}}


def test_final_line_is_compact_and_complete():
    bench = _bench()
    per_config = {("cfg%d_" % i) + "n" * 50: _row("mfma" if i % 2 else "hbm", i) for i in range(40)}
    per_config["next_generate_end_to_end"] = {"us_per_frame": 2550.0, "frames": 96}
    line = {
        "metric": "decode_attn_hbm_GBps", "value": 5923.4, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 5,
        "ms_per_step": 0.10015, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 storage, f32 accumulate", "data": "synthetic",
        "config": {"workload": "ragged_multi_stream_decode_64x[256,4096]_paged16", "streams": 64},
        "roofline": {"bound": "hbm", "achieved": 5923.4, "peak": 8000.0, "unit": "GB/s", "frac": 0.74,
                     "traffic": 600139366, "kernel": "k" * 120},
        "cpu_baseline": {"value": 6.7, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * 150},
        "summary": bench._summary(per_config),
    }
    text = bench.compact_line(line)
    assert "\n" not in text
    assert len(text.encode()) < bench.FINAL_LINE_LIMIT < 8000
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "dtype", "config", "roofline",
                "cpu_baseline"):
        assert key in back
    assert back["roofline"]["frac"] == 0.74 and back["cpu_baseline"]["cores"] == 16


def test_summary_uses_the_bounding_peak():
    bench = _bench()
    s = bench._summary({"a": _row("hbm", 0), "b": _row("mfma", 0), "g": {"us_per_frame": 2550.04}, "skipped": {"skipped": "why"}})
    assert s["a"] == [120.12, round(593202640 / 120.123456e-6 / 8e12, 4)]
    assert s["b"] == [120.12, round(17196646400 / 120.123456e-6 / 2.5e15, 4)]
    assert s["g"] == [2550.0, None] and "skipped" not in s
