"""bench.py's line: one JSON object with the fields its readers depend on."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_prints_one_json_line_with_its_contract():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--layers", "1", "--steps", "3", "--warmup", "2",
                          "--points", "1"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 2 and d["higher_is_better"] is True
    assert d["dtype"] == "bf16" and d["unit"] == "tokens/s" and d["value"] > 0
    cfg = d["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())   # flat, at most 20 keys
    assert cfg["layers"] == 1 and cfg["layers_of_shape"] == 16 and cfg["global_batch"] == 8 and cfg["seq_len"] == 4096
    assert abs(d["value"] - 8 * 1e3 / d["ms_per_step"]) < 0.01 * d["value"]
    assert set(d["prefill"]) == {"value", "tokens", "ms", "frac"} and d["prefill"]["tokens"] == 2048
    assert set(d["roofline"]) == {"bound", "achieved", "peak", "unit", "frac"} and d["roofline"]["peak"] == 8000.0
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / 8000.0) < 1e-3
    assert set(d["points"]) == {"decode_b1"}


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 2 and len(out.stdout.strip().splitlines()) == 1
