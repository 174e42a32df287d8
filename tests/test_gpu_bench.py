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


def _line(*flags, timeout=900):
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True,
                         timeout=timeout)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    cfg = d["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / 8000.0) < 1e-3
    assert d["roofline"]["achieved"] > 0 and d["prefill"]["value"] > 0 and 0 < d["prefill"]["frac"] < 1
    assert abs(d["value"] - cfg["global_batch"] * 1e3 / d["ms_per_step"]) < 0.01 * d["value"]
    return d


def test_bench_unequal_batch_of_eight_with_the_3b_layers():
    """The workload of eight requests with prompts of unequal lengths (their prompts in one packed step, then
    one token each a step), with two of the 28 layers: the line keeps the contract and says what it ran."""
    d = _line("--workload", "unequal8", "--layers", "2", "--steps", "4", "--warmup", "2")
    cfg = d["config"]
    assert cfg["layers"] == 2 and cfg["layers_of_shape"] == 28 and cfg["hidden_size"] == 3072 and cfg["head_dim"] == 128
    assert cfg["global_batch"] == 8 and d["steps"] == 4 and d["warmup"] == 2 and cfg["new_tokens"] == 4
    assert 64 <= cfg["prompt_len_min"] <= cfg["prompt_len_max"] <= 2048
    assert 8 * cfg["prompt_len_min"] <= cfg["prompt_tokens"] <= 8 * cfg["prompt_len_max"]
    assert d["prefill"]["tokens"] == cfg["prompt_tokens"]
    # the mean context of the timed steps: the prompts, the warm-up steps, and half the timed steps
    assert abs(cfg["mean_context"] - (cfg["prompt_tokens"] / 8 + 2 + (4 + 1) / 2)) < 0.11


def test_bench_batch_64_and_a_prefill_of_8192_with_the_8b_layers():
    d = _line("--shape", "8b", "--layers", "2", "--batch", "64", "--prompt-len", "1024", "--prefill-len", "8192",
              "--points", "", "--steps", "3", "--warmup", "2")
    cfg = d["config"]
    assert cfg["layers"] == 2 and cfg["layers_of_shape"] == 32 and cfg["hidden_size"] == 4096
    assert cfg["intermediate_size"] == 14336 and cfg["tied_head"] is False and cfg["seq_len"] == 8192
    assert cfg["global_batch"] == 64 and cfg["prompt_len"] == 1024 and cfg["prefill_len"] == 8192
    assert d["prefill"]["tokens"] == 8192 and d["points"] == {}
