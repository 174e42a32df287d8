"""Weights: container, random-weights mode, and the one error that lists everything (no GPU)."""
import json
import os
import struct

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import gpullama3_java_amd as g
from gpullama3_java_amd.parts import DecoderModel
from gpullama3_java_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError, kept_dtype, load_weights,
                                        random_tensor, write_random_model, write_safetensors)
from tiny import TINY_A, TINY_B, tensor_shapes


def expected(cfgd):
    return DecoderModel(g.config_from_dict(cfgd).model_spec(), torch.float32, "cpu").expected()


def test_expected_tensors_are_the_architecture_s_names():
    for cfgd in (TINY_A, TINY_B):
        exp = expected(cfgd)
        assert {n: tuple(t.shape) for n, t in exp.items()} == tensor_shapes(cfgd)


def test_container_round_trip_against_the_library(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int32),
         "c": torch.randn(4), "empty": torch.zeros(0, 2)}
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, t, metadata={"k": "v"})
    lib = load_file(p)
    for k in t:
        assert torch.equal(lib[k], t[k])
    save_file(t, str(tmp_path / "y.safetensors"))
    f = SafetensorsFile(str(tmp_path / "y.safetensors"))
    assert sorted(f.names()) == sorted(t)
    for k in t:
        assert torch.equal(f.tensor(k), t[k]) and f.dtype(k) == t[k].dtype
    f.close()


def test_truncated_and_broken_files(tmp_path):
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, {"a": torch.randn(64, 64)})
    blob = open(p, "rb").read()
    open(p, "wb").write(blob[:-100])
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 10**9) + b"{}")
    with pytest.raises(SafetensorsError, match="header"):
        SafetensorsFile(p)
    open(p, "wb").write(b"abc")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(p)


def _with_header(path, header, data_bytes):
    import json
    h = json.dumps(header).encode()
    open(path, "wb").write(struct.pack("<Q", len(h)) + h + bytes(data_bytes))


def test_byte_ranges_that_are_no_ranges_or_overlap_are_refused(tmp_path):
    p = str(tmp_path / "y.safetensors")
    ok = {"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}, "b": {"dtype": "F32", "shape": [4], "data_offsets": [16, 32]}}
    _with_header(p, ok, 32)
    SafetensorsFile(p).close()
    # a range that starts before the data (it would read the header's own bytes as weights)
    _with_header(p, {"a": {"dtype": "F32", "shape": [4], "data_offsets": [-16, 0]}}, 32)
    with pytest.raises(SafetensorsError, match="no range"):
        SafetensorsFile(p)
    _with_header(p, {"a": {"dtype": "F32", "shape": [4], "data_offsets": [16, 0]}}, 32)
    with pytest.raises(SafetensorsError, match="no range"):
        SafetensorsFile(p)
    # two tensors over the same bytes
    both = {"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}, "b": {"dtype": "F32", "shape": [4], "data_offsets": [8, 24]}}
    _with_header(p, both, 32)
    with pytest.raises(SafetensorsError, match="overlap"):
        SafetensorsFile(p)


def test_random_model_folder(tmp_path):
    cfg = g.config_from_dict(TINY_B)
    d1 = write_random_model(str(tmp_path / "m1"), cfg, seed=5, norm_std=0.1)
    d2 = write_random_model(str(tmp_path / "m2"), cfg, seed=5, norm_std=0.1)
    d3 = write_random_model(str(tmp_path / "m3"), cfg, seed=6, norm_std=0.1)
    a, b, c = (load_file(os.path.join(d, "model.safetensors")) for d in (d1, d2, d3))
    assert set(a) == set(tensor_shapes(TINY_B))
    assert all(torch.equal(a[k], b[k]) for k in a)                       # a seed fixes the model
    assert not torch.equal(a["lm_head.weight"], c["lm_head.weight"])
    assert a["lm_head.weight"].dtype == torch.bfloat16
    w = a["model.layers.1.mlp.up_proj.weight"].float()
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.002
    nw = a["model.norm.weight"].float()
    assert abs(nw.mean().item() - 1) < 0.05 and 0.05 < nw.std().item() < 0.15
    # values depend on (seed, name) only: making one tensor alone gives the same numbers
    alone = random_tensor(5, "lm_head.weight", (384, 96), "matrix", 0.02).to(torch.bfloat16)
    assert torch.equal(alone, a["lm_head.weight"])
    assert g.load_config(d1) == cfg
    assert json.load(open(os.path.join(d1, "config.json")))["architectures"] == ["LlamaForCausalLM"]


def test_tied_model_has_no_head_tensor(tmp_path):
    d = write_random_model(str(tmp_path / "m"), g.config_from_dict(TINY_A), seed=1)
    assert "lm_head.weight" not in load_file(os.path.join(d, "model.safetensors"))


def test_one_error_lists_missing_unexpected_and_shapes(tmp_path):
    cfg = g.config_from_dict(TINY_B)
    d = write_random_model(str(tmp_path / "m"), cfg, seed=2)
    t = load_file(os.path.join(d, "model.safetensors"))
    del t["model.layers.0.self_attn.k_proj.weight"]
    del t["lm_head.weight"]
    t["model.layers.9.mlp.up_proj.weight"] = torch.zeros(2, 2)
    t["model.layers.1.mlp.down_proj.weight"] = t["model.layers.1.mlp.down_proj.weight"].t().contiguous()
    t["model.norm.weight"] = torch.zeros(96, dtype=torch.int32)
    save_file(t, os.path.join(d, "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_weights(d, expected(TINY_B), torch.bfloat16, "cpu")
    err = e.value
    assert err.missing == ["lm_head.weight", "model.layers.0.self_attn.k_proj.weight"]
    assert err.unexpected == ["model.layers.9.mlp.up_proj.weight"]
    assert err.wrong_shape == [("model.layers.1.mlp.down_proj.weight", (96, 320), (320, 96))]
    assert err.wrong_dtype and err.wrong_dtype[0][0] == "model.norm.weight"
    msg = str(err)
    for word in ("missing (2)", "lm_head.weight", "unexpected (1)", "expected (96, 320), found (320, 96)"):
        assert word in msg
    with pytest.raises(FileNotFoundError):
        load_weights(str(tmp_path), expected(TINY_B), torch.bfloat16, "cpu")


def test_kept_dtypes(tmp_path):
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert kept_dtype(bf, "matrix", bf) == bf and kept_dtype(f16, "matrix", bf) == bf
    assert kept_dtype(f32, "vector", bf) == f32                 # stored in 32-bit: stays so
    assert kept_dtype(bf, "matrix", f32) == f32 and kept_dtype(f32, "matrix", f32) == f32
    assert kept_dtype(torch.int64, "table", bf) == torch.int32
    cfg = g.config_from_dict(TINY_A)
    d = write_random_model(str(tmp_path / "m"), cfg, seed=3, norm_std=0.1, vector_dtype="float32")
    w = load_weights(d, expected(TINY_A), bf, "cpu")
    assert w["model.norm.weight"].dtype == f32 and w["model.embed_tokens.weight"].dtype == bf
    w32 = load_weights(d, expected(TINY_A), f32, "cpu")
    assert all(t.dtype == f32 for t in w32.values())
    assert torch.equal(w32["model.embed_tokens.weight"], w["model.embed_tokens.weight"].float())
