"""Random-weights mode: a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode (it only reads trained files). Every value
depends on the seed, the tensor's name and its index only, never on the order in
which tensors are made, so any reader of the folder sees the same model.
"""
from __future__ import annotations

import json
import os
import zlib

import numpy as np
import torch

from .safetensors_io import write_safetensors

_TORCH = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _generator(seed, name):
    return np.random.Generator(np.random.Philox(key=[int(seed) & (2**64 - 1), zlib.crc32(name.encode("utf-8"))]))


def random_tensor(seed, name, shape, kind, std=0.02, norm_std=0.0, vocab=None):
    """float32 (or int64 for tables) values of one tensor."""
    rng = _generator(seed, name)
    if kind == "table":
        return torch.from_numpy(rng.integers(0, vocab or 2, size=shape, dtype=np.int64))
    if kind == "vector":
        v = np.ones(shape, dtype=np.float32)
        if norm_std:
            v += np.float32(norm_std) * rng.standard_normal(shape, dtype=np.float32)
        return torch.from_numpy(v)
    out = rng.standard_normal(shape, dtype=np.float32)
    out *= np.float32(std)
    return torch.from_numpy(out)


def write_random_model(folder, config, seed, std=0.02, norm_std=0.0, dtype="bfloat16", vector_dtype=None):
    """Write ``config.json`` and ``model.safetensors`` into ``folder``.

    Matrices are N(0, std), vectors (norm weights) 1 + N(0, norm_std); ``dtype``
    is the stored dtype of matrices, ``vector_dtype`` that of vectors (default:
    the same). Returns the folder.
    """
    from ..parts.model import expected_tensors     # late: parts import the device library
    os.makedirs(folder, exist_ok=True)
    spec = config.model_spec()
    expected = expected_tensors(spec)
    mdt = _TORCH[dtype]
    vdt = _TORCH[vector_dtype] if vector_dtype else mdt
    items = []
    for name, ts in expected.items():
        if ts.kind == "table":
            out_dt = torch.int32
        else:
            out_dt = vdt if ts.kind == "vector" else mdt
        items.append((name, tuple(ts.shape), out_dt,
                      (lambda name=name, ts=ts, out_dt=out_dt: random_tensor(
                          seed, name, ts.shape, ts.kind, std, norm_std, spec.vocab_size).to(out_dt))))
    write_safetensors(os.path.join(folder, "model.safetensors"), items,
                      metadata={"format": "pt", "seed": seed, "std": std, "norm_std": norm_std})
    with open(os.path.join(folder, "config.json"), "w") as f:
        d = config.to_dict()
        d["torch_dtype"] = dtype
        json.dump(d, f, indent=1)
    return folder
