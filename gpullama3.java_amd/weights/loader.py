"""Weights by tensor name, checked against what the model expects before any is used.

The reference looks tensors up by name and fails late with a null reference when
one is missing, with no shape check (J/model/loader/ModelLoader.java:285-303);
here every difference between the folder and the model is reported in one error.
"""
from __future__ import annotations

import glob
import os
from dataclasses import dataclass

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile


@dataclass(frozen=True)
class TensorSpec:
    shape: tuple
    kind: str = "matrix"      # "matrix" | "vector" | "table" (integers)


class WeightsError(ValueError):
    """Missing, unexpected or wrongly shaped tensors, all listed."""

    def __init__(self, where, missing=(), unexpected=(), wrong_shape=(), wrong_dtype=()):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_dtype = list(wrong_dtype)
        lines = [f"weights in {where} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        for name, want, found in self.wrong_shape:
            lines.append(f"  wrong shape: {name} expected {tuple(want)}, found {tuple(found)}")
        for name, found in self.wrong_dtype:
            lines.append(f"  unsupported dtype: {name} is {found}")
        super().__init__("\n".join(lines))


def weight_files(folder):
    one = os.path.join(folder, "model.safetensors")
    if os.path.isfile(one):
        return [one]
    files = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no model.safetensors (or any *.safetensors) in {folder}")
    return files


def kept_dtype(stored, kind, engine_dtype):
    """The dtype a stored tensor has on the device.

    float32 engine: every floating tensor becomes float32 (exact for 16-bit
    storage). bfloat16 engine: 16-bit floating tensors are kept in bfloat16, a
    tensor stored in 32-bit stays in 32-bit. Integer tables become int32.
    """
    if kind == "table" or not stored.is_floating_point:
        return torch.int32
    if engine_dtype == torch.float32:
        return torch.float32
    if stored in (torch.float32, torch.float64):
        return torch.float32
    return torch.bfloat16


def load_weights(folder, expected, engine_dtype, device, ignore=()):
    """``expected``: stored name -> TensorSpec. Returns name -> device tensor.

    ``ignore``: stored names that may be present without being used (a separate
    head stored beside a tied embedding is not one of them: it is reported).
    """
    files = [SafetensorsFile(p) for p in weight_files(folder)]
    try:
        where = {}
        for f in files:
            for name in f.names():
                where[name] = f
        missing = [n for n in expected if n not in where]
        unexpected = [n for n in where if n not in expected and n not in ignore]
        wrong_shape, wrong_dtype = [], []
        for name, spec in expected.items():
            f = where.get(name)
            if f is None:
                continue
            if tuple(f.shape(name)) != tuple(spec.shape):
                wrong_shape.append((name, spec.shape, f.shape(name)))
            stored = f.dtype(name)
            if spec.kind == "table" and stored.is_floating_point:
                wrong_dtype.append((name, f"{stored} (an integer table is expected)"))
            if spec.kind != "table" and not stored.is_floating_point:
                wrong_dtype.append((name, f"{stored} (a floating tensor is expected)"))
        if missing or unexpected or wrong_shape or wrong_dtype:
            raise WeightsError(folder, sorted(missing), sorted(unexpected), wrong_shape, wrong_dtype)
        out = {}
        for name, spec in expected.items():
            t = where[name].tensor(name)
            out[name] = t.to(device=device, dtype=kept_dtype(t.dtype, spec.kind, engine_dtype)).contiguous()
        return out
    finally:
        for f in files:
            f.close()


__all__ = ["TensorSpec", "WeightsError", "SafetensorsError", "load_weights", "weight_files", "kept_dtype"]
