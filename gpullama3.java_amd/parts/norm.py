"""RMSNorm: ``w * x / sqrt(mean(x^2) + eps)`` (J/inference/InferenceCore.java:47-56)."""
from __future__ import annotations

import torch

from ..csrc import lib as K
from ..weights.loader import TensorSpec
from .base import register_part


class RMSNorm:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by (T, B)

    def __init__(self, spec, dtype):
        self.dim, self.eps, self.dtype = spec.dim, spec.eps, dtype
        self.name = spec.names["weight"]
        self.weight = None

    def tensors(self):
        return {self.name: TensorSpec((self.dim,), "vector")}

    def load(self, weights):
        self.weight = weights[self.name]

    def __call__(self, ctx, x, rows=None, name="normed"):
        n = x.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(name, (n, self.dim), self.dtype)
        K.rmsnorm(x, self.weight, out, self.eps, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
