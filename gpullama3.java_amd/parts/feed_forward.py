"""Gated feed-forward: ``down(silu(gate(h)) * up(h))`` added into the residual
stream (J/inference/InferenceCore.java:158-172). Gate and up are one product over
the two matrices stacked by rows; the activation is the product's epilogue."""
from __future__ import annotations

import torch

from ..weights.loader import TensorSpec
from . import ops
from .base import register_part


class GatedFeedForward:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by (T, B)

    def __init__(self, spec, dtype, device):
        if spec.activation != "silu":
            raise ValueError(f"activation {spec.activation!r} is not built (silu)")
        self.d, self.F, self.dtype, self.names = spec.hidden, spec.intermediate, dtype, spec.names
        self.w_gate_up = self.w_down = None

    def tensors(self):
        n = self.names
        return {n["gate"]: TensorSpec((self.F, self.d)), n["up"]: TensorSpec((self.F, self.d)),
                n["down"]: TensorSpec((self.d, self.F))}

    def load(self, weights):
        n = self.names
        g, u = weights[n["gate"]], weights[n["up"]]
        dt = g.dtype if g.dtype == u.dtype else torch.float32
        self.w_gate_up = torch.cat([g.to(dt), u.to(dt)], dim=0).contiguous()
        weights[n["gate"]], weights[n["up"]] = self.w_gate_up[:self.F], self.w_gate_up[self.F:]
        self.w_down = weights[n["down"]]

    def forward(self, ctx, h, x):
        act = ctx.buffer("ffn_act", (h.shape[0], self.F), self.dtype)
        ops.linear(h, self.w_gate_up, act, ops.EPI_GATED, ctx)
        ops.linear(act, self.w_down, x, ops.EPI_ADD, ctx)


register_part("ffn", "gated", GatedFeedForward)
