"""Gated feed-forward: ``down(act(gate(h)) * up(h))`` added into the residual
stream; the reference's is silu without biases (J/inference/InferenceCore.java:158-172).
Gate and up are one product over the two matrices stacked by rows; the activation is the
product's epilogue, and so are biases when the description names them
(``gate_bias``, ``up_bias``, ``down_bias`` among its tensor names)."""
from __future__ import annotations

import torch

from ..csrc.lib import ACTIVATIONS
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import register_part


class GatedFeedForward:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by (T, B)
    adds_only = True       # never reads the residual rows: sums of the product before it may still lie in slices

    def __init__(self, spec, dtype, device):
        if spec.activation not in ACTIVATIONS:
            raise ValueError(f"activation {spec.activation!r} is not built ({sorted(ACTIVATIONS)})")
        self.d, self.F, self.dtype, self.names = spec.hidden, spec.intermediate, dtype, spec.names
        self.act = spec.activation
        self.biased = "gate_bias" in self.names
        if self.biased != ("up_bias" in self.names):
            raise ValueError("a gated feed-forward names the biases of gate and up together or neither")
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def tensors(self):
        n = self.names
        out = {n["gate"]: TensorSpec((self.F, self.d)), n["up"]: TensorSpec((self.F, self.d)),
               n["down"]: TensorSpec((self.d, self.F))}
        if self.biased:
            out[n["gate_bias"]] = TensorSpec((self.F,), "vector")
            out[n["up_bias"]] = TensorSpec((self.F,), "vector")
        if "down_bias" in n:
            out[n["down_bias"]] = TensorSpec((self.d,), "vector")
        return out

    def load(self, weights):
        n = self.names
        g, u = weights[n["gate"]], weights[n["up"]]
        dt = g.dtype if g.dtype == u.dtype else torch.float32
        self.w_gate_up = torch.cat([g.to(dt), u.to(dt)], dim=0).contiguous()
        weights[n["gate"]], weights[n["up"]] = self.w_gate_up[:self.F], self.w_gate_up[self.F:]
        without = getattr(self, "without", frozenset())      # the fast paths that the engine does without
        may_hold_once = getattr(self, "may_hold_once", False)
        ops.for_gated(self.w_gate_up, without=without, alone=may_hold_once)
        if may_hold_once and ops.gated_alone(self.w_gate_up, without) and ops.can_hold_once(self.w_gate_up, without):
            # the stored order is let go; the stored names then name rows that are put together on request
            self.w_gate_up = K.hold_once(self.w_gate_up)
            weights[n["gate"]] = ops.StoredRows(self, "w_gate_up", 0, self.F)
            weights[n["up"]] = ops.StoredRows(self, "w_gate_up", self.F, 2 * self.F)
        self.w_down = ops.for_eight_rows(weights[n["down"]], without=without)
        if may_hold_once and ops.can_hold_once(self.w_down, without):
            self.w_down = weights[n["down"]] = K.hold_once(self.w_down)      # (the stored order is let go)
        if self.biased:     # the epilogues read biases as float
            self.b_gate_up = torch.cat([weights[n["gate_bias"]].float(), weights[n["up_bias"]].float()]).contiguous()
        if "down_bias" in n:
            self.b_down = weights[n["down_bias"]].float().contiguous()

    def forward(self, ctx, h, x):
        if self.b_gate_up is None and self.b_down is None and ops.packs_rows(ctx, h, self.w_gate_up, self.w_down, x):
            act = ctx.buffer("ffn_act_packed", (-(-self.F // 64), 64, 8), self.dtype)
            ops.linear(h, self.w_gate_up, act, ops.EPI_GATED, ctx, act=self.act, pack_out=True)
            ops.linear(act, self.w_down, x, ops.EPI_ADD, ctx, a_packed=True)
            return
        act = ctx.buffer("ffn_act", (h.shape[0], self.F), self.dtype)
        ops.linear(h, self.w_gate_up, act, ops.EPI_GATED, ctx, bias=self.b_gate_up, act=self.act)
        ops.linear(act, self.w_down, x, ops.EPI_ADD, ctx, bias=self.b_down)


register_part("ffn", "gated", GatedFeedForward)
