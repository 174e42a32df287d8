"""Causal grouped-query attention over the paged cache.

Order as the reference's layer (J/inference/InferenceCore.java:78-151): q, k, v
projections (one product over the three matrices stacked by rows), rotation of q
and k, cache write at the token's position, attention over positions lo..p of the
token's own sequence, output projection added into the residual stream. The reference's
projections have no biases; a description that names ``q_bias``, ``k_bias``, ``v_bias``
(together) or ``o_bias`` among its tensors gets them added in the products' epilogues.
"""
from __future__ import annotations

import math

import torch

from ..cache import KVNeed
from ..csrc import lib as K
from ..weights.loader import TensorSpec
from . import ops
from .base import build_part, register_part


class GQAAttention:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by (T, B)
    adds_only = True       # never reads the residual rows: sums of the product before it may still lie in slices

    def __init__(self, spec, dtype, device):
        self.spec, self.dtype = spec, dtype
        self.d, self.H, self.Kh, self.hs = spec.hidden, spec.n_heads, spec.n_kv_heads, spec.head_dim
        if self.H % self.Kh:
            raise ValueError(f"{self.H} heads are not a multiple of {self.Kh} kv heads")
        self.window = spec.window
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(self.hs)
        self.position = build_part("position", spec.position, device=device) if spec.position is not None else None
        self.names = spec.names
        self.biased = "q_bias" in self.names
        if self.biased and not ("k_bias" in self.names and "v_bias" in self.names):
            raise ValueError("an attention names the biases of q, k and v together or none of them")
        self.w_qkv = self.w_q = self.w_o = self.b_qkv = self.b_o = None

    def tensors(self):
        n, d, hs = self.names, self.d, self.hs
        out = {n["q"]: TensorSpec((self.H * hs, d)), n["k"]: TensorSpec((self.Kh * hs, d)),
               n["v"]: TensorSpec((self.Kh * hs, d)), n["o"]: TensorSpec((d, self.H * hs))}
        if self.biased:
            out.update({n["q_bias"]: TensorSpec((self.H * hs,), "vector"), n["k_bias"]: TensorSpec((self.Kh * hs,), "vector"),
                        n["v_bias"]: TensorSpec((self.Kh * hs,), "vector")})
        if "o_bias" in n:
            out[n["o_bias"]] = TensorSpec((d,), "vector")
        return out

    def load(self, weights):
        n = self.names
        parts = [weights[n["q"]], weights[n["k"]], weights[n["v"]]]
        dt = parts[0].dtype if all(p.dtype == parts[0].dtype for p in parts) else torch.float32
        self.w_qkv = torch.cat([p.to(dt) for p in parts], dim=0).contiguous()
        qn, kn = self.H * self.hs, self.Kh * self.hs
        # the stored names stay addressable as views of the stacked matrix
        weights[n["q"]], weights[n["k"]], weights[n["v"]] = (
            self.w_qkv[:qn], self.w_qkv[qn:qn + kn], self.w_qkv[qn + kn:])
        self.w_q = self.w_qkv[:qn]
        without = getattr(self, "without", frozenset())      # the fast paths that the engine does without
        ops.for_few_rows(self.w_qkv, (self.H, self.Kh, self.hs, self.position is not None,
                                      bool(self.position is not None and self.position.adjacent)), without=without)
        self.w_o = ops.for_eight_rows(weights[n["o"]], without=without)
        if getattr(self, "may_hold_once", False):
            # the stored order is let go where a copy in the matrix cores' order can stand for the matrix; the stored
            # names then name rows that are put together on request
            if ops.can_hold_once(self.w_qkv, without):
                self.w_qkv, self.w_q = K.hold_once(self.w_qkv), None
                weights[n["q"]], weights[n["k"]], weights[n["v"]] = (
                    ops.StoredRows(self, "w_qkv", 0, qn), ops.StoredRows(self, "w_qkv", qn, qn + kn),
                    ops.StoredRows(self, "w_qkv", qn + kn, qn + 2 * kn))
            if ops.can_hold_once(self.w_o, without):
                self.w_o = weights[n["o"]] = K.hold_once(self.w_o)
        if self.biased:     # the epilogues read biases as float
            self.b_qkv = torch.cat([weights[n[k]].float() for k in ("q_bias", "k_bias", "v_bias")]).contiguous()
        if "o_bias" in n:
            self.b_o = weights[n["o_bias"]].float().contiguous()

    def kv_need(self):
        return KVNeed(self.Kh, self.hs, self.window)

    def state_need(self):
        return None

    def forward(self, ctx, h, x, run):
        T, H, Kh, hs = h.shape[0], self.H, self.Kh, self.hs
        k_cache, v_cache = ctx.cache.layer_kv(run.kv_entry)
        table = ctx.block_table(ctx.cache.group_index(run.kv_entry))
        q = ops.qkv_project(ctx, h, self.w_qkv, self.w_q, self.position, k_cache, v_cache, table, H, Kh, hs,
                            self.dtype, run.writes_kv, bias=self.b_qkv)
        att = ctx.buffer("attn_out", (T, H * hs), self.dtype)
        ops.attention(ctx, q, k_cache, v_cache, table, att, H, Kh, hs, self.window, self.scale)
        ops.linear(att, self.w_o, x, ops.EPI_ADD, ctx, bias=self.b_o)


register_part("mixer", "attention", GQAAttention)
