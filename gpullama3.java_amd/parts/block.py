"""A layer: the arrangement of norm, mixer and feed-forward.

``prenorm`` is the reference's: the normalised copy feeds the mixer, the residual
stream keeps the sum (J/inference/InferenceCore.java:74, :151, :154, :172).
"""
from __future__ import annotations

from . import ops
from .base import build_part, register_part


class PreNormBlock:
    def __init__(self, spec, dtype, device):
        self.mixer_norm = build_part("norm", spec.mixer_norm, dtype=dtype)
        self.mixer = build_part("mixer", spec.mixer, dtype=dtype, device=device)
        self.ffn_norm = build_part("norm", spec.ffn_norm, dtype=dtype) if spec.ffn is not None else None
        self.ffn = build_part("ffn", spec.ffn, dtype=dtype, device=device) if spec.ffn is not None else None

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def cache_needs(self):
        return self.mixer.kv_need(), self.mixer.state_need()

    def first_norm(self):
        """The norm that reads the residual rows first: the block before this one may prepare its rows."""
        return self.mixer_norm

    def forward(self, ctx, x, run, norm_after=None):
        """``norm_after``: the norm that reads the residual rows after this block, if known."""
        h = self._whole_rows_for(self.mixer_norm, "takes_slices", ctx, x)(ctx, x)
        ctx.next_norm = self.ffn_norm if self.ffn is not None else norm_after
        self._whole_rows_for(self.mixer, "adds_only", ctx, x).forward(ctx, h, x, run)
        if self.ffn is not None:
            h = self._whole_rows_for(self.ffn_norm, "takes_slices", ctx, x)(ctx, x)
            ctx.next_norm = norm_after
            self._whole_rows_for(self.ffn, "adds_only", ctx, x).forward(ctx, h, x)
        ctx.next_norm = None

    @staticmethod
    def _whole_rows_for(part, declares, ctx, x):
        """A product of 17 or more rows may have left its sums in slices beside the residual rows. A norm
        that adds them up itself says so (``takes_slices``), a mixer or feed-forward that only adds to the rows
        says that (``adds_only``); for any other part the rows are made whole before it runs, so a part that
        knows nothing of slices reads what it expects."""
        if not getattr(part, declares, False):
            ops.settle_residual(ctx, x)
        return part


register_part("block", "prenorm", PreNormBlock)
