"""RMSNorm: ``w * x / sqrt(mean(x^2) + eps)`` (J/inference/InferenceCore.java:47-56)."""
from __future__ import annotations

import torch

from ..csrc import lib as K
from ..weights.loader import TensorSpec
from .base import register_part
from . import ops
from .ops import Normed



class RMSNorm:
    graph_safe = True      # kernel launches on the current stream only, sizes fixed by (T, B)
    folds = True           # a product can take over this norm's work (see ``ops.Normed``)
    takes_slices = True    # adds up the slices that the product before it left, while it reads the rows anyway

    def __init__(self, spec, dtype):
        self.dim, self.eps, self.dtype = spec.dim, spec.eps, dtype
        self.name = spec.names["weight"]
        self.weight = None

    def tensors(self):
        return {self.name: TensorSpec((self.dim,), "vector")}

    def load(self, weights):
        self.weight = weights[self.name]
        # the kernels that prepare a folded norm's rows read the weight as float (exact for 16-bit storage)
        self.weight_f32 = self.weight if self.weight.dtype == torch.float32 else self.weight.float()

    def __call__(self, ctx, x, rows=None, name="normed"):
        """The normalised rows, or a ``Normed`` when the next product can do the work itself (few
        rows, and the kernel that last wrote exactly this tensor prepared the rows for this norm)."""
        rec = getattr(ctx, "ssq", None)
        if (getattr(ctx, "fuse", False) and rec is not None and rec[0] == x.data_ptr() and rec[4] is self
                and x.shape[0] <= ops.FUSE_ROWS and self.dtype == torch.bfloat16):
            return Normed(ctx, x, self.weight, self.eps, self.dtype, rec[3], rec[1], rec[2], rows, name)
        n = x.shape[0] if rows is None else rows.numel()
        out = ctx.buffer(name, (n, self.dim), self.dtype)
        pending = getattr(ctx, "pending", None)
        if pending is not None and pending[0] == x.data_ptr():
            # the product that last added to x left its sums in slices: add them up and normalise at once
            K.add_slices_rmsnorm(x, pending[1], self.weight, out, self.eps, rows)
            if rows is None:
                ctx.pending = None
            return out
        K.rmsnorm(x, self.weight, out, self.eps, rows)
        return out


register_part("norm", "rmsnorm", RMSNorm)
