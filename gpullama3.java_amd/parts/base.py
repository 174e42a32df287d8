"""What every part must offer, and the registries that build parts from descriptions.

A part is built from its description (``config/specs.py``) and the engine's dtype;
it names the stored tensors it needs (``tensors``), receives them (``load``) and
works on the packed activations of one step. No part knows which model it is in:
sizes and constants come from the description, everything about the step (which
token belongs to which sequence, positions, the cache) from the step context.

Interfaces
----------
Norm:         ``__call__(ctx, x[T,d] float32, rows=None) -> [R,d]`` in the activation dtype.
Mixer:        ``forward(ctx, h[T,d], x[T,d] float32, run)`` adds its output into ``x``;
              ``kv_need()`` / ``state_need()`` tell the cache what one run-order entry stores.
FeedForward:  ``forward(ctx, h[T,d], x[T,d] float32)`` adds its output into ``x``.
Position:     built by the mixer that uses it from its description (``build_part("position", ...)``).
Block:        ``parts()`` and ``forward(ctx, x, run)``; owns the arrangement of norm, mixer and
              feed-forward. Optional: ``cache_needs() -> (KVNeed | None, StateNeed | None)`` (else the
              one part with ``kv_need`` is asked), and ``first_norm()``, with which the block takes
              part in the folding of norms into products and is called with ``norm_after=``.

The residual rows ``x`` between parts: parts only ADD to ``x`` (through ``ops.linear`` with the add
epilogue, or with a kernel of their own followed by ``ops.residual_written``). After a product of 17
or more rows the sums may still lie in slices that the next norm adds up, so whoever READS ``x``
other than through a norm calls ``ops.settle_residual(ctx, x)`` first. A block without ``first_norm``
is handed whole rows, and no product leaves slices or prepared rows while it runs
(``DecoderModel.forward`` sees to both), so an arrangement of one's own need not know any of this.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

_REGISTRY = {"norm": {}, "mixer": {}, "ffn": {}, "position": {}, "block": {}}


def register_part(category, kind, cls):
    """Make ``cls`` the part built for descriptions whose ``kind`` is ``kind``."""
    if category not in _REGISTRY:
        raise KeyError(f"unknown part category {category!r}; known: {sorted(_REGISTRY)}")
    _REGISTRY[category][kind] = cls
    return cls


def build_part(category, spec, **kw):
    kinds = _REGISTRY[category]
    kind = getattr(spec, "kind", None)
    if kind not in kinds:
        raise KeyError(f"no {category} part of kind {kind!r}; registered: {sorted(kinds)}")
    return kinds[kind](spec, **kw)


@dataclass(frozen=True)
class RunInfo:
    """One entry of the run order as a part sees it."""
    entry: int                  # index in the run order: owns state and, unless it reads, keys and values
    kv_entry: Optional[int]     # the entry whose keys and values are read
    writes_kv: bool             # false when this entry reads another entry's keys and values
