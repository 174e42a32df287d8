"""Rotary position encoding: the table of cos and sin per position.

Built on the host exactly as the reference builds it
(J/inference/operation/RoPE.java:6-37): frequency ``1/theta^(i/hs)`` with the pow
in double cast to float, the llama3 rule on the wavelength in float, the angle
``pos * freq`` in float, cos and sin in double cast to float. The rotation itself
is part of the kernel that writes the cache.
"""
from __future__ import annotations

import math
import weakref

import numpy as np
import torch

from .base import register_part

_F = np.float32


def frequencies(head_dim, theta, scaling):
    out = np.zeros(head_dim // 2, dtype=_F)
    for n, i in enumerate(range(0, head_dim, 2)):
        freq = _F(1.0 / math.pow(theta, i / head_dim))
        if scaling is not None:
            factor, lo, hi = _F(scaling.factor), _F(scaling.low_freq_factor), _F(scaling.high_freq_factor)
            old = _F(scaling.original_max_position)
            wavelen = _F(2.0 * math.pi / float(freq))
            if wavelen < _F(old / hi):
                pass
            elif wavelen > _F(old / lo):
                freq = _F(freq / factor)
            else:
                smooth = _F(_F(_F(old / wavelen) - lo) / _F(hi - lo))
                freq = _F(_F(_F(_F(1.0) - smooth) * freq / factor) + _F(smooth * freq))
        out[n] = freq
    return out


class _Tables:
    """cos and sin of one description on one device."""

    def __init__(self, cos, sin):
        self.cos, self.sin = cos, sin


class Rotary:
    """cos/sin ``[max_positions, head_dim/2]`` float32 on the device. The layers of a model (and models
    with the same description) share one pair of tables; the pair lives as long as a part holds it and
    is freed with the last engine that used it."""
    _tables = weakref.WeakValueDictionary()

    def __init__(self, spec, device):
        if spec.head_dim % 2:
            raise ValueError(f"rotary encoding needs an even head size, got {spec.head_dim}")
        self.spec, self.device = spec, device
        self.rot_dim = spec.head_dim
        self.adjacent = spec.pairing == "adjacent"
        self.max_positions = spec.max_positions
        self._held = None

    def _table(self):
        if self._held is None:
            spec = self.spec
            key = (spec.head_dim, spec.theta, spec.scaling, spec.max_positions, str(self.device))
            held = Rotary._tables.get(key)
            if held is None:
                freq = frequencies(spec.head_dim, spec.theta, spec.scaling)
                pos = np.arange(spec.max_positions, dtype=_F)[:, None]
                val = (pos * freq[None, :]).astype(_F).astype(np.float64)
                held = _Tables(torch.from_numpy(np.cos(val).astype(_F)).to(self.device),
                               torch.from_numpy(np.sin(val).astype(_F)).to(self.device))
                Rotary._tables[key] = held
            self._held = held
        return self._held

    @property
    def cos(self):
        return self._table().cos

    @property
    def sin(self):
        return self._table().sin


register_part("position", "rotary", Rotary)
