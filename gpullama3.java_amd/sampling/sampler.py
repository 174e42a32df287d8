"""Token selection: greedy, temperature, and top-p, as the reference's samplers
define them (J/inference/sampler/Sampler.java:56-104, CategoricalSampler.java:31-42,
ToppSampler.java:94-155), on the device with a host twin of the same definition.

The reference draws from one Java generator per sampler, one float per token
(Sampler.java:63, ToppSampler.java:139); its bit stream is not reproduced. Here
the uniform number of a draw depends on (seed, request, step) alone, so a
sequence's tokens do not depend on what else is in its batch.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

_M64 = (1 << 64) - 1


def _mix(z):
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def uniform(seed, request, step):
    """A float32-exact number in [0, 1) from the three counters."""
    z = _mix(int(seed) & _M64)
    z = _mix(z ^ ((int(request) + 1) * 0xD1B54A32D192ED03 & _M64))
    z = _mix(z ^ ((int(step) + 1) * 0x8CB92BA72F3D8DD7 & _M64))
    return (z >> 40) / float(1 << 24)


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0: greedy. top_p outside (0, 1): the whole distribution
    (Sampler.java:58-75). Bounds as J/Options.java:14-15."""
    temperature: float = 0.0
    top_p: float = 1.0
    seed: int = 0

    def __post_init__(self):
        if not self.temperature >= 0:
            raise ValueError("temperature must be non-negative")
        if not 0 <= self.top_p <= 1:
            raise ValueError("top_p must be within [0, 1]")


def select_sampler(vocabulary_size, temperature, top_p, seed):
    """The reference's ``Sampler.selectSampler`` by name and argument order."""
    del vocabulary_size
    return SamplingParams(float(temperature), float(top_p), int(seed))


def sample_host(logits, temperature, top_p, u):
    """The definition, in numpy: what the device kernel must return."""
    logits = np.asarray(logits, dtype=np.float32)
    if temperature == 0:
        best = np.max(logits)
        return int(np.flatnonzero(logits == best)[0]) if best > -np.inf else 0
    s = logits / np.float32(temperature)
    e = np.exp((s - np.max(s)).astype(np.float32), dtype=np.float32)
    z = np.float32(np.sum(e, dtype=np.float64))
    p = (e / z).astype(np.float32)
    p64 = p.astype(np.float64)
    if top_p <= 0 or top_p >= 1:
        cdf = np.cumsum(p64)
        hit = np.flatnonzero(u < cdf)
        return int(hit[0]) if len(hit) else len(p) - 1
    order = np.lexsort((np.arange(len(p)), -p64))
    csum = np.cumsum(p64[order])
    over = np.flatnonzero(csum > top_p)
    n_keep = int(over[0]) + 1 if len(over) else len(p)
    mass = csum[n_keep - 1]
    hit = np.flatnonzero(u * mass < csum[:n_keep])
    return int(order[hit[0]]) if len(hit) else int(order[n_keep - 1])


class DeviceSampler:
    """Runs the selection kernel on rows of logits that stay on the device."""

    def __init__(self, device):
        import torch
        self.device = device
        self._torch = torch
        self._work = None

    def __call__(self, logits, temperatures, top_ps, uniforms):
        """logits ``[R, V]`` float32 on the device -> list of R token ids."""
        torch = self._torch
        from ..csrc import lib as K
        R, V = logits.shape
        if R == 0:
            return []
        if self._work is None or self._work.numel() < K.sample_work_size(R, V):
            self._work = torch.empty(K.sample_work_size(R, V), dtype=torch.float32, device=self.device)
        out = torch.empty(R, dtype=torch.int32, device=self.device)
        if all(t == 0 for t in temperatures):           # every row greedy: the rows are read by many blocks at once
            K.argmax(logits, self._work, out)
            return out.tolist()
        par = torch.tensor([list(temperatures), list(top_ps), list(uniforms)], dtype=torch.float32).to(self.device)
        K.sample(logits, self._work, par[0], par[1], par[2], out)
        return out.tolist()
