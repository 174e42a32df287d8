"""The order of a kv head's elements inside a page of the cache, for code on the host.

The kernels keep keys ``[position, head_dim]`` and values ``[head_dim, position]`` of a page in
tiles of 16 rows by 8 columns (``gl3_k_offset`` and ``gl3_v_offset`` in ``csrc/common.h`` are the
definition), so that a matrix-core operand is consecutive memory. A page's tensor keeps its plain
shape; these functions move between the plain order of that shape and the order the kernels use,
for tensors or numpy arrays whose last two axes are a page of one head. Tests and tools that fill
or read a cache by hand go through them; the engine itself never looks inside a page.
"""
from __future__ import annotations

import numpy as np


def _permute(x, axes):
    return x.transpose(axes) if isinstance(x, np.ndarray) else x.permute(*axes)


def _check(page, head_dim):
    if page % 32 or head_dim % 16:
        raise ValueError(f"the cache lies in tiles: a page of {page} positions must be a multiple of 32, "
                         f"a head of {head_dim} elements a multiple of 16")


def tile_keys(k):
    """``k[..., position, head_dim]`` in plain order -> the same shape in the kernels' order: 32
    positions are two tiles (the positions with bit 2 clear, then those with it set), a tile's
    column blocks of 8 elements one after another, 16 rows of 8 elements each."""
    *lead, page, hs = k.shape
    _check(page, hs)
    n = len(lead)
    x = k.reshape(*lead, page // 32, 4, 2, 4, hs // 8, 8)          # position = 32 g + 8 a + 4 t + b
    x = _permute(x, (*range(n), n, n + 2, n + 4, n + 1, n + 3, n + 5))   # g, t, column block, a, b, element
    return x.reshape(*lead, page, hs)


def untile_keys(k):
    *lead, page, hs = k.shape
    _check(page, hs)
    n = len(lead)
    x = k.reshape(*lead, page // 32, 2, hs // 8, 4, 4, 8)          # g, t, column block, a, b, element
    x = _permute(x, (*range(n), n, n + 3, n + 1, n + 4, n + 2, n + 5))   # g, a, t, b, column block, element
    return x.reshape(*lead, page, hs)


def tile_values(v):
    """``v[..., head_dim, position]`` in plain order -> the kernels' order: tiles of 16 dims by 8
    positions, the tiles of the same 16 dims one after another along the positions."""
    *lead, hs, page = v.shape
    _check(page, hs)
    n = len(lead)
    x = v.reshape(*lead, hs // 16, 16, page // 8, 8)
    x = _permute(x, (*range(n), n, n + 2, n + 1, n + 3))
    return x.reshape(*lead, hs, page)


def untile_values(v):
    *lead, hs, page = v.shape
    _check(page, hs)
    n = len(lead)
    x = v.reshape(*lead, hs // 16, page // 8, 16, 8)
    x = _permute(x, (*range(n), n, n + 2, n + 1, n + 3))
    return x.reshape(*lead, hs, page)
