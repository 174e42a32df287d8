"""Where an element of a kv head lies inside a page of the cache, written out from the two formulas
(as index arrays, apart from the reshapes of ``gpullama3_java_amd/cache/layout.py``): the tests fill
and read pages with these, so a kernel that disagrees with the formulas fails them."""
import numpy as np
import torch


def key_index(page, hs):
    """[page, hs] -> offset inside the page: 32 positions are two tiles of 16 rows (positions with
    bit 2 clear, then set), a tile is hs/8 column blocks of 16 rows x 8 elements."""
    p, d = np.meshgrid(np.arange(page), np.arange(hs), indexing="ij")
    tile = (p >> 5) * 2 + ((p >> 2) & 1)
    row = ((p >> 3) & 3) * 4 + (p & 3)
    return ((tile * (hs >> 3) + (d >> 3)) << 7) + (row << 3) + (d & 7)


def value_index(hs, page):
    """[hs, page] (values lie transposed) -> offset inside the page: tiles of 16 dims x 8 positions."""
    d, p = np.meshgrid(np.arange(hs), np.arange(page), indexing="ij")
    return (((d >> 4) * (page >> 3) + (p >> 3)) << 7) + ((d & 15) << 3) + (p & 7)


def _scatter(x, index):
    flat = x.reshape(*x.shape[:-2], -1)
    out = torch.empty_like(flat) if isinstance(x, torch.Tensor) else np.empty_like(flat)
    idx = index.ravel()
    if isinstance(x, torch.Tensor):
        idx = torch.as_tensor(idx, device=x.device)
    out[..., idx] = flat
    return out.reshape(x.shape)


def _gather(x, index):
    flat = x.reshape(*x.shape[:-2], -1)
    idx = index.ravel()
    if isinstance(x, torch.Tensor):
        idx = torch.as_tensor(idx, device=x.device)
    return flat[..., idx].reshape(x.shape)


def tile_keys(k):            # [..., page, hs] plain -> the kernels' order
    return _scatter(k, key_index(*k.shape[-2:]))


def untile_keys(k):
    return _gather(k, key_index(*k.shape[-2:]))


def tile_values(v):          # [..., hs, page] plain -> the kernels' order
    return _scatter(v, value_index(*v.shape[-2:]))


def untile_values(v):
    return _gather(v, value_index(*v.shape[-2:]))
