"""Where an element of a key or a value lies inside a page of the cache.

A page keeps the keys of one head as [PAGE slots][head_dim] and its values transposed,
[head_dim][PAGE slots]; within each of these rows the groups of eight elements lie in a
permuted order (``sb_key_index`` / ``sb_value_index`` of csrc/sb_hip.h): the order in which the
matrix-core attention reads a page out of LDS without bank conflicts, so that a page is copied
there as it lies.  Kernels know the order; whoever reads or writes a cache tensor from Python
(tests, a part that keeps keys and values of its own and looks into them) goes through here.
"""
from __future__ import annotations

import functools

import numpy as np
import torch

from ..csrc.header import PAGE


def key_swizzle(slot: int, head_dim: int) -> int:
    if head_dim % 16:
        return 0
    groups = head_dim // 8
    mask = 15 if groups % 16 == 0 else 7 if groups % 8 == 0 else 3 if groups % 4 == 0 else 1
    return ((slot & 3) | (((slot >> 3) & 3) << 2)) & mask


@functools.lru_cache(maxsize=None)
def key_positions(head_dim: int) -> np.ndarray:
    """int64 [PAGE, head_dim]: where element d of the key at slot j lies within row j."""
    out = np.empty((PAGE, head_dim), dtype=np.int64)
    d = np.arange(head_dim)
    for j in range(PAGE):
        out[j] = (((d >> 3) ^ key_swizzle(j, head_dim)) << 3) | (d & 7)
    return out


@functools.lru_cache(maxsize=None)
def value_positions(head_dim: int) -> np.ndarray:
    """int64 [head_dim, PAGE]: where the value of slot j lies within row d."""
    d = np.arange(head_dim)[:, None]
    j = np.arange(PAGE)[None, :]
    return ((((j >> 3) ^ ((d >> 1) & 7)) << 3) | (j & 7)).astype(np.int64)


def _index(a: np.ndarray, like: torch.Tensor) -> torch.Tensor:
    return torch.from_numpy(a).to(like.device)


def keys_in_order(k_cache: torch.Tensor) -> torch.Tensor:
    """A copy of a key cache [..., PAGE, head_dim] with every row in the plain order of d."""
    pos = _index(key_positions(k_cache.shape[-1]), k_cache)
    return torch.gather(k_cache, -1, pos.expand(k_cache.shape))


def values_in_order(v_cache: torch.Tensor) -> torch.Tensor:
    """A copy of a value cache [..., head_dim, PAGE] with every row in the plain order of slots."""
    pos = _index(value_positions(v_cache.shape[-2]), v_cache)
    return torch.gather(v_cache, -1, pos.expand(v_cache.shape))


def put_key(k_cache: torch.Tensor, page: int, slot: int, key: torch.Tensor) -> None:
    """Store ``key`` [heads, head_dim] (plain order) as the key of ``slot`` of ``page``."""
    pos = _index(key_positions(k_cache.shape[-1])[slot], k_cache)
    k_cache[page, :, slot, pos] = key.to(k_cache.dtype).to(k_cache.device)


def put_value(v_cache: torch.Tensor, page: int, slot: int, value: torch.Tensor) -> None:
    """Store ``value`` [heads, head_dim] as the value of ``slot`` of ``page``."""
    hd = v_cache.shape[-2]
    pos = _index(value_positions(hd)[:, slot], v_cache)
    v_cache[page, :, torch.arange(hd, device=v_cache.device), pos] = value.to(v_cache.dtype).to(v_cache.device)


def get_key(k_cache: torch.Tensor, page: int, slot: int) -> torch.Tensor:
    pos = _index(key_positions(k_cache.shape[-1])[slot], k_cache)
    return k_cache[page, :, slot, pos]


def get_value(v_cache: torch.Tensor, page: int, slot: int) -> torch.Tensor:
    hd = v_cache.shape[-2]
    pos = _index(value_positions(hd)[:, slot], v_cache)
    return v_cache[page, :, torch.arange(hd, device=v_cache.device), pos]
