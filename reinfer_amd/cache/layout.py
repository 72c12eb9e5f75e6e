"""How keys and values lie inside a cache block on the device.

A block holds ``block_size`` slots (a multiple of 16) of every KV head. The
slab of one (block, KV head) is ``block_size / 16`` tiles of 16 slots times
``head_dim`` elements, and a tile is laid out in the order the matrix cores
take their operands, so that a wave's load of it is one contiguous run:

    K tile  [head_dim / 8][16 slots][8]     element (slot, e) at ((e // 8) * 16 + slot) * 8 + e % 8
    V tile  [head_dim / 16][4][16][4]       element (slot, e) at (((e // 16) * 4 + slot // 4) * 16 + e % 16) * 4 + slot % 4

The kernels index with the same formulas (``cache_k_index`` / ``cache_v_index``
in csrc/common.h). The device tensors have shape
``[blocks, kv_heads, block_size // 16, 16 * head_dim]``; the functions here turn
a plain ``[..., block_size, head_dim]`` view into that order and back (tests,
debugging; the engine itself never converts).
"""
from __future__ import annotations

from typing import Tuple

import torch

TILE = 16


def check_geometry(block_size: int, head_dim: int) -> None:
    if block_size <= 0 or block_size % TILE != 0:
        raise ValueError(f"block_size {block_size}: the cache is tiled by {TILE} slots; use a multiple of {TILE}")
    if head_dim <= 0 or head_dim % TILE != 0:
        raise ValueError(f"head size {head_dim}: the cache is tiled by {TILE} elements; head sizes go in steps of {TILE}")


def cache_shape(num_blocks: int, num_kv_heads: int, block_size: int, head_dim: int) -> Tuple[int, int, int, int]:
    check_geometry(block_size, head_dim)
    return (num_blocks, num_kv_heads, block_size // TILE, TILE * head_dim)


def pack_k(x: torch.Tensor) -> torch.Tensor:
    """[..., block_size, d] -> [..., block_size // 16, 16 * d] in K tile order."""
    *lead, bs, d = x.shape
    check_geometry(bs, d)
    v = x.reshape(*lead, bs // TILE, TILE, d // 8, 8)            # tile, slot, chunk, j
    n = len(lead)
    v = v.permute(*range(n), n, n + 2, n + 1, n + 3)             # tile, chunk, slot, j
    return v.reshape(*lead, bs // TILE, TILE * d).contiguous()


def unpack_k(x: torch.Tensor, head_dim: int) -> torch.Tensor:
    """Inverse of :func:`pack_k`: -> [..., block_size, d]."""
    *lead, nt, td = x.shape
    d = head_dim
    v = x.reshape(*lead, nt, d // 8, TILE, 8)
    n = len(lead)
    v = v.permute(*range(n), n, n + 2, n + 1, n + 3)
    return v.reshape(*lead, nt * TILE, d).contiguous()


def pack_v(x: torch.Tensor) -> torch.Tensor:
    """[..., block_size, d] -> [..., block_size // 16, 16 * d] in V tile order."""
    *lead, bs, d = x.shape
    check_geometry(bs, d)
    v = x.reshape(*lead, bs // TILE, 4, 4, d // TILE, TILE)      # tile, slot group, slot in group, row tile, row
    n = len(lead)
    v = v.permute(*range(n), n, n + 3, n + 1, n + 4, n + 2)      # tile, row tile, slot group, row, slot in group
    return v.reshape(*lead, bs // TILE, TILE * d).contiguous()


def unpack_v(x: torch.Tensor, head_dim: int) -> torch.Tensor:
    """Inverse of :func:`pack_v`: -> [..., block_size, d]."""
    *lead, nt, td = x.shape
    d = head_dim
    v = x.reshape(*lead, nt, d // TILE, 4, TILE, 4)              # tile, row tile, slot group, row, slot in group
    n = len(lead)
    v = v.permute(*range(n), n, n + 2, n + 4, n + 1, n + 3)      # tile, slot group, slot in group, row tile, row
    return v.reshape(*lead, nt * TILE, d).contiguous()
