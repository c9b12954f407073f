"""The order in which a cache page keeps its 64 tokens of one key/value head.

Both orders are those in which the attention kernels read: a wave's 64 lanes
load 16 bytes each from consecutive memory.

    keys    [chunk of 8 channels][token][8 channels]
    values  [tile of 16 channels][half of 32 tokens][group of 8 tokens][channel of the tile][8 tokens]

A head size that is no multiple of 8 (16) leaves the last chunk (tile) partly
unused.  The kernels hold the same formulas (``nnis_k_offset`` and
``nnis_v_offset`` in ``csrc/common.h``).
"""

from __future__ import annotations

from typing import Tuple

from .allocator import PAGE_TOKENS


def k_page_shape(kv_heads: int, head_dim: int) -> Tuple[int, ...]:
    return (kv_heads, (head_dim + 7) // 8, PAGE_TOKENS, 8)


def v_page_shape(kv_heads: int, head_dim: int) -> Tuple[int, ...]:
    return (kv_heads, (head_dim + 15) // 16, 2, 4, 16, 8)


def k_offset(token: int, channel: int) -> int:
    """Element offset of a token's key channel within its head's part of a page."""
    return (channel // 8) * (PAGE_TOKENS * 8) + token * 8 + channel % 8


def v_offset(channel: int, token: int) -> int:
    return ((((channel // 16) * 2 + token // 32) * 4 + (token % 32) // 8) * 16 + channel % 16) * 8 + token % 8
