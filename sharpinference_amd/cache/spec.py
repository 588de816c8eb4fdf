"""What a mixer asks of the cache manager.

Two kinds of per-request memory exist.  ``KVSpec``: keys and values that grow with the
sequence, kept in pages; a window tells which of them a later query can still see, so that
pages behind it go back to the pool.  ``StateSpec``: a block of fixed size per request (a
recurrent state, a convolution tail), kept in a slot
(reference: src/SharpInference.Engine/GdnStateCache.cs:7-33 for the fixed-size kind,
src/SharpInference.Engine/PagedKvCache.cs:20-110 for the paged kind).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

import torch

WINDOW_NONE, WINDOW_CHUNK, WINDOW_SLIDING = 0, 1, 2


@dataclass(frozen=True)
class KVSpec:
    """Paged keys and values of one layer.  ``head_dim`` is the width of a key; ``v_head_dim`` the
    width of a value where it differs (0: the same).  Keys are kept [page, kv head, position,
    head_dim], values transposed inside the page, [page, kv head, v_head_dim, position]."""

    num_kv_heads: int
    head_dim: int
    window_kind: int = WINDOW_NONE
    window: int = 0
    v_head_dim: int = 0

    @property
    def value_dim(self) -> int:
        return self.v_head_dim or self.head_dim

    def first_visible(self, pos: int) -> int:
        """The earliest key position a query at `pos` can see."""
        if self.window_kind == WINDOW_CHUNK:
            return (pos // self.window) * self.window
        if self.window_kind == WINDOW_SLIDING:
            return max(0, pos - self.window + 1)
        return 0

    def group_key(self):
        # layers whose pages live and die together share a block table
        return ("kv", self.window_kind, self.window)


@dataclass(frozen=True)
class StateSpec:
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32

    def group_key(self):
        return ("state",)
