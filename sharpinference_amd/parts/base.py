"""What every part of a model has in common, and what a part sees of a step.

A *part* (norm, position encoding, mixer, feed-forward, block) takes its sizes and constants
as constructor arguments, says which tensors it needs (``param_specs``), takes them from a
source (``load``) and computes (``forward``).  No part knows which model it sits in.

A step hands the parts a :class:`StepContext`: the flat batch of tokens (several requests,
prompt portions beside single decoded tokens) with per-token positions and, for each cache
group, the block tables and the slots where this step's keys and values go.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..weights.loader import INIT_INT, INIT_NORM_WEIGHT, INIT_NORMAL, ParamSpec, TensorSource  # noqa: F401


class Part:
    """Base of all parts.  Children are parts held in attributes listed by ``children()``."""

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        return {}

    def load(self, prefix: str, source: TensorSource) -> None:
        pass

    def step_planners(self) -> Sequence["StepPlanner"]:
        """The index arrays this part wants made once a step (see :class:`StepPlanner`); none by default."""
        return ()


@dataclass
class HostStep:
    """What a step planner sees of a step, on the host: the flat batch's layout."""

    n_entries: int
    n_tokens: int
    lens: List[int]                    # tokens of each entry
    starts: List[int]                  # position of each entry's first token
    cu_tokens: np.ndarray              # int32 [entries + 1]: entry e's tokens are rows cu[e] .. cu[e + 1]


class StepPlanner:
    """Index arrays that a kind of part needs once a step, made on the host from the batch's layout
    and uploaded in the step's one copy: the step function knows nothing of what they mean.

    A part returns its planners from ``step_planners()``; planners with the same ``key`` are one
    (every attention layer shares one set of work lists).  ``plan`` returns int32 arrays and host
    facts; ``attach`` receives their device views and the facts and puts them where the part's
    ``forward`` finds them (fields of the context, or ``ctx.extras[key]``).  For a decode step that
    is replayed from a graph the arrays of a step must have the sizes of every other step of that
    batch size, and ``null`` gives contents under which a trial run touches no request's data."""

    key: str = ""

    def plan(self, host: HostStep) -> Tuple[List[np.ndarray], dict]:
        raise NotImplementedError

    def null(self, host: HostStep, arrays: List[np.ndarray]) -> List[np.ndarray]:
        return [np.zeros_like(a) for a in arrays]

    def attach(self, ctx: "StepContext", views: List[torch.Tensor], facts: dict) -> None:
        raise NotImplementedError


@dataclass
class GroupView:
    """One cache group as a step sees it."""

    block_table: torch.Tensor          # int32 [entries, max_blocks], -1 where no page
    slot_mapping: torch.Tensor         # int32 [tokens]: page * page_size + offset for this step's tokens
    page_size: int
    max_context: int = 0               # longest context (position + 1) of any token in the step


@dataclass
class StepContext:
    n_tokens: int
    n_entries: int
    token_ids: torch.Tensor            # int32 [tokens]
    positions: torch.Tensor            # int32 [tokens]
    entry_of_token: torch.Tensor       # int32 [tokens]
    cu_tokens: torch.Tensor            # int32 [entries + 1]
    state_slots: torch.Tensor          # int32 [entries]: the state slot of each entry's request (device: index
                                       # state tensors with it; a replayed graph sees each step's slots here)
    groups: List[GroupView]
    act_dtype: torch.dtype
    no_store_slots: Optional[torch.Tensor] = None   # int32 [tokens] of -1: "store nothing" for cache readers
    # how attention kernels split the batch: entries of one token, and tiles of the others' tokens
    # (made by the attention parts' planner, parts/attention.py; empty in a model without attention)
    n_decode: int = 0
    decode_tokens: Optional[torch.Tensor] = None    # int32 [n_decode] token indices; None = every token
    n_prefill_tiles: int = 0
    prefill_tiles: Optional[torch.Tensor] = None    # int32 [tiles, 3]: (entry, first token, rows)
    prefill_tile_tokens: int = 128                  # the most rows of a tile (128, or 64 for short prompts)
    # host copies for parts that plan launches
    entry_lens: List[int] = field(default_factory=list)
    entry_starts: List[int] = field(default_factory=list)
    max_entry_len: int = 1
    extras: Dict[str, object] = field(default_factory=dict)


@dataclass
class LayerCache:
    """The cache of one execution of one layer."""

    group: Optional[GroupView] = None
    k: Optional[torch.Tensor] = None   # [pages, kv heads, page_size, head_dim]
    v: Optional[torch.Tensor] = None
    state: Optional[torch.Tensor] = None   # [state slots, ...]
    write: bool = True                 # False: read another layer's cache, store nothing


class ResidualStream:
    """The float32 residual sum ``h`` and the branch output still to be added to it.

    A branch (mixer, feed-forward) leaves its output in ``pending``; the next norm adds it into
    ``h`` in the same kernel that normalises, so the sum is formed once, in float.  ``pending``
    is a tensor [T, H] or an object with ``shape``, ``dtype`` and ``tensor()`` that stands for one
    (``ops.ExpertSum``); a norm that cannot fold such an object in calls ``pending_tensor()``."""

    def __init__(self, h: torch.Tensor):
        self.h = h
        self.pending = None

    def pending_tensor(self) -> Optional[torch.Tensor]:
        p = self.pending
        return p if p is None or isinstance(p, torch.Tensor) else p.tensor()
