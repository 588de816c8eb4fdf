"""The attention mixer: grouped-query attention over the paged cache."""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..ops.lib import PREFILL_TILE_TOKENS
from ..ops.profile import section
from ..cache.spec import KVSpec, WINDOW_CHUNK, WINDOW_NONE, WINDOW_SLIDING  # noqa: F401
from .base import HostStep, LayerCache, ParamSpec, Part, StepContext, StepPlanner, TensorSource

SHORT_PROMPT_TOKENS = 1536   # up to so many prompt tokens in a step, tiles of half as many tokens (measured:
                             # 20-25 % less attention time from 512 to 1,536 tokens, 6 % more at 2,048)


class AttentionWorkLists(StepPlanner):
    """How the attention kernels split a batch: the tokens of entries of one token (the split-K
    decode kernel's list; none when every token is one, the kernel then takes them all) and the
    tiles of the longer entries (entry, first token, rows) for the flash kernel.  A step with few
    prompt tokens is cut into tiles of half the rows: its attention launch lasts as long as its
    longest tile, and twice the blocks of half the rows walk their keys faster."""

    key = "attention"

    def plan(self, host: HostStep) -> Tuple[List[np.ndarray], dict]:
        lens, cu = host.lens, host.cu_tokens
        dec = [int(cu[i]) for i in range(host.n_entries) if lens[i] == 1]
        tile = PREFILL_TILE_TOKENS if sum(n for n in lens if n > 1) > SHORT_PROMPT_TOKENS else PREFILL_TILE_TOKENS // 2
        tiles = [(i, int(cu[i]) + o, min(tile, lens[i] - o)) for i in range(host.n_entries) if lens[i] > 1
                 for o in range(0, lens[i], tile)]
        arrays = [np.asarray(dec, dtype=np.int32), np.asarray(tiles, dtype=np.int32).reshape(-1)]
        return arrays, dict(n_dec=len(dec), n_tiles=len(tiles), tile=tile, all_decode=len(dec) == host.n_tokens)

    def null(self, host: HostStep, arrays: List[np.ndarray]) -> List[np.ndarray]:
        return [np.arange(arrays[0].size, dtype=np.int32), np.zeros_like(arrays[1])]

    def attach(self, ctx: StepContext, views: List[torch.Tensor], facts: dict) -> None:
        ctx.n_decode = facts["n_dec"]
        ctx.decode_tokens = None if facts["all_decode"] else views[0]
        ctx.n_prefill_tiles = facts["n_tiles"]
        ctx.prefill_tiles = views[1].view(-1, 3) if facts["n_tiles"] else None
        ctx.prefill_tile_tokens = facts["tile"]


_WORK_LISTS = AttentionWorkLists()


class Attention(Part):
    """q/k/v projections (with biases if ``bias``) -> position encoding -> optional weightless per-head norm
    -> optional query temperature -> keys and values into the cache -> softmax(q k^T * scale) v
    over the keys the window admits -> output projection
    (reference: src/SharpInference.Engine/ForwardPass.cs:1576-1690, 1838-1912; the norm comes
    after the rotation, 1643-1648; optional biases are added right after their products,
    1605-1613, the output projection's may be absent on its own, 381-383).

    Everything that differs between layers is an argument: ``rotary`` (None = no position
    encoding; otherwise any object with ``table(device)``, ``pair_layout``, ``rotary_dim`` and
    ``head_dim``, see parts/position.py), ``v_head_dim`` (values and a head's output of another width than
    keys: such layers run the float attention kernel), ``qk_norm_eps`` (None = no norm), ``q_temperature`` = (floor_scale, attn_scale)
    multiplying queries by 1 + attn_scale * ln(floor((pos + 1) / floor_scale) + 1), and the
    window: all keys, the chunk [floor(pos/W)*W, pos], or the last W keys."""

    def __init__(self, hidden: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 rotary=None, qk_norm_eps: Optional[float] = None,
                 q_temperature: Optional[Tuple[float, float]] = None, window_kind: int = WINDOW_NONE,
                 window: int = 0, scale: Optional[float] = None, bias: bool = False, o_bias: Optional[bool] = None,
                 v_head_dim: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads cannot share {num_kv_heads} kv heads")
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError(f"head_dim {head_dim} is not taken: multiples of 16 from 16 to 256")
        if rotary is not None and rotary.head_dim != head_dim:
            raise ValueError("the rotary table's head_dim differs from the mixer's")
        if rotary is not None and rotary.pair_layout not in ("interleaved", "half"):
            raise ValueError(f"pair layout {rotary.pair_layout!r} is not taken by the rotation kernel")
        self.hidden, self.nh, self.nkv, self.hd = int(hidden), int(num_heads), int(num_kv_heads), int(head_dim)
        self.vd = int(v_head_dim or head_dim)                    # width of a value (and of a head's output)
        if not 1 <= self.vd <= 256:
            raise ValueError(f"v_head_dim {self.vd} is not taken: 1 to 256")
        self.rotary, self.qk_norm_eps, self.q_temperature = rotary, qk_norm_eps, q_temperature
        self.window_kind, self.window = int(window_kind), int(window)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.bias = bool(bias)                                   # q, k and v carry biases
        self.o_bias = self.bias if o_bias is None else bool(o_bias)   # the output projection carries one
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None                # float32 [q + 2 kv]: added by the rotation kernel
        self.b_o: Optional[torch.Tensor] = None                  # float32 [hidden]

    # -- what it needs --------------------------------------------------------
    def step_planners(self):
        return (_WORK_LISTS,)

    def cache_spec(self) -> KVSpec:
        return KVSpec(self.nkv, self.hd, self.window_kind, self.window, 0 if self.vd == self.hd else self.vd)

    def param_specs(self, prefix: str) -> Dict[str, ParamSpec]:
        q, kv, vv, ov = self.nh * self.hd, self.nkv * self.hd, self.nkv * self.vd, self.nh * self.vd
        specs = {
            prefix + "q_proj.weight": ParamSpec((q, self.hidden)),
            prefix + "k_proj.weight": ParamSpec((kv, self.hidden)),
            prefix + "v_proj.weight": ParamSpec((vv, self.hidden)),
            prefix + "o_proj.weight": ParamSpec((self.hidden, ov)),
        }
        if self.bias:
            specs.update({prefix + "q_proj.bias": ParamSpec((q,)), prefix + "k_proj.bias": ParamSpec((kv,)),
                          prefix + "v_proj.bias": ParamSpec((vv,))})
        if self.o_bias:
            specs[prefix + "o_proj.bias"] = ParamSpec((self.hidden,))
        return specs

    def load(self, prefix: str, source: TensorSource) -> None:
        q, kv, vv = self.nh * self.hd, self.nkv * self.hd, self.nkv * self.vd
        parts = [source.get(prefix + n + "_proj.weight") for n in ("q", "k", "v")]
        dt = torch.float32 if any(p.dtype == torch.float32 for p in parts) else parts[0].dtype
        fused = torch.empty(q + kv + vv, self.hidden, dtype=dt, device=parts[0].device)
        o = 0
        for p in parts:
            fused[o:o + p.shape[0]].copy_(p)
            o += p.shape[0]
        # both also in the order the few-rows kernel streams them; the rows stay for prompt-sized steps
        self.w_qkv = ops.pack_weight(fused)
        self.w_o = ops.pack_weight(source.get(prefix + "o_proj.weight"))
        if self.bias:
            self.b_qkv = torch.cat([source.get(prefix + n + "_proj.bias").float() for n in ("q", "k", "v")]).contiguous()
        if self.o_bias:
            self.b_o = source.get(prefix + "o_proj.bias").float().contiguous()

    # -- compute --------------------------------------------------------------
    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> torch.Tensor:
        g = cache.group
        T = x.shape[0]
        width = 2 if ctx.act_dtype == torch.bfloat16 else 4
        q_dim, kv_dim = self.nh * self.hd, self.nkv * (self.hd + self.vd) // 2    # (kv_dim: the mean of a key's and a value's row)
        with section("qkv", nbytes=width * (q_dim + 2 * kv_dim) * (self.hidden + T) + width * T * self.hidden,
                     flops=2.0 * T * self.hidden * (q_dim + 2 * kv_dim)):
            qkv = ops.linear(x, self.w_qkv, ctx.act_dtype)
        slots = g.slot_mapping if cache.write else ctx.no_store_slots
        inv_freq = self.rotary.table(x.device) if self.rotary is not None else None
        layout = ops.PAIRS_HALF_SPLIT if self.rotary is not None and self.rotary.pair_layout == "half" else ops.PAIRS_INTERLEAVED
        with section("rope + cache write", nbytes=2 * width * T * (q_dim + 2 * kv_dim)):
            q = ops.rope_kv(qkv, cache.k, cache.v, slots, ctx.positions, inv_freq, self.qk_norm_eps is not None,
                            self.qk_norm_eps or 1e-6, self.q_temperature, self.nh, self.nkv, self.hd, layout,
                            bias=self.b_qkv, vd=self.vd)
        with section("attention", nbytes=lambda: self._keys_held(ctx) * 2 * kv_dim * width + 2 * T * q_dim * width,
                     flops=lambda: 4.0 * self._keys_read(ctx) * q_dim):
            o = ops.attention(q, cache.k, cache.v, g, ctx, self.window_kind, self.window, self.scale, self.nh, self.nkv,
                              self.hd, self.vd)
        with section("o", nbytes=width * self.hidden * (q_dim + T) + width * T * q_dim, flops=2.0 * T * self.hidden * q_dim):
            out = ops.linear(o, self.w_o, ctx.act_dtype)
            return ops.add_bias(out, self.b_o) if self.b_o is not None else out

    def _keys_read(self, ctx: StepContext) -> int:
        """(query, key) pairs of the step: what is computed."""
        spec = self.cache_spec()
        return sum(p - spec.first_visible(p) + 1 for s, n in zip(ctx.entry_starts, ctx.entry_lens) for p in range(s, s + n))

    def _keys_held(self, ctx: StepContext) -> int:
        """Keys that some query of the step sees, each counted once per entry: what has to be read."""
        spec = self.cache_spec()
        return sum(s + n - spec.first_visible(s) for s, n in zip(ctx.entry_starts, ctx.entry_lens))
