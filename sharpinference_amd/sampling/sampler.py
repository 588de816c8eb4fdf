"""Token selection for a batch of logit rows, on the device.

Greedy rows take the argmax (lowest index among equal maxima, as the reference's scan,
reference: src/SharpInference.Engine/Sampler.cs:436-449).  Other rows follow the reference's
full-vocabulary order (Sampler.cs:45-106): logit bias, then the window penalties, then
logits / temperature -> softmax -> top-k -> min-p -> top-p -> renormalise -> the first index
whose running sum reaches the request's next uniform (Sampler.cs:564-576).  Greedy rows skip
bias and penalties, as the reference's early return does (Sampler.cs:17-18).

Uniforms come from a counter-based generator on the host, one stream per request keyed by its
seed, so a request's tokens do not depend on what else is in the batch: draw i of seed s is
mix(s * 0x9E3779B97F4A7C15 + (i + 1) * 0xBF58476D1CE4E5B9) >> 40, scaled by 2^-24, where mix
is the splitmix64 finaliser.  (The reference draws from .NET's Random, one per request,
src/SharpInference.Engine/ContinuousBatchingEngine.cs:732.)
"""
from __future__ import annotations

from collections import Counter
from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .params import SamplingParams

_M64 = (1 << 64) - 1


def uniform(seed: int, index: int) -> float:
    """Draw `index` (0-based) of the stream of `seed`: a multiple of 2^-24 in [0, 1)."""
    z = ((seed & _M64) * 0x9E3779B97F4A7C15 + (index + 1) * 0xBF58476D1CE4E5B9) & _M64
    z ^= z >> 30
    z = (z * 0xBF58476D1CE4E5B9) & _M64
    z ^= z >> 27
    z = (z * 0x94D049BB133111EB) & _M64
    z ^= z >> 31
    return (z >> 40) / float(1 << 24)


def penalty_window(params: SamplingParams, prompt: Sequence[int], generated: Sequence[int]) -> List[int]:
    """The tokens the penalties look at (reference: src/SharpInference.Engine/PenaltyWindow.cs;
    Sampler.cs:690-741)."""
    hist = (list(prompt) if params.penalty_seed_from_prompt else []) + list(generated)
    n = params.penalty_last_n
    return hist[-n:] if n > 0 else hist


class Sampler:
    def __init__(self, device):
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, params: Sequence[SamplingParams], draw_index: Sequence[int],
               histories: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """One token per row of float32 logits [rows, vocab].  ``draw_index[r]`` says how many
        uniforms row r's request has used; ``histories[r]`` is its penalty window."""
        R, V = logits.shape
        assert len(params) == R and len(draw_index) == R
        greedy_rows = [r for r in range(R) if params[r].greedy]
        out = [0] * R
        if greedy_rows:
            host = ops.argmax_rows(logits).cpu().tolist()
            for r in greedy_rows:
                out[r] = host[r]
            if len(greedy_rows) == R:
                return out
        rows = [r for r in range(R) if not params[r].greedy]
        sub = logits if len(rows) == R else _gather_rows(logits, rows)
        ps = [params[r] for r in rows]
        if any(p.edits_logits for p in ps):
            if sub is logits:
                sub = ops.cast(logits, torch.float32)   # a copy: the caller's logits stay as they are
            self._edit(sub, ps, [histories[r] if histories is not None else () for r in rows], V)
        dev = self.device
        temp = torch.tensor([p.temperature for p in ps], dtype=torch.float32, device=dev)
        u = torch.tensor([uniform(p.seed, draw_index[r]) for p, r in zip(ps, rows)], dtype=torch.float32, device=dev)
        top_k = torch.tensor([p.top_k for p in ps], dtype=torch.int32, device=dev) if any(p.top_k > 0 for p in ps) else None
        top_p = torch.tensor([p.top_p for p in ps], dtype=torch.float32, device=dev) if any(0 < p.top_p < 1 for p in ps) else None
        min_p = torch.tensor([p.min_p for p in ps], dtype=torch.float32, device=dev) if any(p.min_p > 0 for p in ps) else None
        ids = ops.sample_rows(sub, temp, u, top_k, top_p, min_p).cpu().tolist()
        for r, t in zip(rows, ids):
            out[r] = t
        return out

    def _edit(self, logits: torch.Tensor, ps: Sequence[SamplingParams], hists, vocab: int) -> None:
        offs, ids, counts, bias = [0], [], [], []
        for p, h in zip(ps, hists):
            cnt = Counter(int(t) for t in h) if p.has_penalties else Counter()
            b = dict(p.logit_bias or {})
            for t in sorted(set(cnt) | set(b)):
                if 0 <= t < vocab:
                    ids.append(t)
                    counts.append(cnt.get(t, 0))
                    bias.append(float(b.get(t, 0.0)))
            offs.append(len(ids))
        dev = self.device
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)  # noqa: E731
        f32 = lambda x: torch.tensor(x, dtype=torch.float32, device=dev)  # noqa: E731
        ops.edit_logits(logits, i32(offs), i32(ids), i32(counts), f32(bias),
                        f32([p.repetition_penalty for p in ps]), f32([p.frequency_penalty for p in ps]),
                        f32([p.presence_penalty for p in ps]))


def _gather_rows(logits: torch.Tensor, rows: Sequence[int]) -> torch.Tensor:
    out = torch.empty(len(rows), logits.shape[1], dtype=logits.dtype, device=logits.device)
    for i, r in enumerate(rows):
        out[i].copy_(logits[r])
    return out
