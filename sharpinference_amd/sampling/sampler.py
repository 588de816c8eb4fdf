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
    n = params.penalty_last_n
    if n > 0 and len(generated) >= n:
        return list(generated[-n:])
    if not params.penalty_seed_from_prompt:
        return list(generated)
    if n <= 0:
        return list(prompt) + list(generated)
    return list(prompt[len(prompt) - min(len(prompt), n - len(generated)):]) + list(generated)


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
        n = len(ps)
        # temperature, uniform, top-p and min-p of the rows in one copy, top-k in another
        f = torch.tensor([[p.temperature for p in ps], [uniform(p.seed, draw_index[r]) for p, r in zip(ps, rows)],
                          [p.top_p for p in ps], [p.min_p for p in ps]], dtype=torch.float32).to(dev)
        top_k = torch.tensor([p.top_k for p in ps], dtype=torch.int32).to(dev) if any(p.top_k > 0 for p in ps) else None
        top_p = f[2] if any(0 < p.top_p < 1 for p in ps) else None
        min_p = f[3] if any(p.min_p > 0 for p in ps) else None
        assert f.shape == (4, n)
        ids = ops.sample_rows(sub, f[0], f[1], top_k, top_p, min_p).cpu().tolist()
        for r, t in zip(rows, ids):
            out[r] = t
        return out

    def _edit(self, logits: torch.Tensor, ps: Sequence[SamplingParams], hists, vocab: int) -> None:
        """The rows' sparse edits (distinct tokens of the window with their counts, biased tokens), laid
        out on the host as one integer and one float array: two copies to the device, one launch."""
        R = len(ps)
        if not any(p.logit_bias for p in ps):
            # penalties only (the usual case): the distinct (row, token) pairs of all windows in one sort
            wins = [(r, np.asarray(h, dtype=np.int64)) for r, (p, h) in enumerate(zip(ps, hists))
                    if p.has_penalties and len(h)]
            if all(int(w.min()) >= 0 and int(w.max()) < vocab for _, w in wins):   # (else the careful path drops them)
                flat = np.concatenate([w + r * vocab for r, w in wins]) if wins else np.empty(0, np.int64)
                uniq, cnt = np.unique(flat, return_counts=True)           # ascending by row, then by token
                n = uniq.shape[0]
                ints = np.empty(R + 1 + 2 * n, np.int32)
                ints[0] = 0
                np.cumsum(np.bincount(uniq // vocab, minlength=R)[:R], out=ints[1:R + 1])
                ints[R + 1:R + 1 + n] = uniq % vocab
                ints[R + 1 + n:] = cnt
                flts = np.zeros(n + 3 * R, np.float32)
                flts[n:n + R] = [p.repetition_penalty for p in ps]
                flts[n + R:n + 2 * R] = [p.frequency_penalty for p in ps]
                flts[n + 2 * R:] = [p.presence_penalty for p in ps]
                di = torch.from_numpy(ints).to(self.device)
                df = torch.from_numpy(flts).to(self.device)
                ops.edit_logits(logits, di[:R + 1], di[R + 1:R + 1 + n], di[R + 1 + n:], df[:n], df[n:n + R],
                                df[n + R:n + 2 * R], df[n + 2 * R:])
                return
        row_ids, row_counts, row_bias = [], [], []
        for p, h in zip(ps, hists):
            if p.has_penalties and len(h):
                ids, cnt = np.unique(np.asarray(h, dtype=np.int64), return_counts=True)   # ascending ids
            else:
                ids, cnt = np.empty(0, np.int64), np.empty(0, np.int64)
            b = np.zeros(ids.shape[0], np.float32)
            if p.logit_bias:
                extra = np.asarray(sorted(int(t) for t in p.logit_bias if int(t) not in set(ids.tolist())), dtype=np.int64)
                ids = np.concatenate([ids, extra])
                cnt = np.concatenate([cnt, np.zeros(extra.shape[0], np.int64)])
                order = np.argsort(ids, kind="stable")
                ids, cnt = ids[order], cnt[order]
                b = np.asarray([float(p.logit_bias.get(int(t), 0.0)) for t in ids], dtype=np.float32)
            ok = (ids >= 0) & (ids < vocab)
            row_ids.append(ids[ok]); row_counts.append(cnt[ok]); row_bias.append(b[ok])
        lens = [a.shape[0] for a in row_ids]
        n = int(sum(lens))
        ints = np.empty(R + 1 + 2 * n, np.int32)
        ints[0] = 0
        np.cumsum(lens, out=ints[1:R + 1])
        ints[R + 1:R + 1 + n] = np.concatenate(row_ids) if n else 0
        ints[R + 1 + n:] = np.concatenate(row_counts) if n else 0
        flts = np.empty(n + 3 * R, np.float32)
        flts[:n] = np.concatenate(row_bias) if n else 0
        flts[n:n + R] = [p.repetition_penalty for p in ps]
        flts[n + R:n + 2 * R] = [p.frequency_penalty for p in ps]
        flts[n + 2 * R:] = [p.presence_penalty for p in ps]
        di = torch.from_numpy(ints).to(self.device)
        df = torch.from_numpy(flts).to(self.device)
        ops.edit_logits(logits, di[:R + 1], di[R + 1:R + 1 + n], di[R + 1 + n:], df[:n], df[n:n + R],
                        df[n + R:n + 2 * R], df[n + 2 * R:])


def _gather_rows(logits: torch.Tensor, rows: Sequence[int]) -> torch.Tensor:
    out = torch.empty(len(rows), logits.shape[1], dtype=logits.dtype, device=logits.device)
    for i, r in enumerate(rows):
        out[i].copy_(logits[r])
    return out
