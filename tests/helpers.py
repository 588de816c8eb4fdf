"""Shared helpers of the GPU tests: ways of cutting a request into steps, and comparisons."""
from __future__ import annotations

import functools
import random
from typing import Dict, List, Sequence

import torch

import plain_llama4 as P


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@functools.lru_cache(maxsize=64)
def _plain_cached(model_dir: str, tokens: tuple) -> torch.Tensor:
    c = P.read_config(model_dir)
    W = P.load_weights(model_dir)
    return P.forward(c, W, list(tokens))


def plain_logits(model_dir: str, tokens: Sequence[int]) -> torch.Tensor:
    return _plain_cached(model_dir, tuple(int(t) for t in tokens))


def make_engine(model_dir: str, dtype: str, kv_tokens: int = 1024, max_num_seqs: int = 8, page_size: int = 16, **kw):
    from sharpinference_amd.engine import Engine

    return Engine(model_dir, dtype=dtype, device="cuda:0", kv_tokens=kv_tokens, max_num_seqs=max_num_seqs,
                  page_size=page_size, **kw)


def run_cut(engine, rid, tokens: Sequence[int], sizes: Sequence[int]) -> torch.Tensor:
    """One request alone, cut into steps of the given sizes; logits at every position."""
    from sharpinference_amd.engine import StepEntry

    assert sum(sizes) == len(tokens)
    engine.add_request(rid)
    out, o = [], 0
    for s in sizes:
        lg = engine.step([StepEntry(rid, list(tokens[o:o + s]), list(range(s)))])
        out.append(lg.float().cpu())
        o += s
    engine.free_request(rid)
    engine.cache.check_invariants()
    return torch.cat(out, 0)


def whole(n: int) -> List[int]:
    return [n]


def last_decoded(n: int, tail: int = 32) -> List[int]:
    tail = min(tail, n - 1) if n > 1 else 0
    return ([n - tail] if n - tail > 0 else []) + [1] * tail


def changing_portions(n: int, seed: int = 0) -> List[int]:
    pattern = [7, 2, 13, 5, 2, 3, 17, 2, 11, 1, 29, 2]
    rng = random.Random(seed)
    rng.shuffle(pattern)
    out, left, i = [], n, 0
    while left > 0:
        s = min(pattern[i % len(pattern)], left)
        out.append(s)
        left -= s
        i += 1
    return out


def fp32_tol(ref: torch.Tensor) -> float:
    return 1e-4 * max(1.0, float(ref.abs().max()))


def assert_close_fp32(got: torch.Tensor, ref: torch.Tensor, what: str = "") -> None:
    err = (got.double() - ref.double()).abs()
    worst = float(err.max())
    tol = fp32_tol(ref)
    if not worst <= tol:
        row = int(err.max(dim=-1).values.argmax())
        first = int((err.max(dim=-1).values > tol).nonzero()[0])
        raise AssertionError(f"{what}: max abs diff {worst:.3e} > {tol:.1e}; worst row {row}, first wrong row {first}")


def bf16_error(got: torch.Tensor, ref: torch.Tensor) -> float:
    """Largest row-wise error relative to that row's rms."""
    err = (got.double() - ref.double())
    rms = ref.double().pow(2).mean(dim=-1).sqrt().clamp_min(1e-6)
    return float((err.abs().max(dim=-1).values / rms).max())


def assert_close_bf16(got: torch.Tensor, ref: torch.Tensor, what: str = "", tol: float = 0.06) -> None:
    e = bf16_error(got, ref)
    if not e <= tol:
        err = (got.double() - ref.double()).abs().max(dim=-1).values
        rms = ref.double().pow(2).mean(dim=-1).sqrt().clamp_min(1e-6)
        first = int(((err / rms) > tol).nonzero()[0])
        raise AssertionError(f"{what}: max |diff| / row rms = {e:.3f} > {tol}; first wrong row {first}")
