"""Shared helpers of the GPU tests: ways of cutting a request into steps, and comparisons."""
from __future__ import annotations

import functools
import random
from typing import Dict, List, Sequence

import torch

import plain_llama4 as P

# A bfloat16 run may pick another expert than 32-bit arithmetic where two router logits are
# closer than rounding; its pick must still lie within this of the best (relative to the rms of
# the token's router logits).
ROUTE_REGRET = 0.02


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@functools.lru_cache(maxsize=128)
def _plain_cached(model_dir: str, tokens: tuple, bf16_storage: bool) -> torch.Tensor:
    c = P.read_config(model_dir)
    W = P.load_weights(model_dir)
    return P.forward(c, W, list(tokens), store=P.store_bf16 if bf16_storage else P._same)


def plain_logits(model_dir: str, tokens: Sequence[int], bf16_storage: bool = False) -> torch.Tensor:
    """Whole-sequence logits of the plain implementation; with bf16_storage, tensors are rounded
    where the engine's bfloat16 path stores them (the arithmetic stays float)."""
    return _plain_cached(model_dir, tuple(int(t) for t in tokens), bool(bf16_storage))


def moe_layers_of(model_dir: str) -> List[int]:
    c = P.read_config(model_dir)
    return [l for l in range(int(c["num_hidden_layers"])) if P.layer_is_moe(c, l)]


def plain_logits_routed(model_dir: str, tokens: Sequence[int], routes: Dict[int, torch.Tensor]):
    """The plain implementation with bfloat16 storage and the engine's own expert picks.
    Returns (logits, regret): regret is how far the worst forced pick lies below the plain
    implementation's own, relative to the rms of that token's router logits."""
    c = P.read_config(model_dir)
    W = P.load_weights(model_dir)
    trace: dict = {}
    lg = P.forward(c, W, list(tokens), store=P.store_bf16, routes=routes, trace=trace)
    return lg, trace.get("route_regret", 0.0)


def make_engine(model_dir: str, dtype: str, kv_tokens: int = 1024, max_num_seqs: int = 8, page_size: int = 16, **kw):
    from sharpinference_amd.engine import Engine

    return Engine(model_dir, dtype=dtype, device="cuda:0", kv_tokens=kv_tokens, max_num_seqs=max_num_seqs,
                  page_size=page_size, **kw)


def run_cut(engine, rid, tokens: Sequence[int], sizes: Sequence[int], with_routes: bool = False):
    """One request alone, cut into steps of the given sizes; logits at every position (and,
    if asked, the expert picks {layer: ids [T, k]} the engine made)."""
    from sharpinference_amd.engine import StepEntry

    assert sum(sizes) == len(tokens)
    engine.add_request(rid)
    out, o = [], 0
    picks: List[List[torch.Tensor]] = []
    for s in sizes:
        trace: list = []
        lg = engine.step([StepEntry(rid, list(tokens[o:o + s]), list(range(s)))], router_trace=trace)
        out.append(lg.float().cpu())
        picks.append([ids.cpu() for ids, _ in trace])
        o += s
    engine.free_request(rid)
    engine.cache.check_invariants()
    logits = torch.cat(out, 0)
    if not with_routes:
        return logits
    n_moe = len(picks[0])
    return logits, [torch.cat([p[i] for p in picks], 0) for i in range(n_moe)]


def check_against_plain(engine, model_dir: str, dtype: str, rid, tokens: Sequence[int], sizes: Sequence[int],
                        what: str) -> torch.Tensor:
    """Run one request cut into `sizes` and compare every position's logits with the plain
    implementation: 32-bit against pure 32-bit arithmetic; bfloat16 against the plain
    implementation with bfloat16 storage and the engine's own expert picks, which must be
    picks the plain implementation could have made itself (regret within rounding)."""
    if dtype == "float32":
        got = run_cut(engine, rid, tokens, sizes)
        assert_close_fp32(got, plain_logits(model_dir, tokens), what)
        return got
    got, picks = run_cut(engine, rid, tokens, sizes, with_routes=True)
    routes = dict(zip(moe_layers_of(model_dir), picks))
    ref, regret = plain_logits_routed(model_dir, tokens, routes)
    assert regret <= ROUTE_REGRET, f"{what}: the engine picked an expert {regret:.3f} (relative) below the best"
    assert_close_bf16(got, ref, what)
    return got


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


def assert_close_bf16(got: torch.Tensor, ref: torch.Tensor, what: str = "", tol_max: float = 0.05,
                      tol_rms: float = 0.02) -> None:
    """Per row: largest error and rms error, both relative to the row's rms.  Storage rounding
    that falls the other way on single elements gives a few per cent at most; a wrong key, page
    or mask gives errors of the order of the logits themselves."""
    err = got.double() - ref.double()
    rms = ref.double().pow(2).mean(dim=-1).sqrt().clamp_min(1e-6)
    e_max = err.abs().max(dim=-1).values / rms
    e_rms = err.pow(2).mean(dim=-1).sqrt() / rms
    bad = (e_max > tol_max) | (e_rms > tol_rms)
    if bool(bad.any()):
        first = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: max |diff| / row rms = {float(e_max.max()):.3f} (tol {tol_max}), "
                             f"rms diff / row rms = {float(e_rms.max()):.3f} (tol {tol_rms}); first wrong row {first}")
