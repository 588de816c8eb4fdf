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


def assert_route_regret(regret: float, what: str) -> None:
    assert regret <= ROUTE_REGRET, f"{what}: the engine picked an expert {regret:.3f} (relative) below the best"


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
        picks.append([ids.cpu() for ids, _, _ in trace])
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
    assert_route_regret(regret, what)
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


# ---------------------------------------------------------------------------
# traces: the same requests replayed step by step, several live at a time
# ---------------------------------------------------------------------------
def mixed_trace(requests: Dict[str, Sequence[int]], seed: int, max_live: int = 4, tail: int = 32) -> List[dict]:
    """Steps in the format of bin/trace_run.  Up to `max_live` requests are live; each reads its
    prompt in portions of changing size (down to two tokens) and its last `tail` tokens one by
    one; a live request is sometimes left out of a step; logits are wanted everywhere."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}              # id -> tokens done
    steps: List[dict] = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, end = [], []
        for rid in list(live):
            toks = requests[rid]
            done = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                               # sits this step out
            left = len(toks) - done
            if left <= tail:
                take = 1
            else:
                take = min(left - tail, rng.choice([2, 2, 3, 5, 7, 13, 21]))
            entries.append({"id": rid, "tokens": list(toks[done:done + take]), "want": list(range(take))})
            live[rid] = done + take
            if live[rid] == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def tokens_held(steps: List[dict], round_to: int = 64) -> int:
    """The most tokens that live requests hold at any time, each rounded up to `round_to`."""
    held: Dict[str, int] = {}
    worst = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum((n + round_to - 1) // round_to * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return worst


def replay(engine, steps: List[dict], with_routes: bool = False):
    """Feed a trace through the engine's step function.  Returns {id: logits [len, vocab]} for
    the wanted places in order (and {id: [ids per routed layer]} if asked)."""
    from sharpinference_amd.engine import StepEntry

    logits: Dict[str, List[torch.Tensor]] = {}
    picks: Dict[str, List[List[torch.Tensor]]] = {}
    live = set()
    for st in steps:
        entries = []
        for e in st["entries"]:
            if e["id"] not in live:
                engine.add_request(e["id"])
                live.add(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        trace: list = []
        lg = engine.step(entries, router_trace=trace if with_routes else None)
        lg = lg.float().cpu() if lg is not None else None
        row, tok = 0, 0
        for e in st["entries"]:
            n = len(e["want"])
            if n:
                logits.setdefault(e["id"], []).append(lg[row:row + n])
                row += n
            if with_routes:
                picks.setdefault(e["id"], []).append([ids[tok:tok + len(e["tokens"])].cpu() for ids, _, _ in trace])
            tok += len(e["tokens"])
        for rid in st["end"]:
            engine.free_request(rid)
            live.discard(rid)
        engine.cache.check_invariants()
    out = {rid: torch.cat(v, 0) for rid, v in logits.items()}
    if not with_routes:
        return out
    routes = {}
    for rid, per_step in picks.items():
        n_moe = len(per_step[0])
        routes[rid] = [torch.cat([p[i] for p in per_step], 0) for i in range(n_moe)]
    return out, routes


def check_trace_against_plain(engine, model_dir: str, dtype: str, requests: Dict[str, Sequence[int]],
                              steps: List[dict], what: str) -> None:
    if dtype == "float32":
        got = replay(engine, steps)
        for rid, toks in requests.items():
            assert_close_fp32(got[rid], plain_logits(model_dir, toks), f"{what} request {rid}")
        return
    got, picks = replay(engine, steps, with_routes=True)
    layers = moe_layers_of(model_dir)
    for rid, toks in requests.items():
        ref, regret = plain_logits_routed(model_dir, toks, dict(zip(layers, picks[rid])))
        assert_route_regret(regret, f"{what} request {rid}")
        assert_close_bf16(got[rid], ref, f"{what} request {rid}")
