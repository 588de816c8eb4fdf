"""Shared helpers of the GPU tests: ways of cutting a request into steps, and comparisons."""
from __future__ import annotations

import functools
import math
import random
from typing import Dict, List, Optional, Sequence

import torch

import plain_llama4 as P

# ---------------------------------------------------------------------------
# What a bfloat16 run may differ by, derived from bfloat16's rounding
# ---------------------------------------------------------------------------
# The plain implementation rounds every tensor where the engine stores one (``store_bf16``), with
# float arithmetic in between, so storage rounding as such is reproduced exactly.  What is left is
# the order of the float sums: where a sum lies near the middle of two bfloat16 values, another
# order rounds it to the other one, a difference of one spacing (2^-8 of the value: bfloat16 has 8
# significant bits); downstream of the first such difference the two runs are two separate
# roundings of slightly different numbers.  The bound below takes the two runs as INDEPENDENT
# roundings to nearest at every store: each rounding errs uniformly within half a spacing (rms
# 2^-8 / sqrt(12) of the value), the difference of two has rms 2^-8 / sqrt(6), and the stores
# along a token's path (STORES_PER_LAYER a layer: normed rows, q|k|v, rotated q and k, attention
# output, o-projection; normed rows, gate|up, activation, down, the experts' sum; and the final
# norm) add in quadrature, each taken to reach the logits with a relative weight of at most
# AMPLIFICATION (norms rescale, the softmax and SiLU have slopes of order one: stated, not
# derived).  Per row of logits, relative to the row's rms:
#   rms error  <=  AMPLIFICATION * 2^-8 / sqrt(6) * sqrt(STORES_PER_LAYER * layers + 1)
#   max error  <=  that * sqrt(2 ln(2 V)), the largest of V Gaussian values.
# tests/test_plain.py checks the model on the CPU: two plain runs that differ in the order of
# their sums only (float against double accumulation) lie within the bound and no more than a
# factor of twenty below it.  A wrong key, page, mask or weight gives errors of the size of the
# logits themselves, fifty times the bound.
BF16_SPACING = 2.0 ** -8
STORES_PER_LAYER = 10
AMPLIFICATION = 2.0


def bf16_bounds(n_layers: int, vocab: int):
    """(largest error, rms error) a row of bfloat16 logits may have against the plain
    implementation with bfloat16 storage, both relative to the row's rms."""
    tol_rms = AMPLIFICATION * BF16_SPACING / math.sqrt(6.0) * math.sqrt(STORES_PER_LAYER * n_layers + 1)
    return tol_rms * math.sqrt(2.0 * math.log(2.0 * vocab)), tol_rms


def bounds_of(model_dir: str):
    c = P.read_config(model_dir)
    return bf16_bounds(int(c["num_hidden_layers"]), int(c["vocab_size"]))


# The router works in float on the rows it is given, so its picks are checked exactly, against the
# rows the engine's router saw (the trace hands them out): a pick may lie below the best expert
# only by what the order of a float sum of H terms can change, H * 2^-24 * sum_i |x_i w_ei| for
# each of the two logits compared (the standard bound of a dot product).  That a bfloat16 run may
# route a token otherwise than a 32-bit run (its rows differ by roundings) is no error of the
# router: the plain implementation is then given the engine's picks, and the logits are compared
# under them.
def assert_picks_are_the_best(x: torch.Tensor, router_weight: torch.Tensor, ids: torch.Tensor, what: str) -> None:
    """ids [T, k] must name k different experts with the k largest router logits of rows x [T, H],
    up to float summation order."""
    x, w = x.double(), router_weight.double()
    r = x @ w.T
    k = ids.shape[1]
    srt = ids.long().sort(dim=1).values
    assert k == 1 or bool((srt[:, 1:] != srt[:, :-1]).all()), f"{what}: an expert picked twice for one token"
    best = r.sort(dim=1, descending=True).values[:, :k]
    got = torch.gather(r, 1, ids.long()).sort(dim=1, descending=True).values
    slack = 2.0 * x.shape[1] * 2.0 ** -24 * (x.abs() @ w.abs().T).max(dim=1).values
    below = (best - got).max(dim=1).values
    if bool((below > slack).any()):
        t = int((below - slack).argmax())
        raise AssertionError(f"{what}: token {t} was routed to experts {ids[t].tolist()}, {float(below[t]):.3e} below "
                             f"the best (float sums may differ by {float(slack[t]):.1e})")


def assert_routes_are_the_best(model_dir: str, picks, inputs, what: str) -> None:
    """Every routed layer's picks against the rows its router saw (see assert_picks_are_the_best)."""
    W = _model(model_dir)[1]
    for layer, ids, x in zip(moe_layers_of(model_dir), picks, inputs):
        assert_picks_are_the_best(x, W[f"model.layers.{layer}.feed_forward.router.weight"], ids, f"{what} layer {layer}")


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


@functools.lru_cache(maxsize=2)
def _model(model_dir: str):
    """(config, weights in float32) of a model folder, read once (a folder is written once by the tests)."""
    W = {k: v.float() if v.is_floating_point() else v for k, v in P.load_weights(model_dir).items()}
    return P.read_config(model_dir), W


@functools.lru_cache(maxsize=128)
def _plain_cached(model_dir: str, tokens: tuple, bf16_storage: bool) -> torch.Tensor:
    c, W = _model(model_dir)
    return P.forward(c, W, list(tokens), store=P.store_bf16 if bf16_storage else P._same)


def plain_logits(model_dir: str, tokens: Sequence[int], bf16_storage: bool = False) -> torch.Tensor:
    """Whole-sequence logits of the plain implementation; with bf16_storage, tensors are rounded
    where the engine's bfloat16 path stores them (the arithmetic stays float)."""
    return _plain_cached(model_dir, tuple(int(t) for t in tokens), bool(bf16_storage))


def moe_layers_of(model_dir: str) -> List[int]:
    c = P.read_config(model_dir)
    return [l for l in range(int(c["num_hidden_layers"])) if P.layer_is_moe(c, l)]


def plain_logits_routed(model_dir: str, tokens: Sequence[int], routes: Dict[int, torch.Tensor]) -> torch.Tensor:
    """The plain implementation with bfloat16 storage and the engine's own expert picks."""
    c, W = _model(model_dir)
    return P.forward(c, W, list(tokens), store=P.store_bf16, routes=routes)


def make_engine(model_dir: str, dtype: str, kv_tokens: int = 1024, max_num_seqs: int = 8, page_size: int = 16, **kw):
    from sharpinference_amd.engine import Engine

    return Engine(model_dir, dtype=dtype, device="cuda:0", kv_tokens=kv_tokens, max_num_seqs=max_num_seqs,
                  page_size=page_size, **kw)


def run_cut(engine, rid, tokens: Sequence[int], sizes: Sequence[int], with_routes: bool = False):
    """One request alone, cut into steps of the given sizes; logits at every position (and, if
    asked, per routed layer the expert picks ids [T, k] the engine made and the rows [T, H] its
    router saw)."""
    from sharpinference_amd.engine import StepEntry

    assert sum(sizes) == len(tokens)
    engine.add_request(rid)
    out, o = [], 0
    picks: List[List[torch.Tensor]] = []
    seen: List[List[torch.Tensor]] = []
    for s in sizes:
        trace: list = []
        lg = engine.step([StepEntry(rid, list(tokens[o:o + s]), list(range(s)))], router_trace=trace)
        out.append(lg.float().cpu())
        picks.append([ids.cpu() for ids, _, _ in trace])
        seen.append([x.float().cpu() for _, _, x in trace])
        o += s
    engine.free_request(rid)
    engine.cache.check_invariants()
    logits = torch.cat(out, 0)
    if not with_routes:
        return logits
    n_moe = len(picks[0])
    return (logits, [torch.cat([p[i] for p in picks], 0) for i in range(n_moe)],
            [torch.cat([p[i] for p in seen], 0) for i in range(n_moe)])


def check_against_plain(engine, model_dir: str, dtype: str, rid, tokens: Sequence[int], sizes: Sequence[int],
                        what: str) -> torch.Tensor:
    """Run one request cut into `sizes` and compare every position's logits with the plain
    implementation: 32-bit against pure 32-bit arithmetic; bfloat16 against the plain
    implementation with bfloat16 storage and the engine's own expert picks, which must be the
    best for the rows the engine's router saw."""
    if dtype == "float32":
        got = run_cut(engine, rid, tokens, sizes)
        assert_close_fp32(got, plain_logits(model_dir, tokens), what)
        return got
    got, picks, seen = run_cut(engine, rid, tokens, sizes, with_routes=True)
    assert_routes_are_the_best(model_dir, picks, seen, what)
    ref = plain_logits_routed(model_dir, tokens, dict(zip(moe_layers_of(model_dir), picks)))
    assert_close_bf16(got, ref, what, *bounds_of(model_dir))
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


def assert_close_bf16(got: torch.Tensor, ref: torch.Tensor, what: str, tol_max: float, tol_rms: float) -> None:
    """Per row: largest error and rms error, both relative to the row's rms, against the bounds
    of ``bf16_bounds``."""
    err = got.double() - ref.double()
    rms = ref.double().pow(2).mean(dim=-1).sqrt().clamp_min(1e-6)
    e_max = err.abs().max(dim=-1).values / rms
    e_rms = err.pow(2).mean(dim=-1).sqrt() / rms
    bad = (e_max > tol_max) | (e_rms > tol_rms)
    if bool(bad.any()):
        first = int(bad.nonzero()[0])
        raise AssertionError(f"{what}: max |diff| / row rms = {float(e_max.max()):.4f} (bound {tol_max:.4f}), "
                             f"rms diff / row rms = {float(e_rms.max()):.4f} (bound {tol_rms:.4f}); first wrong row {first}")


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


def wide_trace(requests: Dict[str, Sequence[int]], tail: int = 3, per_prefill_step: int = 8,
               late: Optional[str] = None) -> List[dict]:
    """Steps in the format of bin/trace_run for MANY live requests: the prompts (all but the last
    `tail` tokens of each) go in `per_prefill_step` at a time, then `tail` steps bring one token of
    every request.  `late` names a request whose whole prompt portion arrives in the first of
    those steps instead, beside the others' single tokens.  Logits are wanted everywhere."""
    steps: List[dict] = []
    ids = [r for r in requests if r != late]
    for i in range(0, len(ids), per_prefill_step):
        entries = []
        for rid in ids[i:i + per_prefill_step]:
            n = len(requests[rid]) - tail
            entries.append({"id": rid, "tokens": list(requests[rid][:n]), "want": list(range(n))})
        steps.append({"step": len(steps), "entries": entries, "end": []})
    for j in range(tail):
        entries = []
        for rid in ids:
            n = len(requests[rid]) - tail + j
            entries.append({"id": rid, "tokens": [requests[rid][n]], "want": [0]})
        if late is not None:
            toks = requests[late]
            n = len(toks) - tail + 1
            entries.append({"id": late, "tokens": list(toks[:n]) if j == 0 else [toks[n + j - 1]],
                            "want": list(range(n)) if j == 0 else [0]})
        steps.append({"step": len(steps), "entries": entries, "end": list(requests) if j == tail - 1 else []})
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
    the wanted places in order (and, if asked, {id: [ids per routed layer]} and {id: [router
    input rows per routed layer]})."""
    from sharpinference_amd.engine import StepEntry

    logits: Dict[str, List[torch.Tensor]] = {}
    picks: Dict[str, List[List[torch.Tensor]]] = {}
    seen: Dict[str, List[List[torch.Tensor]]] = {}
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
        trace = [(ids.cpu(), x.float().cpu()) for ids, _, x in trace]
        row, tok = 0, 0
        for e in st["entries"]:
            n = len(e["want"])
            if n:
                logits.setdefault(e["id"], []).append(lg[row:row + n])
                row += n
            if with_routes:
                picks.setdefault(e["id"], []).append([ids[tok:tok + len(e["tokens"])] for ids, _ in trace])
                seen.setdefault(e["id"], []).append([x[tok:tok + len(e["tokens"])] for _, x in trace])
            tok += len(e["tokens"])
        for rid in st["end"]:
            engine.free_request(rid)
            live.discard(rid)
        engine.cache.check_invariants()
    out = {rid: torch.cat(v, 0) for rid, v in logits.items()}
    if not with_routes:
        return out

    def joined(per_request):
        return {rid: [torch.cat([p[i] for p in per_step], 0) for i in range(len(per_step[0]))]
                for rid, per_step in per_request.items()}

    return out, joined(picks), joined(seen)


def check_trace_against_plain(engine, model_dir: str, dtype: str, requests: Dict[str, Sequence[int]],
                              steps: List[dict], what: str) -> None:
    if dtype == "float32":
        got = replay(engine, steps)
        for rid, toks in requests.items():
            assert_close_fp32(got[rid], plain_logits(model_dir, toks), f"{what} request {rid}")
        return
    got, picks, seen = replay(engine, steps, with_routes=True)
    layers = moe_layers_of(model_dir)
    bounds = bounds_of(model_dir)
    for rid, toks in requests.items():
        assert_routes_are_the_best(model_dir, picks[rid], seen[rid], f"{what} request {rid}")
        ref = plain_logits_routed(model_dir, toks, dict(zip(layers, picks[rid])))
        assert_close_bf16(got[rid], ref, f"{what} request {rid}", *bounds)
