"""Generation through the entry points, sampling kernels, long decoding."""
import math
import os
import subprocess
import sys

import pytest
import torch

import helpers as H
import plain_llama4 as P
from tiny_configs import CONFIGS, make_model_dir

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"


def test_greedy_generation_matches_plain(tmp_path):
    """Tiny A, 32-bit: prompts of 5 / 23 / 40 tokens, 16 greedy steps each, under continuous
    batching with prompts cut into portions."""
    d = make_model_dir(tmp_path, "A", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    prompts = [H.random_tokens(n, 256, 40 + n) for n in (5, 23, 40)]
    want = [P.generate(c, W, p, 16) for p in prompts]
    eng = H.make_engine(d, "float32", kv_tokens=256, max_num_seqs=3, max_tokens_per_step=16)
    got = eng.generate(prompts, max_new_tokens=16, temperature=0.0)
    assert [r.token_ids for r in got] == want
    assert all(r.finish_reason == "length" and r.prompt_tokens == len(p) for r, p in zip(got, prompts))
    assert eng.last_stats.prefill_tokens == 68 and eng.last_stats.decode_tokens == 3 * 15
    eng.cache.check_invariants()
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    # one request at a time gives the same tokens
    solo = H.make_engine(d, "float32", kv_tokens=128, max_num_seqs=1)
    assert [solo.generate([p], max_new_tokens=16)[0].token_ids for p in prompts] == want


@pytest.mark.parametrize("which,std", [("B", 0.1), ("D", 0.06)])
def test_greedy_generation_in_bfloat16_token_for_token(tmp_path, which, std):
    """Greedy generation in bfloat16 through the entry point, then every generated token against
    the plain implementation with bfloat16 storage and the engine's own routes: the token must be
    the plain implementation's best, or lie below its best by no more than the bound on a
    bfloat16 logit (two logits, each off by at most the bound).  The generation's steps (prompt
    whole, then one token a step) are replayed through the step function for the routes, and the
    replay must give the generated tokens exactly."""
    d = make_model_dir(tmp_path, which, std=std)
    vocab = CONFIGS[which]["vocab_size"]
    tol_max, _ = H.bounds_of(d)
    n_new = 24
    strict = 0
    for i, n in enumerate((6, 30, 50)):
        prompt = H.random_tokens(n, vocab, 60 + i)
        eng = H.make_engine(d, "bfloat16", kv_tokens=256, max_num_seqs=2, max_tokens_per_step=64)
        out = eng.generate([prompt], max_new_tokens=n_new, temperature=0.0)[0].token_ids
        assert len(out) == n_new
        toks = prompt + out[:-1]
        got, picks, seen = H.run_cut(eng, "g", toks, [n] + [1] * (n_new - 1), with_routes=True)
        assert got[n - 1:].argmax(dim=-1).tolist() == out, "the replayed steps choose other tokens than the generation did"
        H.assert_routes_are_the_best(d, picks, seen, f"{which} generation {i}")
        ref = H.plain_logits_routed(d, toks, dict(zip(H.moe_layers_of(d), picks)))[n - 1:]
        rms = ref.double().pow(2).mean(dim=-1).sqrt()
        chosen = ref.gather(1, torch.tensor(out)[:, None])[:, 0]
        below = (ref.max(dim=-1).values - chosen).double() / rms
        assert float(below.max()) <= 2 * tol_max, f"{which} prompt {i}: a generated token lies {float(below.max()):.3f} row rms below the plain best"
        strict += int((ref.argmax(dim=-1) == torch.tensor(out)).sum())
    assert strict >= 3 * n_new - 3, f"only {strict} of {3 * n_new} tokens are the plain implementation's own choice"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_chosen_on_the_device_are_the_argmax_of_the_logits(tmp_path, dtype):
    """select="argmax": only token ids leave the device; they are the lowest index of the largest
    logit, whether the step is launched part by part, replayed from a graph, or mixed."""
    from sharpinference_amd.engine import StepEntry

    d = make_model_dir(tmp_path, "D", std=0.06)
    toks = {r: H.random_tokens(30, 500, 20 + i) for i, r in enumerate("abc")}
    engs = [H.make_engine(d, dtype, kv_tokens=192, max_num_seqs=3) for _ in range(2)]
    for e in engs:
        for r in toks:
            e.add_request(r)
    plan = [[("a", 12), ("b", 20)], [("a", 1), ("b", 1), ("c", 9)], [("a", 1), ("b", 1), ("c", 1)], [("a", 1), ("b", 1), ("c", 1)],
            [("c", 1)], [("c", 1)]]
    at = {r: 0 for r in toks}
    for step in plan:
        entries = []
        for r, n in step:
            entries.append(StepEntry(r, toks[r][at[r]:at[r] + n], (n - 1,)))
            at[r] += n
        lg = engs[0].step(entries)
        ids = engs[1].step(entries, select="argmax")
        assert ids.dtype == torch.int32 and ids.shape == (len(entries),)
        assert ids.cpu().tolist() == [P.greedy(row) for row in lg.float().cpu()]
    assert engs[1].runner.graph_replays >= 4 and any(len(k) == 3 and k[2] == "argmax" for k in engs[1].runner._graphs)


def test_temperature_generation_matches_plain(tmp_path):
    """Tiny B, 32-bit: prompts of 1 / 17 / 50 / 77 tokens, 24 steps at temperature 0.8 with
    fixed seeds: the same uniforms give the same tokens."""
    d = make_model_dir(tmp_path, "B", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    prompts = [H.random_tokens(n, 384, 70 + n) for n in (1, 17, 50, 77)]
    seeds = [11, 12, 13, 14]
    want = [P.generate(c, W, p, 24, temperature=0.8, seed=s) for p, s in zip(prompts, seeds)]
    eng = H.make_engine(d, "float32", kv_tokens=512, max_num_seqs=4, max_tokens_per_step=40)
    got = eng.generate(prompts, max_new_tokens=24, temperature=0.8, seeds=seeds)
    assert [r.token_ids for r in got] == want
    assert len({tuple(w) for w in want}) == 4


@pytest.mark.parametrize("which,std", [("B", 0.1), ("D", 0.06)])
def test_temperature_generation_in_bfloat16_token_for_token(tmp_path, which, std):
    """Sampled generation in bfloat16 (temperature 0.8, fixed seeds) through the entry point, then
    every drawn token twice over.  (1) The draw itself: the plain sampling function on the ENGINE's
    own logits of that step (the generation's steps replayed through the step function) and the
    same uniform u gives the same token.  (2) The logits behind it: against the plain implementation
    with bfloat16 storage and the engine's own routes, fed the engine's tokens, u must lie in the
    token's interval of the plain cumulative distribution, widened by what the bound on a bfloat16
    logit allows (logits off by at most d move every probability by a factor within
    exp(+-2 d / T), and so any cumulative sum by at most exp(2 d / T) - 1).  With distributions as
    flat as a random model's, a shift of a thousandth already moves u into a neighbour's interval,
    so the plain implementation's own draw is the same token for most steps, not for all."""
    d = make_model_dir(tmp_path, which, std=std)
    vocab = CONFIGS[which]["vocab_size"]
    tol_max, _ = H.bounds_of(d)
    n_new, temp = 24, 0.8
    same = total = 0
    for i, (n, seed) in enumerate(((6, 21), (30, 22), (50, 23))):
        prompt = H.random_tokens(n, vocab, 80 + i)
        eng = H.make_engine(d, "bfloat16", kv_tokens=256, max_num_seqs=2, max_tokens_per_step=64)
        out = eng.generate([prompt], max_new_tokens=n_new, temperature=temp, seeds=[seed])[0].token_ids
        assert len(out) == n_new
        toks = prompt + out[:-1]
        got, picks, seen = H.run_cut(eng, "g", toks, [n] + [1] * (n_new - 1), with_routes=True)
        H.assert_routes_are_the_best(d, picks, seen, f"{which} sampled generation {i}")
        ref = H.plain_logits_routed(d, toks, dict(zip(H.moe_layers_of(d), picks)))[n - 1:]
        us = P.uniform_stream(seed, n_new)
        own = [P.sample(got[n - 1 + j], us[j], temp) for j in range(n_new)]
        assert sum(a != b for a, b in zip(own, out)) <= 1, f"{which} prompt {i}: the tokens drawn are not the draws from the engine's own logits: {out} vs {own}"
        for j, tok in enumerate(out):
            total += 1
            if P.sample(ref[j], us[j], temp) == tok:
                same += 1
                continue
            rms = float(ref[j].double().pow(2).mean().sqrt())
            slack = math.expm1(2.0 * tol_max * rms / temp)
            cdf = torch.cumsum(P.softmax_f32(ref[j].float() * (1.0 / temp)).double(), 0)
            lo = float(cdf[tok - 1]) if tok > 0 else 0.0
            assert lo - slack <= us[j] <= float(cdf[tok]) + slack, \
                f"{which} prompt {i} step {j}: token {tok} drawn at u = {us[j]:.4f}, its plain interval is [{lo:.4f}, {float(cdf[tok]):.4f}] (slack {slack:.4f})"
    assert same >= total * 3 // 4, f"only {same} of {total} sampled tokens are the plain implementation's own draw"


def test_stop_tokens_and_tiny_pool(tmp_path):
    d = make_model_dir(tmp_path, "A", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    prompts = [H.random_tokens(n, 256, 5 + n) for n in (9, 30, 12, 25, 18)]
    free = [P.generate(c, W, p, 12) for p in prompts]
    stop = free[1][4]
    want = [P.generate(c, W, p, 12, stop=(stop,)) for p in prompts]
    assert len(want[1]) < 12
    # pool of 64 tokens: at most one or two requests fit; the rest wait for pages
    eng = H.make_engine(d, "float32", kv_tokens=64, max_num_seqs=4, max_tokens_per_step=24)
    got = eng.generate(prompts, max_new_tokens=12, temperature=0.0, stop_token_ids=(stop,))
    assert [r.token_ids for r in got] == want
    assert [r.finish_reason for r in got] == ["stop" if len(w) < 12 else "length" for w in want]
    assert all(g.pool.total_allocs > g.pool.num_pages for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("graphs", [True, False])
def test_steps_launched_on_end_give_the_same_generation(tmp_path, dtype, graphs):
    """While every request decodes greedily the engine launches several steps on end, each on
    what the step before chose (on the device), and reads the tokens back together.  The tokens,
    the reasons to stop and the pages are those of an engine that waits for every step, whatever
    the number of steps on end, also when a request meets its stop token in the middle of a run
    or the requests end at different lengths."""
    from sharpinference_amd import SamplingParams
    from sharpinference_amd.engine import StepEntry

    d = make_model_dir(tmp_path, "D", std=0.06)
    prompts = [H.random_tokens(n, 500, 70 + n) for n in (9, 30, 12, 25, 18)]
    one = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=5, decode_graphs=graphs, decode_run_ahead=1)
    free = one.generate(prompts, max_new_tokens=23)
    stop = free[1].token_ids[9]
    params = [SamplingParams(temperature=0.0, max_new_tokens=m, stop_token_ids=(stop,)) for m in (23, 23, 14, 20, 6)]
    want = one.generate(prompts, params)
    assert any(r.finish_reason == "stop" for r in want) and any(r.finish_reason == "length" for r in want)
    for ahead in (2, 4, 7):
        eng = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=5, decode_graphs=graphs, decode_run_ahead=ahead)
        got = eng.generate(prompts, params)
        assert [r.token_ids for r in got] == [r.token_ids for r in want], ahead
        assert [r.finish_reason for r in got] == [r.finish_reason for r in want]
        assert eng.last_stats.decode_tokens == one.last_stats.decode_tokens and eng.last_stats.steps == one.last_stats.steps
        eng.cache.check_invariants()
        assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    # the runner's own entry: steps on end against the same steps one by one
    ids = ["x", "y", "z"]
    runs = []
    for on_end in (True, False):
        eng = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=3, decode_graphs=graphs)
        first = []
        for r, p in zip(ids, prompts):
            eng.add_request(r)
            first.append(int(eng.step([StepEntry(r, p, (len(p) - 1,))], select="argmax").cpu()[0]))
        if on_end:
            runs.append(eng.decode_steps([StepEntry(r, (t,), (0,)) for r, t in zip(ids, first)], 6).cpu().tolist())
        else:
            rows, cur = [], first
            for _ in range(6):
                cur = eng.step([StepEntry(r, (t,), (0,)) for r, t in zip(ids, cur)], select="argmax").cpu().tolist()
                rows.append(cur)
            runs.append(rows)
    assert runs[0] == runs[1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_token_budget_below_the_live_requests_generates_the_same(tmp_path, dtype):
    """Two tokens a step for three requests: the batch is then a changing part of the running
    requests.  Steps are never launched on end for a batch that leaves a running request out (its
    cache would not have been stepped), a stop token met on the way ends its request where the
    waiting engine ends it, nobody starves, and in 32-bit the tokens are the plain
    implementation's, which knows nothing of steps."""
    from sharpinference_amd import SamplingParams

    d = make_model_dir(tmp_path, "A", std=0.1)
    prompts = [H.random_tokens(n, 256, 40 + n) for n in (7, 12, 5)]
    one = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=3, max_tokens_per_step=2, decode_run_ahead=1)
    free = one.generate(prompts, max_new_tokens=14)
    stop = free[0].token_ids[6]
    params = [SamplingParams(temperature=0.0, max_new_tokens=m, stop_token_ids=(stop,)) for m in (14, 14, 9)]
    want = one.generate(prompts, params)
    assert want[0].finish_reason == "stop" and len(want[0].token_ids) <= 6
    if dtype == "float32":
        c, W = P.read_config(d), P.load_weights(d)
        plain = [P.generate(c, W, p, q.max_new_tokens, stop=(stop,)) for p, q in zip(prompts, params)]
        assert [r.token_ids for r in want] == plain
    for ahead in (4, 7):
        eng = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=3, max_tokens_per_step=2, decode_run_ahead=ahead)
        got = eng.generate(prompts, params)
        assert [r.token_ids for r in got] == [r.token_ids for r in want], ahead
        assert [r.finish_reason for r in got] == [r.finish_reason for r in want]
        eng.cache.check_invariants()
        assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    # the same prompts with room for everybody: the budget changes the steps, not the tokens
    wide = H.make_engine(d, dtype, kv_tokens=512, max_num_seqs=3, max_tokens_per_step=64)
    if dtype == "float32":
        assert [r.token_ids for r in wide.generate(prompts, params)] == [r.token_ids for r in want]


@pytest.mark.parametrize("seed", [3, 11, 17, 54, 75, 81])
def test_random_workloads_generate_the_same_batched_as_alone(tmp_path, seed):
    """Random workloads (2 to 9 requests of random lengths; greedy and sampled rows, top-k on some, a
    stop token each; random limits on live requests, tokens a step, pages, steps launched on end)
    in 32-bit: every request gets the tokens and the finish reason it gets alone, nothing is left in
    the pools.  (In 32-bit a row's logits do not depend on the batch; in bfloat16 they do, within
    rounding, and a near-tie may flip there.)"""
    import random
    from sharpinference_amd import SamplingParams
    from sharpinference_amd.engine import Engine

    rng = random.Random(seed)
    which = rng.choice("ABCD")
    d = make_model_dir(tmp_path, which, std=0.05)
    vocab = CONFIGS[which]["vocab_size"]
    n = rng.randint(2, 9)
    prompts = [H.random_tokens(rng.choice([1, 2, 5, 17, 40, 64, 65, 100, 130]), vocab, seed * 100 + i) for i in range(n)]
    new = [rng.choice([1, 2, 7, 20, 40]) for _ in range(n)]
    params = [SamplingParams(temperature=rng.choice([0.0, 0.0, 0.8]), max_new_tokens=m, seed=seed * 7 + i, top_k=rng.choice([0, 5]),
                             stop_token_ids=(rng.randrange(vocab),)) for i, m in enumerate(new)]
    seqs, budget, ps, ahead = rng.randint(1, 6), rng.choice([1, 2, 3, 8, 33, 2048]), rng.choice([16, 32]), rng.choice([1, 4])
    need = max((len(p) + m + ps - 1) // ps * ps for p, m in zip(prompts, new))
    kv = rng.choice([need, 2 * need, 4 * need])
    eng = Engine(d, dtype="float32", max_num_seqs=seqs, max_tokens_per_step=budget, kv_tokens=kv, page_size=ps,
                 decode_run_ahead=ahead)
    got = eng.generate(prompts, params)
    eng.cache.check_invariants()
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    one = Engine(d, dtype="float32", max_num_seqs=1, kv_tokens=need, page_size=ps, decode_run_ahead=1, decode_graphs=False)
    for i, (p, sp) in enumerate(zip(prompts, params)):
        ref = one.generate([p], [sp])[0]
        assert (got[i].token_ids, got[i].finish_reason) == (ref.token_ids, ref.finish_reason), \
            f"request {i} of {n} (live {seqs}, budget {budget}, page {ps}, ahead {ahead}, pool {kv})"
        assert len(ref.token_ids) <= new[i]


def test_chunks_stream_in_order_and_cancelling_gives_pages_back(tmp_path):
    """The typed chunks of a generation: per prompt one usage chunk first, its tokens in order,
    one stop chunk last; the tokens are those of generate().  A prompt cancelled half-way ends
    with "abort" while the others go on unchanged, a prompt too long for the pool ends at once,
    and closing the generator early leaves no page held."""
    d = make_model_dir(tmp_path, "A", std=0.1)
    prompts = [H.random_tokens(n, 256, 90 + n) for n in (7, 21, 33)]
    eng = H.make_engine(d, "float32", kv_tokens=256, max_num_seqs=3, max_tokens_per_step=16)
    want = [r.token_ids for r in eng.generate(prompts, max_new_tokens=10)]
    seen = {i: [] for i in range(3)}
    for c in eng.generate_chunks(prompts, max_new_tokens=10):
        seen[c.index].append(c)
        if c.kind == "usage":
            assert eng.queue_depth == 3 and eng.active_requests == 0     # nothing is admitted before the first step
        elif sum(len(v) for v in seen.values()) == 4:                    # the first token: the others still run
            assert c.kind == "token" and eng.active_requests >= 2
    for i, p in enumerate(prompts):
        kinds = [c.kind for c in seen[i]]
        assert kinds == ["usage"] + ["token"] * 10 + ["stop"]
        assert seen[i][0].prompt_tokens == len(p) and [c.token_id for c in seen[i][1:-1]] == want[i]
        assert seen[i][-1].finish_reason == "length" and seen[i][-1].truncated_by_max_tokens
    assert eng.active_requests == 0 and eng.queue_depth == 0
    # prompt 1 is cancelled once it has 4 tokens; a 300-token prompt can never fit into 256
    got = {i: [] for i in range(4)}
    reasons = {}
    for c in eng.generate_chunks(prompts + [H.random_tokens(300, 256, 1)], max_new_tokens=10,
                                 should_cancel=lambda i: i == 1 and len(got[1]) >= 4):
        if c.kind == "token":
            got[c.index].append(c.token_id)
        elif c.kind == "stop":
            reasons[c.index] = c.finish_reason
    assert reasons == {0: "length", 1: "abort", 2: "length", 3: "too_long"}
    assert got[0] == want[0] and got[2] == want[2] and got[1] == want[1][:4] and got[3] == []
    # closed early
    gen = eng.generate_chunks(prompts, max_new_tokens=10)
    for c in gen:
        if c.kind == "token":
            break
    gen.close()
    eng.cache.check_invariants()
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups) and not eng.cache.requests
    assert [r.token_ids for r in eng.generate(prompts, max_new_tokens=10)] == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path, dtype):
    """Hundreds of single-token steps: windows slide over many pages that are released and reused."""
    d = make_model_dir(tmp_path, "A", std=0.1)
    toks = H.random_tokens(330, 256, 8)
    eng = H.make_engine(d, dtype, kv_tokens=352, max_num_seqs=1)
    H.check_against_plain(eng, d, dtype, "long", toks, [10] + [1] * 320, f"A {dtype} long decoding")
    assert eng.cache.groups[0].pool.total_allocs >= 20


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(tmp_path, dtype):
    d = make_model_dir(tmp_path, "B", std=0.1)
    eng = H.make_engine(d, dtype)
    for toks in ([7], [7, 300], [1, 2, 3]):
        H.check_against_plain(eng, d, dtype, "f", toks, [1] * len(toks), f"B {dtype} first tokens")


def test_sampling_kernels_against_plain():
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(0)
    V = 1003
    logits = (torch.randn(6, V, generator=g) * 3).to(DEV)
    logits[2, 17] = logits[2, 900] = logits[2].max() + 1.0             # a tie: the lower index wins
    logits[3] = -5.0                                                   # all equal
    am = ops.argmax_rows(logits).cpu().tolist()
    assert am == [P.greedy(logits[i].cpu()) for i in range(6)] and am[2] == 17 and am[3] == 0
    cases = [dict(temperature=0.8), dict(temperature=1.0, top_k=5), dict(temperature=1.3, top_p=0.7),
             dict(temperature=0.9, min_p=0.1), dict(temperature=0.7, top_k=40, top_p=0.95, min_p=0.05),
             dict(temperature=2.0, top_k=1)]
    for case in cases:
        us = P.uniform_stream(3, 6)
        temp = torch.full((6,), case["temperature"], device=DEV)
        tk = torch.full((6,), case.get("top_k", 0), dtype=torch.int32, device=DEV)
        tp = torch.full((6,), case.get("top_p", 1.0), device=DEV)
        mp = torch.full((6,), case.get("min_p", 0.0), device=DEV)
        got = ops.sample_rows(logits, temp, torch.tensor(us, device=DEV), tk, tp, mp).cpu().tolist()
        want = [P.sample(logits[i].cpu(), us[i], **case) for i in range(6)]
        if "top_p" in case:
            # row 3 is all ties: which of equal values the nucleus keeps is left open by the
            # reference (an unstable sort, Sampler.cs:543); the kernel keeps them all
            got[3] = want[3] = -1
        assert got == want, case


def test_sampling_with_a_small_top_k_over_a_large_vocabulary():
    """Rows with a small top-k gather the few entries that can survive and finish in LDS; larger k, and
    rows where too many entries tie at the cut, take the full path: both against the plain implementation,
    over many uniforms (also at the ends of [0, 1)), with ties at the k-th value."""
    from sharpinference_amd import ops

    g = torch.Generator().manual_seed(4)
    V = 50021
    R = 8
    logits = torch.randn(R, V, generator=g) * 2.5
    logits[1, 40000] = logits[1, 7] = logits[1, 123]                      # ties somewhere
    top = torch.topk(logits[2], 5).values[-1].item()
    logits[2, 11] = logits[2, 30011] = top                               # three entries tie at the 5th value
    logits[3] = 0.25                                                     # all equal: every entry survives any k
    logits[4] *= 0.01                                                    # nearly flat
    logits[5, 49999] = 30.0                                              # one entry holds all the mass
    logits[6] *= 3.0                                                     # peaked: a few hundred entries hold nearly all
    logits[7] *= 2.0
    logits = logits.to(DEV)
    # (without a top-k the few-entries path stands only where it can show that nothing else survives: the
    # peaked rows; the flat ones go on to the full path)
    cases = [dict(temperature=1.0, top_k=5), dict(temperature=0.7, top_k=40, top_p=0.95, min_p=0.05),
             dict(temperature=1.5, top_k=256, top_p=0.9), dict(temperature=0.8, top_k=300, min_p=0.02),
             dict(temperature=1.1, top_k=1), dict(temperature=0.9, top_k=64, top_p=0.5),
             dict(temperature=1.0, top_p=0.9), dict(temperature=0.8, min_p=0.05),
             dict(temperature=1.2, top_p=0.6, min_p=0.01), dict(temperature=0.6, top_p=0.99),
             dict(temperature=0.9), dict(temperature=1.0)]             # no filter at all: nothing is written, two passes
    for case in cases:
        for draw in range(3):
            us = P.uniform_stream(11 + draw, R)
            if draw == 0:
                us[0] = 0.0
                if "top_k" in case:      # (over thousands of entries it is the order of the additions that decides
                    us[7] = 1.0 - 2.0 ** -24   # whether the running sum reaches the largest uniform at all)
            temp = torch.full((R,), case["temperature"], device=DEV)
            tk = torch.full((R,), case.get("top_k", 0), dtype=torch.int32, device=DEV)
            tp = torch.full((R,), case.get("top_p", 1.0), device=DEV)
            mp = torch.full((R,), case.get("min_p", 0.0), device=DEV)
            got = ops.sample_rows(logits, temp, torch.tensor(us, device=DEV), tk, tp, mp).cpu().tolist()
            want = [P.sample(logits[i].cpu(), us[i], **case) for i in range(R)]
            if len(case) == 1:
                # no filter: the kernel keeps its running sums in double, so over 50,021 entries it is compared with
                # the same definition in double (a 32-bit running sum is off by more than an entry's probability)
                cum = torch.cumsum(torch.softmax(logits.double().cpu() / case["temperature"], -1), -1)
                want = [0 if us[i] <= 0 else int((cum[i] >= us[i]).float().argmax()) for i in range(R)]
                assert got[3] == want[3]           # also over 50,021 equal probabilities
            # row 3 is 50,021 equal probabilities: where their running sum passes u depends on the order of
            # the additions to the last bit, and which of equal values the nucleus keeps is left open
            assert "top_p" in case or abs(got[3] - want[3]) <= 2, (case, draw, got[3], want[3])
            got[3] = want[3] = -1
            assert got == want, (case, draw, got, want)


def test_penalties_and_bias_follow_the_reference_order():
    """reference: src/SharpInference.Engine/Sampler.cs:52-69, 414-433: bias, then the repetition
    penalty once per distinct token (divide if positive, multiply if negative), then
    count * frequency + presence subtracted."""
    from sharpinference_amd.sampling.params import SamplingParams
    from sharpinference_amd.sampling.sampler import Sampler

    logits = torch.tensor([[2.0, -1.0, 0.5, 3.0, 1.0]], device=DEV)
    p = SamplingParams(temperature=1e-4, repetition_penalty=2.0, frequency_penalty=0.5, presence_penalty=0.25,
                       logit_bias={4: 1.5}, penalty_last_n=0)
    # history 3, 3, 0: token 3 -> 3/2 - (2*0.5 + 0.25) = 0.25; token 0 -> 2/2 - 0.75 = 0.25; token 4 -> 2.5
    assert Sampler(DEV).sample(logits, [p], [0], [[3, 3, 0]]) == [4]
    q = SamplingParams(temperature=1e-4, repetition_penalty=2.0, penalty_last_n=0)
    assert Sampler(DEV).sample(logits, [q], [0], [[3]]) == [0]          # 3 -> 1.5 < 2
    assert Sampler(DEV).sample(torch.tensor([[-1.0, -1.5]], device=DEV), [q], [0], [[0]]) == [1]   # -1 * 2 = -2 < -1.5
    greedy = SamplingParams(temperature=0.0, repetition_penalty=5.0)    # greedy rows skip the penalties
    assert Sampler(DEV).sample(logits, [greedy], [0], [[3]]) == [3]


def test_command_line(tmp_path):
    d = make_model_dir(tmp_path, "A", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    prompt = H.random_tokens(12, 256, 1)
    want = P.generate(c, W, prompt, 8)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "sharpi-cli"), "-m", d, "-p", ",".join(map(str, prompt)),
                          "-n", "8", "--temp", "0", "--dtype", "fp32", "--kv-tokens", "128"],
                         capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.strip().splitlines()
    assert lines[0] == " ".join(map(str, prompt))
    assert lines[1].startswith(" ".join(map(str, want))) and lines[1].endswith("(length)")
    assert lines[-1].startswith("Prefill: 12 tokens, ") and "| Decode: 7 tokens, " in lines[-1] and lines[-1].endswith("t/s")


def test_command_line_interactive_mode_and_profile(tmp_path):
    """Without a prompt option the command reads prompts from standard input, a line a turn, every
    turn from an empty cache (the reference's interactive mode); --single-turn ends after the
    first; --profile prints a table of kernel classes."""
    d = make_model_dir(tmp_path, "A", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    p1, p2 = H.random_tokens(9, 256, 4), H.random_tokens(14, 256, 5)
    base = [sys.executable, os.path.join(ROOT, "bin", "sharpi-cli"), "-m", d, "-n", "5", "--temp", "0", "--dtype", "fp32",
            "--kv-tokens", "128"]
    feed = " ".join(map(str, p1)) + "\n\n" + ",".join(map(str, p2)) + "\n/exit\nnever read\n"
    out = subprocess.run(base, input=feed, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    body = out.stdout
    assert " ".join(map(str, P.generate(c, W, p1, 5))) + "  (length)" in body
    assert " ".join(map(str, P.generate(c, W, p2, 5))) + "  (length)" in body
    assert body.count("t/s") == 2 and "never" not in body
    out = subprocess.run(base + ["--single-turn", "--profile"], input=feed, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.count("(length)") == 1
    table = out.stderr
    for word in ("qkv", "attention", "experts", "head", "GB/s"):
        assert word in table, table


def test_command_line_with_text_and_the_model_s_end_token(tmp_path):
    """A folder with a tokenizer.json takes a text prompt and prints text; generation ends at the
    configuration's eos_token_id unless --ignore-eos is given."""
    import json

    from tokenizers import Tokenizer, models, pre_tokenizers

    d = make_model_dir(tmp_path, "A", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    prompt = H.random_tokens(12, 256, 2)
    want = P.generate(c, W, prompt, 8)
    end = want[4]
    cut = want.index(end)                                    # the end token's first appearance
    with open(os.path.join(d, "config.json")) as f:
        cfg = json.load(f)
    cfg["eos_token_id"] = [end, 255]
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    tok = Tokenizer(models.WordLevel({f"w{i}": i for i in range(256)}, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(os.path.join(d, "tokenizer.json"))
    text = " ".join(f"w{t}" for t in prompt)
    base = [sys.executable, os.path.join(ROOT, "bin", "sharpi-cli"), "-m", d, "-p", text, "-n", "8", "--temp", "0",
            "--dtype", "fp32", "--kv-tokens", "128"]
    out = subprocess.run(base, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.strip().splitlines()
    assert lines[0] == text
    assert lines[1] == " ".join(f"w{t}" for t in want[:cut]) + "  (stop)", lines[1]
    out = subprocess.run(base + ["--ignore-eos"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip().splitlines()[1] == " ".join(f"w{t}" for t in want) + "  (length)"
