"""The scheduler's decisions, driven by a scripted step function (no GPU), in the way the
reference tests its engines with a scripted forward pass
(reference: tests/SharpInference.Tests.ForwardPass/InferenceEngineChunkTests.cs:417-456)."""
from sharpinference_amd.cache.manager import CacheManager
from sharpinference_amd.cache.spec import KVSpec, WINDOW_CHUNK, WINDOW_NONE
from sharpinference_amd.engine.scheduler import Request, Scheduler
from sharpinference_amd.sampling.params import SamplingParams


def _cache(num_pages, max_requests=8):
    return CacheManager([KVSpec(1, 16, WINDOW_CHUNK, 32), KVSpec(1, 16, WINDOW_NONE, 0)], 16, num_pages, max_requests,
                        allocate=False)


def _run(sched, script, max_iters=10000):
    """script(request) -> next token.  Plays steps until nothing is left; returns the batches."""
    batches = []
    for _ in range(max_iters):
        if not sched.has_work():
            break
        batch = sched.schedule()
        if not batch:
            break
        for s in batch:                                   # what the step function does to the cache
            assert sched.cache.append(s.request.req_id, len(s.tokens)), "a running request ran out of pages"
        for s in batch:
            sched.cache.commit(s.request.req_id)
        sched.cache.check_invariants()
        batches.append([(s.request.req_id, list(s.tokens), s.samples) for s in batch])
        sched.update(batch, [script(s.request) if s.samples else None for s in batch])
    return batches


def _req(i, n_prompt, max_new, stop=()):
    return Request(i, list(range(1, n_prompt + 1)), SamplingParams(temperature=0.0, max_new_tokens=max_new, stop_token_ids=stop))


def test_portions_respect_the_budget_and_decodes_come_first():
    sched = Scheduler(_cache(64), max_num_seqs=4, max_tokens_per_step=16, max_model_len=256)
    reqs = [_req(0, 5, 3), _req(1, 40, 2), _req(2, 7, 2)]
    for r in reqs:
        sched.add(r)
    batches = _run(sched, lambda r: 100 + len(r.output))
    assert all(sum(len(t) for _, t, _ in b) <= 16 for b in batches)
    # step 0: request 0 whole (5), request 1 gets the rest of the budget (11)
    assert batches[0] == [(0, [1, 2, 3, 4, 5], True), (1, list(range(1, 12)), False)]
    # step 1: request 0 decodes first, then prompts in arrival order
    assert batches[1][0] == (0, [100], True) and batches[1][1][0] == 1 and len(batches[1][1][1]) == 15
    # each request's prompt went through exactly once, in order
    for r in reqs:
        seen = [t for b in batches for rid, toks, _ in b if rid == r.req_id for t in toks]
        assert seen[:len(r.prompt)] == r.prompt
        assert seen[len(r.prompt):] == r.output[:-1]      # the last token drawn is never fed back
    assert [r.finish_reason for r in reqs] == ["length"] * 3
    assert [len(r.output) for r in reqs] == [3, 2, 2]
    assert all(g.pool.num_free == g.pool.num_pages for g in sched.cache.groups)


def test_a_budget_below_the_number_of_decoders_starves_nobody():
    """Two tokens a step for three decoding requests: the reference decodes every active sequence
    in every iteration (reference: src/SharpInference.Engine/ContinuousBatchingEngine.cs:314-347);
    with less budget than that, whoever was left out goes first next time, so no request is ever
    more than one token behind another that was admitted with it."""
    sched = Scheduler(_cache(64), max_num_seqs=4, max_tokens_per_step=2, max_model_len=256)
    reqs = [_req(i, 2, 30) for i in range(3)]
    for r in reqs:
        sched.add(r)
    spread, base = [], None
    script = lambda r: 100 + len(r.output)
    for _ in range(200):
        if not sched.has_work():
            break
        batch = sched.schedule()
        assert 0 < sum(len(s.tokens) for s in batch) <= 2
        assert len(set(s.request.req_id for s in batch)) == len(batch)
        for s in batch:
            assert sched.cache.append(s.request.req_id, len(s.tokens))
            sched.cache.commit(s.request.req_id)
        sched.update(batch, [script(s.request) if s.samples else None for s in batch])
        if all(not r.finished and not r.in_prefill for r in reqs):
            base = base or [len(r.output) for r in reqs]
            gains = [len(r.output) - b for r, b in zip(reqs, base)]
            spread.append(max(gains) - min(gains))
    assert len(spread) >= 6 and max(spread) <= 1, spread
    assert [len(r.output) for r in reqs] == [30, 30, 30]
    assert all(g.pool.num_free == g.pool.num_pages for g in sched.cache.groups)


def test_stop_token_ends_without_being_emitted_even_as_first_token():
    sched = Scheduler(_cache(64), 4, 64, 256)
    a, b = _req("a", 4, 10, stop=(7,)), _req("b", 4, 10, stop=(7,))
    sched.add(a)
    sched.add(b)
    _run(sched, lambda r: 7 if r.req_id == "a" or len(r.output) == 2 else 50)
    assert a.output == [] and a.finish_reason == "stop"
    assert b.output == [50, 50] and b.finish_reason == "stop"


def test_fifo_admission_waits_for_pages_and_everything_completes():
    """A pool too small for all requests at once: later ones wait for the earlier ones' pages
    (reference: tests/SharpInference.Tests.ForwardPass/ContinuousBatchingTests.cs:504-539)."""
    sched = Scheduler(_cache(num_pages=6), max_num_seqs=8, max_tokens_per_step=32, max_model_len=256)
    reqs = [_req(i, 30 + i, 10) for i in range(5)]        # each needs 3 pages of the all-keys group
    for r in reqs:
        sched.add(r)
    first_step = {}
    batches = _run(sched, lambda r: 9)
    for n, b in enumerate(batches):
        for rid, _, _ in b:
            first_step.setdefault(rid, n)
    assert [first_step[i] for i in range(5)] == sorted(first_step[i] for i in range(5))   # nobody overtakes
    assert first_step[2] > first_step[1]                   # the third had to wait for pages
    assert all(len(set(rid for rid, _, _ in b)) <= 2 for b in batches)
    assert all(r.finish_reason == "length" and len(r.output) == 10 for r in reqs)
    assert all(g.pool.total_allocs > g.pool.num_pages for g in sched.cache.groups[1:])


def test_a_request_that_can_never_fit_is_refused_not_admitted():
    sched = Scheduler(_cache(num_pages=4), 4, 32, max_model_len=1000)
    big, ok = _req("big", 100, 10), _req("ok", 20, 5)
    sched.add(big)
    sched.add(ok)
    _run(sched, lambda r: 3)
    assert big.finish_reason == "too_long" and big.output == []
    assert ok.finish_reason == "length" and len(ok.output) == 5
    too_long = _req("ctx", 300, 5)
    sched2 = Scheduler(_cache(64), 4, 32, max_model_len=256)
    sched2.add(too_long)
    _run(sched2, lambda r: 3)
    assert too_long.finish_reason == "too_long"


def test_context_limit_and_zero_tokens_and_cancel():
    sched = Scheduler(_cache(64), 4, 32, max_model_len=24)
    r = _req("r", 20, 100)
    z = _req("z", 5, 0)
    c = _req("c", 5, 50)
    for x in (r, z, c):
        sched.add(x)
    steps = {"n": 0}

    def script(req):
        steps["n"] += 1
        if steps["n"] == 3:
            c.cancelled = True
        return 4

    _run(sched, script)
    assert r.finish_reason == "length" and len(r.prompt) + len(r.output) == 24
    assert z.finish_reason == "length" and z.output == []
    assert c.finish_reason == "abort" and 0 < len(c.output) < 50
    assert all(g.pool.num_free == g.pool.num_pages for g in sched.cache.groups)


def test_max_num_seqs_bounds_the_batch():
    sched = Scheduler(_cache(256), max_num_seqs=2, max_tokens_per_step=64, max_model_len=128)
    reqs = [_req(i, 3, 4) for i in range(5)]
    for r in reqs:
        sched.add(r)
    batches = _run(sched, lambda r: 1)
    assert max(len(b) for b in batches) == 2
    assert all(r.finish_reason == "length" for r in reqs)


def test_the_model_s_end_tokens_stop_a_request_unless_it_replaces_them():
    """None = the model's end-of-generation tokens, a tuple replaces them, additional ones are added to
    either (reference: src/SharpInference.Engine/Sampler.cs:724-741)."""
    assert SamplingParams().stop_set((5, 6)) == {5, 6}
    assert SamplingParams(stop_token_ids=()).stop_set((5, 6)) == set()
    assert SamplingParams(stop_token_ids=(9,)).stop_set((5, 6)) == {9}
    assert SamplingParams(additional_stop_token_ids=(9,)).stop_set((5, 6)) == {5, 6, 9}
    assert SamplingParams(stop_token_ids=(1,), additional_stop_token_ids=(9,)).stop_set((5, 6)) == {1, 9}

    sched = Scheduler(_cache(64), 4, 64, 256, end_of_generation=(7, 8))
    plain = Request("plain", [1, 2, 3], SamplingParams(temperature=0.0, max_new_tokens=6))
    deaf = Request("deaf", [1, 2, 3], SamplingParams(temperature=0.0, max_new_tokens=6, stop_token_ids=()))
    more = Request("more", [1, 2, 3], SamplingParams(temperature=0.0, max_new_tokens=6, additional_stop_token_ids=(50,)))
    for r in (plain, deaf, more):
        sched.add(r)
    _run(sched, lambda r: 8 if len(r.output) == 2 else 50)
    assert plain.output == [50, 50] and plain.finish_reason == "stop"
    assert deaf.output == [50, 50, 8, 50, 50, 50] and deaf.finish_reason == "length"
    assert more.output == [] and more.finish_reason == "stop"


def test_the_penalty_window_is_the_tail_of_prompt_and_output():
    """The last penalty_last_n tokens of prompt + output (0 = all), the prompt left out if it is not to
    seed the window (reference: src/SharpInference.Engine/Sampler.cs:764-798)."""
    import random

    from sharpinference_amd.sampling.sampler import penalty_window

    rng = random.Random(0)
    for _ in range(2000):
        p = SamplingParams(penalty_last_n=rng.choice([0, 1, 3, 5, 8, 100]), penalty_seed_from_prompt=rng.random() < 0.5)
        prompt = [rng.randrange(50) for _ in range(rng.randrange(0, 9))]
        out = [rng.randrange(50) for _ in range(rng.randrange(0, 9))]
        whole = (prompt if p.penalty_seed_from_prompt else []) + out
        assert penalty_window(p, prompt, out) == (whole[-p.penalty_last_n:] if p.penalty_last_n > 0 else whole)


def test_windowed_pools_are_bounded_by_the_window_and_admission_never_runs_dry():
    """A windowed group's pool is made for what its windows can hold at once, (window + one step)
    per request, however long the requests grow; admission reserves against exactly that, so a
    running request never finds the pool empty."""
    from sharpinference_amd.cache.manager import pool_sizes

    page, window, step, n_req, length = 16, 32, 24, 5, 4000
    specs = [KVSpec(1, 16, WINDOW_CHUNK, window), KVSpec(1, 16, WINDOW_NONE, 0)]
    sizes = pool_sizes(specs, page, n_req, length, step)
    assert sizes[("kv", 0, 0)] == n_req * (length // page)
    assert sizes[("kv", 1, window)] * page <= (window + step + 2 * page) * n_req       # two pages of slack for the edges
    assert sizes[("kv", 1, window)] < sizes[("kv", 0, 0)] // 20
    cache = CacheManager(specs, page, sizes, n_req, allocate=False)
    sched = Scheduler(cache, max_num_seqs=n_req, max_tokens_per_step=step, max_model_len=length)
    reqs = [_req(i, 300 + 37 * i, 150) for i in range(n_req + 2)]
    for r in reqs:
        sched.add(r)
    batches = _run(sched, lambda r: 1)            # _run asserts that no append of a running request fails
    assert all(r.finish_reason == "length" and len(r.output) == 150 for r in reqs)
    assert max(len(b) for b in batches) == n_req
    assert all(g.pool.num_free == g.pool.num_pages for g in cache.groups)
    # a budget in pages caps the unwindowed group only when it is the smaller
    capped = pool_sizes(specs, page, n_req, length, step, budget_pages=100)
    assert capped[("kv", 0, 0)] == 100 and capped[("kv", 1, window)] == sizes[("kv", 1, window)]
