"""The engine against the plain implementation: every way of cutting a request into steps."""
import pytest
import torch

import helpers as H
import plain_llama4 as P
from tiny_configs import CONFIGS, as_other_tools_write_it, make_model_dir, write_other_layout

pytestmark = pytest.mark.gpu

PROMPTS = {"A": [5, 23, 40 + 16], "B": [1, 17, 50, 77 + 24], "C": [3, 64, 95], "D": [2, 70, 150, 260]}


@pytest.fixture(scope="module", params=[("A", 0.02), ("B", 0.02), ("C", 0.02), ("A", 0.1), ("B", 0.08), ("C", 0.1), ("D", 0.02), ("D", 0.06)],
                ids=lambda p: f"{p[0]}-std{p[1]}")
def model_dir(request, tmp_path_factory):
    which, std = request.param
    return which, make_model_dir(tmp_path_factory.mktemp(f"m{which}"), which, std=std)


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def engine(request, model_dir):
    which, d = model_dir
    return which, d, request.param, H.make_engine(d, request.param)


def _requests(which):
    vocab = CONFIGS[which]["vocab_size"]
    return [H.random_tokens(n, vocab, 100 + i) for i, n in enumerate(PROMPTS[which])]


def test_whole(engine):
    which, d, dtype, eng = engine
    for i, toks in enumerate(_requests(which)):
        H.check_against_plain(eng, d, dtype, f"w{i}", toks, H.whole(len(toks)), f"{which} {dtype} whole request {i}")


def test_last_tokens_decoded(engine):
    which, d, dtype, eng = engine
    for i, toks in enumerate(_requests(which)):
        H.check_against_plain(eng, d, dtype, f"d{i}", toks, H.last_decoded(len(toks)),
                              f"{which} {dtype} last-32-decoded request {i}")


def test_changing_portions(engine):
    which, d, dtype, eng = engine
    for i, toks in enumerate(_requests(which)):
        for seed in (0, 1):
            H.check_against_plain(eng, d, dtype, f"p{i}", toks, H.changing_portions(len(toks), seed),
                                  f"{which} {dtype} portions(seed {seed}) request {i}")


def test_token_by_token(engine):
    which, d, dtype, eng = engine
    toks = _requests(which)[-1]
    H.check_against_plain(eng, d, dtype, "t", toks, [1] * len(toks), f"{which} {dtype} token by token")


def test_cuts_agree_fp32(engine):
    """In 32-bit the cut must not change a logit beyond rounding: far below the tolerance."""
    which, d, dtype, eng = engine
    if dtype != "float32":
        pytest.skip("32-bit only")
    toks = _requests(which)[-1]
    a = H.run_cut(eng, "x", toks, H.whole(len(toks)))
    b = H.run_cut(eng, "y", toks, H.changing_portions(len(toks), 3))
    assert float((a - b).abs().max()) <= 1e-5 * max(1.0, float(a.abs().max()))


@pytest.mark.parametrize("seed", [0, 1])
def test_mixed_batches_with_page_reuse(model_dir, seed):
    """Up to four live requests, portions of some beside decoded tokens of others, in a pool so
    small that pages of finished requests are used again."""
    which, d = model_dir
    vocab = CONFIGS[which]["vocab_size"]
    lens = [37, 70, 5, 101, 64, 49, 83]
    reqs = {f"r{i}": H.random_tokens(n, vocab, 300 + 10 * seed + i) for i, n in enumerate(lens)}
    steps = H.mixed_trace(reqs, seed)
    assert max(len(s["entries"]) for s in steps) >= 3
    assert any(len(e["tokens"]) == 1 for s in steps for e in s["entries"]) and \
        any(len(e["tokens"]) > 1 for s in steps for e in s["entries"])
    held = H.tokens_held(steps)
    for dtype in ("float32", "bfloat16"):
        eng = H.make_engine(d, dtype, kv_tokens=held, max_num_seqs=4)
        H.check_trace_against_plain(eng, d, dtype, reqs, steps, f"{which} {dtype} mixed(seed {seed})")
        for g in eng.cache.groups:
            assert g.pool.total_allocs > g.pool.num_pages, "the pool was large enough to never reuse a page"
            assert g.pool.num_free == g.pool.num_pages


@pytest.mark.parametrize("seed,lens,tail,max_live,page_size", [
    (112, [65, 64, 200, 129, 5, 40, 17, 90], 32, 2, 32), (133, [40, 200, 128, 200, 200, 40], 1, 4, 16),
    (156, [17, 200, 40, 5, 17, 5, 257, 5], 32, 3, 32)])
def test_mixed_traces_with_a_sharp_softmax_stay_inside_the_bound(tmp_path, seed, lens, tail, max_live, page_size):
    """Configuration D at a weight scale of 0.08: scores spread so far that a probability rounded to
    8 bits before the product with the values shows in the logits (these traces left the bound
    when the prompt kernel kept only the high half of its probabilities).  In bfloat16 under the
    engine's picks; in 32-bit under them too, so that a near-tie of two experts is no failure."""
    d = make_model_dir(tmp_path, "D", std=0.08)
    vocab = CONFIGS["D"]["vocab_size"]
    reqs = {f"r{i}": H.random_tokens(n, vocab, 1000 * seed + i) for i, n in enumerate(lens)}
    steps = H.mixed_trace(reqs, seed, max_live=max_live, tail=tail)
    held = H.tokens_held(steps, round_to=max(64, page_size))
    eng = H.make_engine(d, "bfloat16", kv_tokens=held, max_num_seqs=4, page_size=page_size)
    H.check_trace_against_plain(eng, d, "bfloat16", reqs, steps, f"D 0.08 bfloat16 mixed(seed {seed})")
    eng = H.make_engine(d, "float32", kv_tokens=held, max_num_seqs=4, page_size=page_size)
    got, picks, seen = H.replay(eng, steps, with_routes=True)
    layers = H.moe_layers_of(d)
    c, W = H._model(d)
    for rid, toks in reqs.items():
        H.assert_routes_are_the_best(d, picks[rid], seen[rid], f"request {rid}")
        ref = P.forward(c, W, list(toks), store=P._same, routes=dict(zip(layers, picks[rid])))
        H.assert_close_fp32(got[rid], ref, f"D 0.08 float32 mixed(seed {seed}) request {rid}")


WIDTHS = [5, 8, 16, 17, 32, 33, 64, 65]   # both sides of every batch size at which a step changes kernels


def wide_requests(n: int, vocab: int, seed: int, lo: int = 4, hi: int = 40):
    import random

    rng = random.Random(seed)
    return {f"w{i}": H.random_tokens(rng.randint(lo, hi), vocab, 7000 + 100 * seed + i) for i in range(n)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("width", WIDTHS)
def test_wide_decode_batches(tmp_path_factory, width, dtype):
    """As many live requests as a serving step has: 5 to 65 single-token entries in one step
    (graphs at once up to 16; the shared expert riding with the routed ones up to 16 tokens; the few-rows
    products up to 16 rows and the library beyond; picks taken straight from the router up to 64
    pairs and sorted beyond), every logit against the plain implementation."""
    d = make_model_dir(tmp_path_factory.mktemp("wide"), "D", std=0.06)
    reqs = wide_requests(width, 500, width)
    steps = H.wide_trace(reqs)
    assert max(len(st["entries"]) for st in steps) == width and all(len(e["tokens"]) == 1 for e in steps[-1]["entries"])
    eng = H.make_engine(d, dtype, kv_tokens=H.tokens_held(steps), max_num_seqs=width)
    H.check_trace_against_plain(eng, d, dtype, reqs, steps, f"D {dtype} {width} live requests")
    assert (eng.runner.graph_replays > 0) == (width <= 16)
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sixty_decoded_tokens_beside_a_portion(tmp_path, dtype):
    d = make_model_dir(tmp_path, "D", std=0.06)
    reqs = wide_requests(60, 500, 3)
    reqs["late"] = H.random_tokens(42, 500, 99)
    steps = H.wide_trace(reqs, late="late")
    mixed = steps[-3]["entries"]
    assert len(mixed) == 61 and sum(len(e["tokens"]) == 1 for e in mixed) == 60 and len(mixed[-1]["tokens"]) == 40
    eng = H.make_engine(d, dtype, kv_tokens=H.tokens_held(steps), max_num_seqs=61)
    H.check_trace_against_plain(eng, d, dtype, reqs, steps, f"D {dtype} 60 decoded tokens beside a portion of 40")


@pytest.mark.parametrize("width", [8, 16, 40, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_of_wide_batches_equal_eager_steps(tmp_path, width, dtype):
    """The graphs of batch 8 to 64 (what a served batch replays) against the same steps launched
    kernel by kernel: the same bits, on the first replay and on later ones.  Up to 16 requests a
    graph is captured at the first step of its shape, wider ones at the fourth."""
    d = make_model_dir(tmp_path, "D", std=0.06)
    tail = 4 if width <= 16 else 8
    reqs = wide_requests(width, 500, 50 + width, lo=tail + 2)
    steps = H.wide_trace(reqs, tail=tail)
    out = {}
    for graphs in (True, False):
        eng = H.make_engine(d, dtype, kv_tokens=H.tokens_held(steps), max_num_seqs=width, decode_graphs=graphs)
        out[graphs] = H.replay(eng, steps)
        assert eng.runner.graph_replays == ((tail if width <= 16 else tail - 3) if graphs else 0)
    for r in reqs:
        assert torch.equal(out[True][r], out[False][r]), r


@pytest.mark.parametrize("page_size", [16, 32])
def test_a_mixed_trace_whose_routes_are_near_ties(tmp_path, page_size):
    """Configuration D in bfloat16 with requests among which a token's two best router logits lie
    within a rounding of each other: the engine may route it otherwise than 32-bit arithmetic
    would.  Its picks must still be the best for the rows its router saw, and the logits right
    under those picks."""
    import random

    d = make_model_dir(tmp_path, "D", std=0.06)
    rng = random.Random(10)
    lens = [rng.choice([3, 17, 33, 48, 64, 65, 97, 130, 200]) for _ in range(rng.randint(4, 8))]
    reqs = {f"r{i}": H.random_tokens(n, 500, 1000 + 10 * 10 + i) for i, n in enumerate(lens)}
    steps = H.mixed_trace(reqs, 10)
    held = H.tokens_held(steps)
    eng = H.make_engine(d, "bfloat16", kv_tokens=((held + page_size - 1) // page_size + 4) * page_size, max_num_seqs=4,
                        page_size=page_size)
    H.check_trace_against_plain(eng, d, "bfloat16", reqs, steps, f"D bfloat16 near ties, pages of {page_size}")


@pytest.mark.parametrize("page_size", [32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_page_sizes(model_dir, page_size, dtype):
    """Pages of 32 and 64 positions: the windows' edges, the decode kernel's runs and the prefill
    kernel's chunks then fall inside pages, not on their edges."""
    which, d = model_dir
    if which not in ("B", "D"):
        pytest.skip("two configurations are enough here")
    toks = _requests(which)[-1]
    eng = H.make_engine(d, dtype, kv_tokens=2 * ((len(toks) + page_size - 1) // page_size) * page_size,
                        max_num_seqs=2, page_size=page_size)
    H.check_against_plain(eng, d, dtype, "a", toks, H.changing_portions(len(toks), 5), f"{which} {dtype} pages of {page_size}")
    H.check_against_plain(eng, d, dtype, "b", toks, H.last_decoded(len(toks)), f"{which} {dtype} pages of {page_size}, decoded")
    for g in eng.cache.groups:
        assert g.pool.num_free == g.pool.num_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graph_replays_equal_eager_steps(model_dir, dtype):
    """Decode-only steps replay a captured graph per batch size.  Every replay (the first and later
    ones, with prefill steps, mixed steps, other graphs and a freed request in between) must give
    the bits of the same step launched kernel by kernel."""
    which, d = model_dir
    if which not in ("B", "D"):
        pytest.skip("two configurations are enough here")
    vocab = CONFIGS[which]["vocab_size"]
    toks = {r: H.random_tokens(n, vocab, 900 + i) for i, (r, n) in enumerate((("a", 40), ("b", 30), ("c", 33)))}
    at = {r: 0 for r in toks}

    def take(r, n, want_last=True):
        e = {"id": r, "tokens": toks[r][at[r]:at[r] + n], "want": [n - 1] if want_last else []}
        at[r] += n
        return e

    steps = [{"entries": [take("a", 20)], "end": []}]
    steps += [{"entries": [take("a", 1)], "end": []} for _ in range(3)]                       # batch 1, three replays
    steps += [{"entries": [take("a", 1), take("b", 15)], "end": []}]                           # mixed: launched eagerly
    steps += [{"entries": [take("a", 1), take("b", 1)], "end": []} for _ in range(3)]          # batch 2
    steps += [{"entries": [take("c", 18)], "end": []}]                                         # a prompt alone in between
    steps += [{"entries": [take("a", 1), take("b", 1), take("c", 1)], "end": []} for _ in range(2)]   # batch 3
    steps[-1]["end"] = ["a"]
    steps += [{"entries": [take("c", 1), take("b", 1)], "end": []} for _ in range(2)]          # batch 2 again, other requests
    steps += [{"entries": [take("b", 1)], "end": []} for _ in range(2)]                        # batch 1 again
    steps[-1]["end"] = ["b", "c"]
    for i, st in enumerate(steps):
        st["step"] = i
    out = {}
    for graphs in (True, False):
        eng = H.make_engine(d, dtype, kv_tokens=256, max_num_seqs=4, decode_graphs=graphs)
        out[graphs] = H.replay(eng, steps)
        if graphs:
            graphs_made = eng.runner._graphs
            assert sorted(n for n, _ in graphs_made) == [1, 2, 3] and all(g is not False for g in graphs_made.values()), \
                "decode steps of batch 1, 2 and 3 should each have captured a graph"
            assert eng.runner.graph_replays == 12
    for r in toks:
        assert torch.equal(out[True][r], out[False][r]), r
    # no more graphs are kept than the limit says: the one used longest ago goes, and is captured
    # again when its shape comes back (batch 1 here, after batches 2 and 3)
    from sharpinference_amd.engine import runner as R
    limit = R.MAX_GRAPHS
    R.MAX_GRAPHS = 2
    try:
        eng = H.make_engine(d, dtype, kv_tokens=256, max_num_seqs=4, decode_graphs=True)
        capped = H.replay(eng, steps)
        assert len(eng.runner._graphs) == 2 and eng.runner.graph_replays == 12
    finally:
        R.MAX_GRAPHS = limit
    for r in toks:
        assert torch.equal(capped[r], out[False][r]), r


def test_decode_graphs_follow_the_context(tmp_path):
    """A graph's shapes are fixed at a bound on its requests' contexts, and bounds grow in steps
    of four: a request that decodes across a bound moves on to the next graph, a short one beside
    it is carried along, and every step gives the bits of the same step launched kernel by kernel."""
    from sharpinference_amd.engine import runner as R

    d = make_model_dir(tmp_path, "D", std=0.06, max_position_embeddings=20000)
    first = R.GRAPH_CONTEXT_MIN
    toks = {"long": H.random_tokens(first + 8, 500, 1), "short": H.random_tokens(40, 500, 2)}
    steps = [{"entries": [{"id": "long", "tokens": toks["long"][:first - 6], "want": [first - 7]}], "end": []},
             {"entries": [{"id": "short", "tokens": toks["short"][:30], "want": [29]}], "end": []}]
    for i in range(10):     # contexts first - 5 ... first + 4: the bound is crossed half-way
        steps.append({"entries": [{"id": "long", "tokens": [toks["long"][first - 6 + i]], "want": [0]},
                                  {"id": "short", "tokens": [toks["short"][30 + i]], "want": [0]}], "end": []})
    steps[-1]["end"] = ["long"]
    steps += [{"entries": [{"id": "short", "tokens": [toks["short"][40 - 1]], "want": [0]}], "end": ["short"]}]
    for i, st in enumerate(steps):
        st["step"] = i
    out = {}
    for graphs in (True, False):
        eng = H.make_engine(d, "bfloat16", kv_tokens=first + 128, max_num_seqs=2, decode_graphs=graphs)
        out[graphs] = H.replay(eng, steps)
        if graphs:
            assert sorted(eng.runner._graphs) == [(1, first), (2, first), (2, 4 * first)]
            assert eng.runner.graph_replays == 11
    for r in toks:
        assert torch.equal(out[True][r], out[False][r]), r



@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("prefix", ["", "language_model."])
def test_a_folder_in_the_other_form_against_plain(tmp_path, dtype, prefix):
    """The same model as another tool writes it: text keys nested, rotary base and llama3 scaling
    in ``rope_parameters``, ``layer_types``, a container prefix, experts fused as [E, in, 2 * out]
    and stored [E, in, out].  The engine reads that folder; the plain implementation reads the
    canonical one.  (A reader that dropped ``rope_parameters`` would rotate with another base
    and no scaling: every rotary layer's logits would differ.)"""
    import json
    import os

    d = make_model_dir(tmp_path, "B", std=0.1)
    other = write_other_layout(d, str(tmp_path / "other"), prefix,
                               extra={"vision_model.patch.weight": torch.zeros(3, 5, dtype=torch.bfloat16)} if prefix else ())
    with open(os.path.join(other, "config.json"), "w") as f:
        json.dump(as_other_tools_write_it(CONFIGS["B"]), f)
    toks = H.random_tokens(90, 384, 3)           # crosses three chunk edges of 24
    eng = H.make_engine(other, dtype)
    assert eng.config.rope_scaling is not None and eng.config.rope_scaling.factor == 8.0
    if dtype == "float32":
        H.assert_close_fp32(H.run_cut(eng, "a", toks, H.changing_portions(len(toks), 1)), H.plain_logits(d, toks), "other form")
    else:
        got, picks, seen = H.run_cut(eng, "a", toks, H.last_decoded(len(toks)), with_routes=True)
        H.assert_routes_are_the_best(d, picks, seen, "other form")
        ref = H.plain_logits_routed(d, toks, dict(zip(H.moe_layers_of(d), picks)))
        H.assert_close_bf16(got, ref, "other form", *H.bounds_of(d))
