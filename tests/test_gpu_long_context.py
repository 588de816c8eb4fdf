"""A context of twenty thousand tokens compared, not only timed: a prompt fed in 4,096-token
portions across five chunk edges, the last tokens decoded one by one from a graph whose bound lies
beyond 16,384, pages behind the chunk given back and used again on the way, and the logits of the
last 64 positions against the plain implementation (whole sequence, no cache; its own code with
its tensors on the GPU, where torch's float32 product takes seconds for what takes minutes on the
host)."""
import os

import pytest
import torch

import helpers as H
import plain_llama4 as P
from tiny_configs import make_model_dir

pytestmark = pytest.mark.gpu

CHUNK = 4096
N_TOKENS = 5 * CHUNK + 210       # positions 0 .. 20,689: edges at 4,096 ... 20,480 are crossed
TAIL = 8                         # decoded one by one
COMPARED = 64


def _sharpened(tmp_path, factor):
    """Configuration D with a chunk of 4,096, a temperature that steps every 2,048 positions (eleven
    values over the run), and the layer without rotary made to look far: its query and key
    projections are scaled by `factor` so that a query's largest scores stand out among twenty
    thousand keys, and a key that is lost, read from a wrong page or masked by mistake moves the
    logits.  The 32-bit run takes 3 (scores nine times as large).  The bfloat16 run takes the
    weights as they are: with sharper scores the softmax's slope outgrows what the bfloat16 bound
    assumes (two plain runs that differ in the order of their sums only lie 0.04 of a row's rms
    apart at factor 1, 0.09 at 2 and 0.11 at 3, against a bound of 0.066: measured on the CPU over
    3,000 tokens), so a sharpened model would need a wider bound, which would hide more."""
    from safetensors.torch import load_file, save_file

    d = make_model_dir(tmp_path, "D", std=0.06, max_position_embeddings=24576, attention_chunk_size=CHUNK,
                       floor_scale=2048.0)
    path = os.path.join(d, "model.safetensors")
    W = load_file(path)
    for name in ("q_proj", "k_proj"):
        key = f"model.layers.1.self_attn.{name}.weight"
        W[key] = (W[key].float() * factor).to(W[key].dtype)
    save_file(W, path)
    return d


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_twenty_thousand_tokens_against_plain(tmp_path, dtype):
    d = _sharpened(tmp_path, 3.0 if dtype == "float32" else 1.0)
    c = P.read_config(d)
    assert P.layer_uses_rope(c, 0) and not P.layer_uses_rope(c, 1)
    toks = H.random_tokens(N_TOKENS, c["vocab_size"], 77)
    n_prompt = N_TOKENS - TAIL
    steps, at = [], 0
    while at < n_prompt:
        take = min(CHUNK, n_prompt - at)
        last = at + take == n_prompt
        want = list(range(take - (COMPARED - TAIL), take)) if last else []
        steps.append({"step": len(steps), "entries": [{"id": "long", "tokens": toks[at:at + take], "want": want}], "end": []})
        at += take
    assert len(steps[-1]["entries"][0]["want"]) == COMPARED - TAIL
    for i in range(TAIL):
        steps.append({"step": len(steps), "entries": [{"id": "long", "tokens": [toks[n_prompt + i]], "want": [0]}], "end": []})
    steps[-1]["end"] = ["long"]
    eng = H.make_engine(d, dtype, kv_tokens=N_TOKENS + 64, max_num_seqs=1, max_tokens_per_step=CHUNK)
    with_routes = dtype == "bfloat16"
    out = H.replay(eng, steps, with_routes=with_routes)
    got = (out[0] if with_routes else out)["long"]
    assert got.shape == (COMPARED, c["vocab_size"])

    # the plain implementation over the whole sequence, its tensors on the GPU
    Wg = {k: (v.float() if v.is_floating_point() else v).to("cuda:0") for k, v in P.load_weights(d).items()}
    if dtype == "float32":
        ref = P.forward(c, Wg, toks)[-COMPARED:].cpu()
        H.assert_close_fp32(got, ref, "long context, 32-bit")
    else:
        _, picks, seen = out
        H.assert_routes_are_the_best(d, picks["long"], seen["long"], "long context")
        routes = dict(zip(H.moe_layers_of(d), picks["long"]))
        ref = P.forward(c, Wg, toks, store=P.store_bf16, routes=routes)[-COMPARED:].cpu()
        H.assert_close_bf16(got, ref, "long context, bfloat16", *H.bounds_of(d))
    # the far keys count: the same tokens with the first chunk's tokens changed give other logits
    # at the end in the layer that sees every key (a kernel that dropped far keys would not notice)
    other = list(toks)
    other[:CHUNK] = H.random_tokens(CHUNK, c["vocab_size"], 78)
    moved = P.forward(c, Wg, other)[-COMPARED:].cpu() if dtype == "float32" else None
    if moved is not None:
        assert float((moved - ref).abs().max()) > 50 * H.fp32_tol(ref)

    # pages behind the chunk were given back and used again; pages of the layer that sees all stayed
    windowed = [g for g in eng.cache.groups if g.spec.window_kind != 0]
    full = [g for g in eng.cache.groups if g.spec.window_kind == 0]
    assert windowed and full
    for g in windowed:
        assert g.pool.num_pages < (N_TOKENS + 15) // 16, "the chunked layers' pool holds every key: nothing had to be reused"
        assert g.pool.total_allocs > g.pool.num_pages, "no page of the chunked layers was used twice"
    for g in full:
        assert g.pool.total_allocs >= (N_TOKENS + 15) // 16
    assert all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    # the decoded tokens came from a graph whose bound lies beyond 16,384 contexts
    bounds = sorted(k[1] for k in eng.runner._graphs)
    assert bounds and bounds[-1] > 16384 and eng.runner.graph_replays >= TAIL - 1, (bounds, eng.runner.graph_replays)
