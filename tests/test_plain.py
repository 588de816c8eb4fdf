"""What pins the plain implementation besides the reference's text: vectors that the reference's
own tests hold, special cases that reduce to library routines, and invariants; each is chosen so
that a plausible mistake (a sign, a pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama4 as P
from tiny_configs import CONFIGS, make_model_dir


def test_rms_norm_vectors():
    """reference: tests/SharpInference.Tests.ForwardPass/PipelineStepTests.cs:214-229;
    tests/SharpInference.Tests.Cpu/CpuBackendTests.cs:163-180."""
    x = torch.tensor([1.0, 2.0, 3.0, 4.0])
    assert torch.allclose(P.rms_norm(x, torch.ones(4), 0.0), x / math.sqrt(7.5))
    y = P.rms_norm(torch.tensor([3.0, 4.0]), torch.tensor([2.0, 0.5]), 1e-5)
    assert torch.allclose(y, torch.tensor([1.6971, 0.5657]), atol=1e-4)
    assert torch.allclose(P.rms_norm(torch.ones(8), torch.ones(8), 1e-6), torch.ones(8), atol=1e-5)
    z = torch.randn(5, 48)
    assert torch.allclose(P.rms_norm(z, torch.ones(48) * 1.3, 1e-5), F.rms_norm(z, (48,), torch.ones(48) * 1.3, 1e-5), atol=1e-6)


def test_l2_head_norm_gives_unit_rms():
    """reference: PipelineStepTests.cs:231-248, 282-302: rms 1, norm sqrt(dim)."""
    x = torch.randn(7, 3, 32) * 5
    y = P.l2_head_norm(x, 1e-6)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(7, 3), atol=1e-4)
    assert torch.allclose(y.norm(dim=-1), torch.full((7, 3), math.sqrt(32)), atol=1e-3)


def test_rope_identity_norm_and_pairing():
    """reference: CpuBackendTests.cs:286-339: position 0 is the identity, pair norms survive;
    interleaved pairing differs from half-split on a hand example."""
    inv = P.rope_inv_freq(8, 10000.0, None)
    x = torch.randn(4, 2, 8)
    assert torch.allclose(P.apply_rope_interleaved(x, torch.zeros(4, dtype=torch.long), inv), x)
    y = P.apply_rope_interleaved(x, torch.tensor([3, 9, 100, 4095]), inv)
    pair = lambda t: t.view(4, 2, 4, 2).norm(dim=-1)  # noqa: E731
    assert torch.allclose(pair(x), pair(y), atol=1e-5)
    e = torch.zeros(1, 1, 8)
    e[0, 0, 0] = 1.0                                    # (x0, x1) = (1, 0) rotates into slots 0 and 1
    r = P.apply_rope_interleaved(e, torch.tensor([1]), inv)
    assert abs(float(r[0, 0, 0]) - math.cos(1.0)) < 1e-6 and abs(float(r[0, 0, 1]) - math.sin(1.0)) < 1e-6
    assert float(r[0, 0, 4:].abs().max()) == 0.0        # a half-split pairing would put sin(1) at slot 4
    assert abs(float(inv[1]) - 10000.0 ** (-2.0 / 8)) < 1e-8


def test_rope_scores_depend_on_distance_only():
    inv = P.rope_inv_freq(16, 500000.0, {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                         "original_max_position_embeddings": 32})
    q, k = torch.randn(1, 1, 16), torch.randn(1, 1, 16)

    def score(m, n):
        return float((P.apply_rope_interleaved(q, torch.tensor([m]), inv) * P.apply_rope_interleaved(k, torch.tensor([n]), inv)).sum())

    assert abs(score(10, 3) - score(110, 103)) < 1e-4 and abs(score(10, 3) - score(3, 10)) > 1e-3


def test_llama3_scaling_edges():
    plain = P.rope_inv_freq(32, 500000.0, None)
    same = P.rope_inv_freq(32, 500000.0, {"factor": 1.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                          "original_max_position_embeddings": 32})
    assert torch.allclose(plain, same)
    huge = P.rope_inv_freq(32, 500000.0, {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                          "original_max_position_embeddings": 10 ** 9})
    assert torch.equal(plain, huge)                     # every wavelength is short: unscaled
    tiny = P.rope_inv_freq(32, 500000.0, {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                          "original_max_position_embeddings": 1})
    assert torch.allclose(tiny, plain / 8.0)            # every wavelength is long: divided by the factor
    mid = P.rope_inv_freq(32, 500000.0, {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                         "original_max_position_embeddings": 32})
    ratio = mid / plain
    assert float(ratio[0]) == 1.0 and abs(float(ratio[-1]) - 0.125) < 1e-6
    assert all(float(ratio[i]) >= float(ratio[i + 1]) - 1e-7 for i in range(15))      # monotone blend


def test_query_temperature():
    pos = torch.arange(0, 100)
    t = P.query_temperature(pos, 32.0, 0.2)
    assert torch.equal(t[:31], torch.ones(31))          # floor((p+1)/32) = 0 below position 31
    assert abs(float(t[31]) - (1 + 0.2 * math.log(2.0))) < 1e-6 and abs(float(t[95]) - (1 + 0.2 * math.log(4.0))) < 1e-6
    assert bool((t[1:] >= t[:-1]).all())


def test_attention_reduces_to_the_library_routine():
    T, nh, nkv, hd = 19, 6, 3, 16
    q, k, v = torch.randn(T, nh, hd), torch.randn(T, nkv, hd), torch.randn(T, nkv, hd)
    pos = torch.arange(T)
    kk, vv = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    lib = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(P.attention(q, k, v, P.attention_mask(pos, None)), lib, atol=1e-5)
    assert torch.allclose(P.attention(q, k, v, P.attention_mask(pos, 64)), lib, atol=1e-5)     # chunk >= length
    own = P.attention(q, k, v, P.attention_mask(pos, 1))                                       # chunk 1: own value
    assert torch.allclose(own, vv, atol=1e-6)
    mask = P.attention_mask(pos, 5)
    blocks = (pos[:, None] // 5 == pos[None, :] // 5) & (pos[None, :] <= pos[:, None])
    assert torch.equal(mask, blocks)
    lib5 = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1), attn_mask=blocks).transpose(0, 1)
    assert torch.allclose(P.attention(q, k, v, mask), lib5, atol=1e-5)
    # a shift of all positions moves chunk edges: only with no chunk is the mask shift-invariant
    assert torch.equal(P.attention_mask(pos + 7, None), P.attention_mask(pos, None))
    assert not torch.equal(P.attention_mask(pos + 2, 5), P.attention_mask(pos, 5))


def test_gate_vectors_and_silu():
    """reference: PipelineStepTests.cs:41-74, 136-149, 155-182; CpuBackendTests.cs:184-281."""
    assert abs(float(P.router_gates(torch.zeros(1, 4), torch.zeros(3, 4))[0, 0]) - 0.5) < 1e-7
    s = P.silu(torch.tensor([1.0, -1.0, 0.0]))
    assert torch.allclose(s, torch.tensor([0.7311, -0.2689, 0.0]), atol=1e-4)
    x = torch.randn(9, 12)
    assert torch.allclose(P.silu(x), F.silu(x), atol=1e-6)
    row = torch.full((16, 1), -2.0)                      # a 16-expert router row: input [1.0], weights = the logits
    row[11, 0] = -0.845                                  # sigmoid(-0.845) = 0.3005
    ids, w = P.router_topk(torch.ones(1, 1), row, 1)
    assert int(ids[0, 0]) == 11 and abs(float(w[0, 0]) - 0.3005) < 1e-3


def test_gelu_tanh_is_the_library_routine_and_only_chosen_by_name(tmp_path):
    """reference: src/SharpInference.Cpu/SimdKernels.cs:4474-4484 (the scalar form) and its tests'
    zero-input case (tests/SharpInference.Tests.ForwardPass/SimdKernelsGemma4Tests.cs:71-90).  The
    formula is the library's tanh GELU; it differs from SiLU (a swapped activation fails) and from
    the erf form; a dense feed-forward with it is the library's."""
    x = torch.linspace(-3, 3, 97)
    assert torch.allclose(P.gelu_tanh(x), F.gelu(x, approximate="tanh"), atol=1e-6)
    assert float(P.gelu_tanh(torch.zeros(1))) == 0.0
    assert float((P.gelu_tanh(x) - P.silu(x)).abs().max()) > 0.1
    assert float((P.gelu_tanh(x) - F.gelu(x)).abs().max()) > 1e-4
    assert P.activation_of({}) is P.silu and P.activation_of({"hidden_act": "gelu_pytorch_tanh"}) is P.gelu_tanh
    with pytest.raises(ValueError):
        P.activation_of({"hidden_act": "relu"})
    n, wg, wu, wd = torch.randn(5, 8), torch.randn(12, 8), torch.randn(12, 8), torch.randn(8, 12)
    want = (F.gelu(n @ wg.T, approximate="tanh") * (n @ wu.T)) @ wd.T
    assert torch.allclose(P.swiglu(n, wg, wu, wd, act=P.gelu_tanh), want, atol=1e-5)


def test_attention_biases_shift_the_projections(tmp_path):
    """reference: src/SharpInference.Engine/ForwardPass.cs:1605-1613, 893: biases are added right
    after their products.  Pinned by what a bias must do: zero biases change nothing; a value bias b_v
    moves every attention output by exactly W_o b_v's share (softmax weights sum to one), i.e. the layer's
    output by W_o (b_v repeated per query head); an output bias adds itself."""
    d = make_model_dir(tmp_path, "A", std=0.1, attention_bias=True)
    c, W = P.read_config(d), {k: v.float() for k, v in P.load_weights(d).items()}
    assert c["attention_bias"] is True
    p = "model.layers.1.self_attn."                  # layer 1 of A has no rotary: v's bias passes straight through
    n = torch.randn(9, c["hidden_size"])
    pos = torch.arange(9)
    zero = dict(W)
    for name in "qkvo":
        zero[p + f"{name}_proj.bias"] = torch.zeros_like(W[p + f"{name}_proj.bias"])
    c0 = {**c, "attention_bias": False}
    base = P.attention_layer(c0, W, 1, n, pos)
    assert torch.equal(P.attention_layer(c, zero, 1, n, pos), base)
    only_v = dict(zero)
    only_v[p + "v_proj.bias"] = W[p + "v_proj.bias"]
    nh, nkv, hd = c["num_attention_heads"], c["num_key_value_heads"], P.head_dim_of(c)
    per_head = W[p + "v_proj.bias"].view(nkv, hd).repeat_interleave(nh // nkv, dim=0).reshape(-1)
    shift = W[p + "o_proj.weight"] @ per_head
    assert torch.allclose(P.attention_layer(c, only_v, 1, n, pos), base + shift, atol=1e-5)
    only_o = dict(zero)
    only_o[p + "o_proj.bias"] = W[p + "o_proj.bias"]
    assert torch.allclose(P.attention_layer(c, only_o, 1, n, pos), base + W[p + "o_proj.bias"], atol=1e-6)
    only_q = dict(zero)
    only_q[p + "q_proj.bias"] = W[p + "q_proj.bias"] * 30
    assert not torch.allclose(P.attention_layer(c, only_q, 1, n, pos), base, atol=1e-3)


def test_router_ties_and_topk_order():
    n = torch.randn(3, 8)
    ids, w = P.router_topk(n, torch.zeros(5, 8), 2)       # all gates 0.5: lowest indices win
    assert ids.tolist() == [[0, 1]] * 3 and torch.allclose(w, torch.full((3, 2), 0.5))
    wr = torch.randn(6, 8)
    ids, w = P.router_topk(n, wr, 3)
    g = P.router_gates(n, wr)
    assert torch.equal(ids, torch.topk(g, 3, dim=-1).indices) and torch.allclose(w, torch.topk(g, 3, dim=-1).values)


def _moe_weights(E, H, I, seed=0, same_experts=False):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g) * 0.3  # noqa: E731
    p = "model.layers.0.feed_forward."
    W = {p + "router.weight": r(E, H), p + "experts.gate_proj": r(E, I, H), p + "experts.up_proj": r(E, I, H),
         p + "experts.down_proj": r(E, H, I), p + "shared_expert.gate_proj.weight": r(I, H),
         p + "shared_expert.up_proj.weight": r(I, H), p + "shared_expert.down_proj.weight": r(H, I)}
    if same_experts:
        for k in ("gate_proj", "up_proj", "down_proj"):
            W[p + "experts." + k][:] = W[p + "experts." + k][0]
    return W, p


def test_moe_special_cases():
    H, I = 12, 20
    n = torch.randn(5, H)
    # one expert: shared(n) + expert(sigmoid * n) through two dense calls
    W, p = _moe_weights(1, H, I)
    c = {"num_experts_per_tok": 1}
    sig = P.router_gates(n, W[p + "router.weight"])
    want = P.swiglu(n, W[p + "shared_expert.gate_proj.weight"], W[p + "shared_expert.up_proj.weight"], W[p + "shared_expert.down_proj.weight"]) \
        + P.swiglu(n * sig, W[p + "experts.gate_proj"][0], W[p + "experts.up_proj"][0], W[p + "experts.down_proj"][0])
    assert torch.allclose(P.moe_layer(c, W, 0, n), want, atol=1e-5)
    # the score goes in before the non-linearity: scaling the output instead gives something else
    # (reference: PipelineStepTests.cs:184-208)
    after = P.swiglu(n, W[p + "shared_expert.gate_proj.weight"], W[p + "shared_expert.up_proj.weight"], W[p + "shared_expert.down_proj.weight"]) \
        + sig * P.swiglu(n, W[p + "experts.gate_proj"][0], W[p + "experts.up_proj"][0], W[p + "experts.down_proj"][0])
    assert float((after - want).abs().max()) > 1e-3
    # zero router: every gate 0.5, expert 0 chosen, input scaled by 0.5
    W, p = _moe_weights(4, H, I, seed=1)
    W[p + "router.weight"].zero_()
    want0 = P.swiglu(n, W[p + "shared_expert.gate_proj.weight"], W[p + "shared_expert.up_proj.weight"], W[p + "shared_expert.down_proj.weight"]) \
        + P.swiglu(n * 0.5, W[p + "experts.gate_proj"][0], W[p + "experts.up_proj"][0], W[p + "experts.down_proj"][0])
    assert torch.allclose(P.moe_layer(c, W, 0, n), want0, atol=1e-5)
    # top-2 without renormalisation: the sum of two single-expert results
    W, p = _moe_weights(5, H, I, seed=2)
    ids, wts = P.router_topk(n, W[p + "router.weight"], 2)
    two = P.moe_layer({"num_experts_per_tok": 2}, W, 0, n)
    shared = P.swiglu(n, W[p + "shared_expert.gate_proj.weight"], W[p + "shared_expert.up_proj.weight"], W[p + "shared_expert.down_proj.weight"])
    acc = shared.clone()
    for t in range(5):
        for j in range(2):
            e = int(ids[t, j])
            acc[t] += P.swiglu(n[t:t + 1] * wts[t, j], W[p + "experts.gate_proj"][e], W[p + "experts.up_proj"][e], W[p + "experts.down_proj"][e])[0]
    assert torch.allclose(two, acc, atol=1e-5)
    assert float(wts.sum(-1).sub(1).abs().min()) > 1e-3   # the two scores do not sum to one
    # identical experts: the route matters only through the score
    W, p = _moe_weights(4, H, I, seed=3, same_experts=True)
    sig = P.router_gates(n, W[p + "router.weight"]).max(dim=-1, keepdim=True).values
    same = shared * 0 + P.swiglu(n, W[p + "shared_expert.gate_proj.weight"], W[p + "shared_expert.up_proj.weight"], W[p + "shared_expert.down_proj.weight"]) \
        + P.swiglu(n * sig, W[p + "experts.gate_proj"][0], W[p + "experts.up_proj"][0], W[p + "experts.down_proj"][0])
    assert torch.allclose(P.moe_layer(c, W, 0, n), same, atol=1e-5)


def test_temperature_touches_only_layers_without_rotary(tmp_path):
    d = make_model_dir(tmp_path, "A", std=0.1)
    c, W = P.read_config(d), {k: v.float() for k, v in P.load_weights(d).items()}
    toks = list(range(3, 40))
    n = torch.randn(len(toks), 64)
    pos = torch.arange(len(toks))
    off = dict(c, attn_scale=0.0)
    assert torch.equal(P.attention_layer(c, W, 0, n, pos), P.attention_layer(off, W, 0, n, pos))          # rotary layer
    assert not torch.equal(P.attention_layer(c, W, 1, n, pos), P.attention_layer(off, W, 1, n, pos))      # the other
    early = dict(c, floor_scale=1000.0)
    assert torch.equal(P.attention_layer(early, W, 1, n, pos), P.attention_layer(off, W, 1, n, pos))      # factor 1 below floor_scale
    # with a chunk covering everything and no temperature, the rotary layer shifts with its positions
    wide = dict(c, attention_chunk_size=4096)
    assert torch.allclose(P.attention_layer(wide, W, 0, n, pos), P.attention_layer(wide, W, 0, n, pos + 64), atol=1e-4)


def test_whole_model_is_causal_and_deterministic(tmp_path):
    d = make_model_dir(tmp_path, "B", std=0.1)
    c, W = P.read_config(d), P.load_weights(d)
    toks = [5, 9, 200, 31, 7, 7, 150, 2, 77, 300, 12, 4]
    full = P.forward(c, W, toks)
    assert torch.allclose(P.forward(c, W, toks[:7]), full[:7], atol=1e-5)
    assert full.shape == (12, CONFIGS["B"]["vocab_size"]) and bool(torch.isfinite(full).all())
    assert float((P.forward(c, W, toks, dtype=torch.float64).float() - full).abs().max()) < 1e-4


def test_sampling_vectors():
    """reference: tests/SharpInference.Tests.ForwardPass/SamplerTests.cs:8-133."""
    assert P.greedy(torch.tensor([1.0, 5.0, 3.0, 5.0])) == 1          # first maximum wins
    assert P.greedy(torch.tensor([-3.0, -1.0, -2.0])) == 1
    logits = torch.tensor([1.0, 2.0, 3.0, 4.0])
    assert P.sample(logits, 0.5, 1e-3) == 3                            # temperature -> 0 peaks
    assert P.sample(logits, 0.999, 1.0, top_k=2) in (2, 3) and P.sample(logits, 1e-6, 1.0, top_k=2) == 2
    assert P.sample(logits, 1e-6, 1.0, top_p=0.5) == 3                  # the nucleus of 0.5 is the top token alone
    assert P.sample(logits, 1e-6, 1.0, min_p=0.9) == 3
    p = torch.softmax(logits, 0)
    assert P.sample(logits, float(p[0]) - 1e-4, 1.0) == 0 and P.sample(logits, float(p[0]) + 1e-4, 1.0) == 1
    counts = [0] * 4
    us = P.uniform_stream(123, 4000)
    assert all(0.0 <= u < 1.0 for u in us) and abs(sum(us) / 4000 - 0.5) < 0.02
    for u in us:
        counts[P.sample(torch.zeros(4), u, 100.0)] += 1
    assert all(850 <= n <= 1150 for n in counts)                       # hot temperature: near uniform
    assert P.uniform_stream(5, 3) == P.uniform_stream(5, 3) and P.uniform_stream(5, 3) != P.uniform_stream(6, 3)


@pytest.mark.parametrize("which,std", [("A", 0.1), ("B", 0.08), ("D", 0.06)])
def test_the_bfloat16_bound_is_what_two_orders_of_summation_differ_by(tmp_path, which, std):
    """The bound that bfloat16 engine runs are held to (helpers.bf16_bounds) against what it is
    derived for: two runs of the plain implementation with the same stores and the same routes,
    one summing in float and one in double.  They must lie within the bound, and not more than
    twenty times below it (else the bound would be loose enough to hide a fault of the size of a
    rounding)."""
    import helpers as H

    d = make_model_dir(tmp_path, which, std=std)
    c, W = P.read_config(d), P.load_weights(d)
    tol_max, tol_rms = H.bounds_of(d)
    worst_rms = worst_max = 0.0
    for seed in range(2):
        toks = H.random_tokens(100, c["vocab_size"], 70 + seed)
        made: dict = {}
        a = P.forward(c, W, toks, store=P.store_bf16, trace=made)
        picks = made["picks"]                 # the float run's own picks, given to the other run
        b = P.forward(c, W, toks, dtype=torch.float64, store=P.store_bf16, routes=picks)
        err = a.double() - b.double()
        rms = b.double().pow(2).mean(dim=-1).sqrt()
        worst_rms = max(worst_rms, float((err.pow(2).mean(dim=-1).sqrt() / rms).max()))
        worst_max = max(worst_max, float((err.abs().max(dim=-1).values / rms).max()))
    assert tol_rms / 20 <= worst_rms <= tol_rms, (worst_rms, tol_rms)
    assert tol_max / 20 <= worst_max <= tol_max, (worst_max, tol_max)


def test_the_router_check_tells_a_worse_pick_from_a_rounding():
    import helpers as H

    torch.manual_seed(0)
    x = torch.randn(6, 64).to(torch.bfloat16).float()
    w = torch.randn(8, 64)
    r = x.double() @ w.double().T
    best = r.topk(2, dim=1).indices.to(torch.int32)
    H.assert_picks_are_the_best(x, w, best, "best")
    H.assert_picks_are_the_best(x, w, best.flip(1), "order does not matter")
    third = r.topk(3, dim=1).indices[:, [0, 2]].to(torch.int32)
    with pytest.raises(AssertionError, match="below the best"):
        H.assert_picks_are_the_best(x, w, third, "third instead of second")
    twice = best.clone()
    twice[:, 1] = twice[:, 0]
    with pytest.raises(AssertionError, match="twice"):
        H.assert_picks_are_the_best(x, w, twice, "twice")
    # two experts with the same weights: either is right
    w[5] = w[2]
    r = x.double() @ w.double().T
    top = r.topk(1, dim=1).indices.to(torch.int32)
    swapped = torch.where(top == 2, torch.full_like(top, 5), top)
    H.assert_picks_are_the_best(x, w, swapped, "a tie")
