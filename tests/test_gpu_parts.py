"""Each part alone, the arrangement of layers as data, and a toy mixer with state of its own."""
import math
from dataclasses import dataclass

import pytest
import torch

import helpers as H
import plain_llama4 as P
from tiny_configs import make_model_dir

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ctx(entries, page_size=16, dtype=torch.float32, totals=None):
    """A StepContext for requests given as (start position, tokens in this step), each with its
    own pages in one group (`totals`: final lengths, so that pages stay put from step to step)."""
    from sharpinference_amd.ops import PREFILL_TILE_TOKENS as TILE
    from sharpinference_amd.parts.base import GroupView, StepContext

    T = sum(n for _, n in entries)
    pos, ent, slots, tables, cu = [], [], [], [], [0]
    page = 0
    for i, (start, n) in enumerate(entries):
        nb = ((totals[i] if totals else start + n) + page_size - 1) // page_size
        tbl = list(range(page, page + nb))
        page += nb
        tables.append(tbl)
        for p in range(start, start + n):
            pos.append(p)
            ent.append(i)
            slots.append(tbl[p // page_size] * page_size + p % page_size)
        cu.append(cu[-1] + n)
    maxb = max(len(t) for t in tables)
    bt = torch.full((len(entries), maxb), -1, dtype=torch.int32)
    for i, t in enumerate(tables):
        bt[i, :len(t)] = torch.tensor(t, dtype=torch.int32)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)  # noqa: E731
    g = GroupView(bt.to(DEV), i32(slots), page_size, max_context=max(pos) + 1)
    lens = [n for _, n in entries]
    dec = [cu[i] for i, n in enumerate(lens) if n == 1]
    tiles = [(i, cu[i] + o, min(TILE, n - o)) for i, n in enumerate(lens) if n > 1 for o in range(0, n, TILE)]
    ctx = StepContext(n_tokens=T, n_entries=len(entries), token_ids=i32([0] * T), positions=i32(pos), entry_of_token=i32(ent),
                      cu_tokens=i32(cu), state_slots=i32(list(range(len(entries)))), groups=[g], act_dtype=dtype,
                      no_store_slots=i32([-1] * T), entry_lens=lens, entry_starts=[s for s, _ in entries],
                      max_entry_len=max(lens), n_decode=len(dec), decode_tokens=None if len(dec) == T else i32(dec),
                      n_prefill_tiles=len(tiles), prefill_tiles=i32(tiles).view(-1, 3) if tiles else None)
    return ctx, page


class _Dict:
    where = "test"

    def __init__(self, tensors, dtype):
        self.t, self.dtype = tensors, dtype

    def get(self, name):
        return self.t[name].to(self.dtype).to(DEV)


def test_norm_part():
    from sharpinference_amd.parts.base import ResidualStream
    from sharpinference_amd.parts.norm import RMSNorm

    h = torch.randn(9, 80)
    delta = torch.randn(9, 80)
    w = torch.rand(80) + 0.5
    part = RMSNorm(80, 1e-4)
    part.load("n.", _Dict({"n.weight": w}, torch.float32))
    stream = ResidualStream(h.clone().to(DEV))
    stream.pending = delta.to(DEV)
    out = part.forward(stream, torch.float32).cpu()
    assert torch.allclose(out, P.rms_norm(h + delta, w, 1e-4), atol=1e-5)
    assert stream.pending is None and torch.allclose(stream.h.cpu(), h + delta)
    rows = torch.tensor([7, 2], dtype=torch.int32, device=DEV)
    stream.pending = delta.to(DEV)
    some = part.forward(stream, torch.float32, rows=rows).cpu()
    assert torch.allclose(some, P.rms_norm(h + 2 * delta, w, 1e-4)[[7, 2]], atol=1e-5)
    assert stream.pending is not None and torch.allclose(stream.h.cpu(), h + delta)   # gathered rows leave the stream alone
    bare = RMSNorm(80, 1e-4, has_weight=False)
    stream.pending = None
    assert torch.allclose(bare.forward(stream, torch.float32).cpu(), P.l2_head_norm(h + delta, 1e-4), atol=1e-5)


def test_rotary_table_matches_plain():
    from sharpinference_amd.config.llama4 import RopeScaling
    from sharpinference_amd.parts.position import RotaryInterleaved

    sc = {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 32}
    for hd, theta, s in ((16, 10000.0, None), (32, 500000.0, sc), (128, 500000.0, dict(sc, factor=16.0, original_max_position_embeddings=8192))):
        part = RotaryInterleaved(hd, theta, RopeScaling(**{"rope_type": "llama3", **s}) if s else None)
        assert torch.equal(part.frequencies(), P.rope_inv_freq(hd, theta, s))


@pytest.mark.parametrize("layer,dtype", [(0, torch.float32), (1, torch.float32), (0, torch.bfloat16), (1, torch.bfloat16)])
def test_attention_part_alone(tmp_path, layer, dtype):
    """The mixer with a cache of its own: a prompt in two portions for one request beside single
    tokens for two others, against the plain layer on the whole sequences.  Layer 0 of tiny B has
    rotary and a chunk of 24, layer 3 (here: index 1) has neither but the temperature."""
    from sharpinference_amd import build_model, load_config
    from sharpinference_amd.parts.base import LayerCache
    from sharpinference_amd.weights.loader import SafetensorsSource

    d = make_model_dir(tmp_path, "B", std=0.1)
    lay = [0, 3][layer]
    c, W = P.read_config(d), {k: v.float() for k, v in P.load_weights(d).items()}
    model = build_model(load_config(d))
    mixer = model.blocks[lay].mixer
    mixer.load(f"model.layers.{lay}.self_attn.", SafetensorsSource(d, dtype, DEV))
    lens = [61, 30, 47]
    xs = [torch.randn(L, 96).to(torch.bfloat16).float() for L in lens]
    store = P.store_bf16 if dtype == torch.bfloat16 else P._same
    want = [P.attention_layer(c, W, lay, x, torch.arange(L), store) for x, L in zip(xs, lens)]
    spec = mixer.cache_spec()
    k = torch.zeros(16, spec.num_kv_heads, 16, spec.head_dim, dtype=dtype, device=DEV)
    v = torch.zeros(16, spec.num_kv_heads, spec.head_dim, 16, dtype=dtype, device=DEV)
    # step 1: the three requests' first parts; step 2: request 0 goes on with 21 tokens, the others decode one token
    first = [40, 29, 46]
    done = [0, 0, 0]
    outs = [[], [], []]
    for sizes in (first, [21, 1, 1]):
        ctx, pages = _ctx([(done[i], sizes[i]) for i in range(3)], dtype=dtype, totals=lens)
        assert pages <= 16
        x = torch.cat([xs[i][done[i]:done[i] + sizes[i]] for i in range(3)]).to(dtype).to(DEV)
        out = mixer.forward(x, ctx, LayerCache(ctx.groups[0], k, v)).float().cpu()
        o = 0
        for i in range(3):
            outs[i].append(out[o:o + sizes[i]])
            o += sizes[i]
            done[i] += sizes[i]
    for i in range(3):
        got = torch.cat(outs[i])
        tol = 1e-4 if dtype == torch.float32 else 3e-2
        assert float((got - want[i]).abs().max()) <= tol * max(1.0, float(want[i].abs().max())), (i, lay)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window_kind,window", [(0, 0), (2, 20)])
def test_attention_part_with_values_of_another_width_than_keys(dtype, window_kind, window):
    """A mixer whose values (and heads' outputs) are 24 wide beside keys of 48: its cache holds V
    [page, kv head, 24, position], the projections take the widths from it, and the result is the
    library's attention on unrotated, unnormed q and k (softmax(q k^T / sqrt(48)) v per head, kv
    heads repeated), for a prompt portion beside two decode tokens."""
    from sharpinference_amd.parts.attention import Attention
    from sharpinference_amd.parts.base import LayerCache

    H, nh, nkv, hd, vd = 80, 4, 2, 48, 24
    mixer = Attention(H, nh, nkv, hd, window_kind=window_kind, window=window, v_head_dim=vd)
    spec = mixer.cache_spec()
    assert spec.value_dim == vd and spec.head_dim == hd
    specs = mixer.param_specs("a.")
    assert specs["a.v_proj.weight"].shape == (nkv * vd, H) and specs["a.o_proj.weight"].shape == (H, nh * vd)
    g = torch.Generator().manual_seed(3)
    W = {n: (torch.randn(*sp.shape, generator=g) * 0.2).to(torch.bfloat16).float() for n, sp in specs.items()}
    mixer.load("a.", _Dict(W, dtype))
    lens = [37, 30, 45]
    xs = [torch.randn(L, H, generator=g).to(torch.bfloat16).float() for L in lens]
    store = P.store_bf16 if dtype == torch.bfloat16 else P._same

    def plain(x):
        L = x.shape[0]
        q = store(x @ W["a.q_proj.weight"].T).view(L, nh, hd).transpose(0, 1)
        k = store(x @ W["a.k_proj.weight"].T).view(L, nkv, hd).transpose(0, 1).repeat_interleave(nh // nkv, 0)
        v = store(x @ W["a.v_proj.weight"].T).view(L, nkv, vd).transpose(0, 1).repeat_interleave(nh // nkv, 0)
        pos = torch.arange(L)
        mask = pos[None, :] <= pos[:, None]
        if window_kind == 2:
            mask = mask & (pos[None, :] > pos[:, None] - window)
        o = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=hd ** -0.5)
        return store(store(o.transpose(0, 1).reshape(L, nh * vd)) @ W["a.o_proj.weight"].T)

    want = [plain(x) for x in xs]
    k = torch.zeros(12, nkv, 16, hd, dtype=dtype, device=DEV)
    v = torch.zeros(12, nkv, vd, 16, dtype=dtype, device=DEV)
    done, outs = [0, 0, 0], [[], [], []]
    for sizes in ([20, 29, 44], [17, 1, 1]):
        ctx, pages = _ctx([(done[i], sizes[i]) for i in range(3)], dtype=dtype, totals=lens)
        assert pages <= 12
        x = torch.cat([xs[i][done[i]:done[i] + sizes[i]] for i in range(3)]).to(dtype).to(DEV)
        out = mixer.forward(x, ctx, LayerCache(ctx.groups[0], k, v)).float().cpu()
        o = 0
        for i in range(3):
            outs[i].append(out[o:o + sizes[i]])
            o += sizes[i]
            done[i] += sizes[i]
    for i in range(3):
        tol = 1e-4 if dtype == torch.float32 else 3e-2
        assert float((torch.cat(outs[i]) - want[i]).abs().max()) <= tol * max(1.0, float(want[i].abs().max())), i


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_parts_alone(tmp_path, dtype):
    from sharpinference_amd import build_model, load_config
    from sharpinference_amd.weights.loader import SafetensorsSource

    d = make_model_dir(tmp_path, "B", std=0.1)
    c, W = P.read_config(d), {k: v.float() for k, v in P.load_weights(d).items()}
    model = build_model(load_config(d))
    src = SafetensorsSource(d, dtype, DEV)
    x = torch.randn(70, 96).to(torch.bfloat16).float()
    ctx, _ = _ctx([(0, 70)], dtype=dtype)
    store = P.store_bf16 if dtype == torch.bfloat16 else P._same
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    dense = model.blocks[0].ffn
    dense.load("model.layers.0.feed_forward.", src)
    got = dense.forward(x.to(dtype).to(DEV), ctx).float().cpu()
    want = P.dense_layer(c, W, 0, x, store)
    assert float((got - want).abs().max()) <= tol * float(want.abs().max())
    moe = model.blocks[1].ffn
    moe.load("model.layers.1.feed_forward.", src)
    trace = []
    ctx.extras["router_trace"] = trace
    # the routed feed-forward leaves its output as a sum for the next norm to form (with many rows:
    # the experts' rows and the shared expert's; with a few rows in bfloat16 the shared expert is one
    # more group of the experts' launches); formed by the norm kernel or by the combine kernel it is
    # the same bits
    from sharpinference_amd import ops
    from sharpinference_amd.parts.base import ResidualStream
    from sharpinference_amd.parts.norm import RMSNorm
    norm = RMSNorm(96, 1e-5)
    norm.weight = torch.rand(96, device=DEV) + 0.5
    for n_rows in (70, 5):
        ctxn, _ = _ctx([(0, n_rows)], dtype=dtype)
        trace = []
        ctxn.extras["router_trace"] = trace
        out = moe.forward(x[:n_rows].to(dtype).to(DEV), ctxn)
        assert isinstance(out, ops.ExpertSum)
        got = out.tensor().float().cpu()
        want = P.moe_layer(c, W, 1, x[:n_rows], None, store, routes={1: trace[0][0].cpu()} if dtype == torch.bfloat16 else None)
        assert float((got - want).abs().max()) <= tol * float(want.abs().max())
        h0 = torch.randn(n_rows, 96, device=DEV)
        rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
        for r in (None, rows):
            a, b = ResidualStream(h0.clone()), ResidualStream(h0.clone())
            a.pending, b.pending = out, out.tensor()
            na, nb = norm.forward(a, dtype, rows=r), norm.forward(b, dtype, rows=r)
            assert torch.equal(na, nb) and torch.equal(a.h, b.h)
            assert torch.equal(a.pending_tensor(), b.pending) if r is not None else a.pending is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_feed_forwards_take_another_activation(dtype):
    """The gate's function is an argument of the feed-forward parts (a code the kernels take: in
    the activation kernel and in the epilogues of the few-rows and many-rows products alike): GELU
    in its tanh form, dense and routed, with few rows and with many, against the formula."""
    from sharpinference_amd import ops
    from sharpinference_amd.parts.feedforward import DenseSwiGLU, MoESwiGLU

    HID, INTER, E = 128, 128, 4
    g = torch.Generator().manual_seed(11)
    rnd = lambda *shape: (torch.randn(*shape, generator=g) * 0.1).to(torch.bfloat16).float()  # noqa: E731
    W = {"d.gate_proj.weight": rnd(INTER, HID), "d.up_proj.weight": rnd(INTER, HID), "d.down_proj.weight": rnd(HID, INTER),
         "m.router.weight": rnd(E, HID) * 10, "m.experts.gate_proj": rnd(E, INTER, HID), "m.experts.up_proj": rnd(E, INTER, HID),
         "m.experts.down_proj": rnd(E, HID, INTER), "m.shared_expert.gate_proj.weight": rnd(INTER, HID),
         "m.shared_expert.up_proj.weight": rnd(INTER, HID), "m.shared_expert.down_proj.weight": rnd(HID, INTER)}
    src = _Dict(W, dtype)
    with pytest.raises(ValueError, match="not known"):
        DenseSwiGLU(HID, INTER, activation="relu6")
    dense = DenseSwiGLU(HID, INTER, activation="gelu_tanh")
    dense.load("d.", src)
    moe = MoESwiGLU(HID, E, 1, INTER, shared_intermediate=INTER, activation="gelu_tanh")
    moe.load("m.", src)
    store = P.store_bf16 if dtype == torch.bfloat16 else P._same
    gelu = lambda v: torch.nn.functional.gelu(v, approximate="tanh")  # noqa: E731

    def unit(x, wg, wu, wd, s=None):
        gg, uu = store(x @ wg.T), store(x @ wu.T)
        if s is not None:
            gg, uu = gg * s[:, None], uu * s[:, None]
        return store(store(gelu(gg) * uu) @ wd.T)

    tol = 1e-4 if dtype == torch.float32 else 3e-2
    x_all = torch.randn(200, HID, generator=g).to(torch.bfloat16).float()
    for n_rows in (200, 70, 5):       # many rows, some, a few (the picked form in bfloat16)
        x = x_all[:n_rows]
        ctx, _ = _ctx([(0, n_rows)], dtype=dtype)
        got = dense.forward(x.to(dtype).to(DEV), ctx).float().cpu()
        want = unit(x, W["d.gate_proj.weight"], W["d.up_proj.weight"], W["d.down_proj.weight"])
        assert float((got - want).abs().max()) <= tol * float(want.abs().max()), (n_rows, "dense")
        trace = []
        ctx.extras["router_trace"] = trace
        got = moe.forward(x.to(dtype).to(DEV), ctx).tensor().float().cpu()
        ids = trace[0][0].cpu().long()[:, 0]                 # the experts the router took (its own choice in both dtypes)
        score = torch.sigmoid((x @ W["m.router.weight"].T).gather(1, ids[:, None]))[:, 0]
        want = unit(x, W["m.shared_expert.gate_proj.weight"], W["m.shared_expert.up_proj.weight"], W["m.shared_expert.down_proj.weight"])
        for e in range(E):
            rows = (ids == e).nonzero().flatten()
            if rows.numel():
                want[rows] = store(want[rows] + unit(x[rows], W["m.experts.gate_proj"][e], W["m.experts.up_proj"][e],
                                                     W["m.experts.down_proj"][e], score[rows]))
        assert float((got - want).abs().max()) <= tol * float(want.abs().max()), (n_rows, "routed")
    # the activation kernel alone, both codes
    gu = torch.randn(9, 2 * 40, generator=g).to(DEV)
    assert torch.allclose(ops.gated_act(gu, None, ops.ACT_GELU_TANH).cpu(), gelu(gu[:, :40].cpu()) * gu[:, 40:].cpu(), atol=1e-6)
    assert torch.equal(ops.gated_act(gu, None, ops.ACT_SILU), ops.silu_mul(gu))


def test_schedule_runs_a_layer_twice_and_shares_a_cache(tmp_path):
    """The order of execution is data: layer 0 runs twice (two cache slots), and the second run of
    layer 1 reads the keys and values that its first run stored."""
    from sharpinference_amd import load_config
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.parts.model import Run
    from sharpinference_amd.registry import register_architecture, unregister_architecture
    from sharpinference_amd.config.llama4 import Llama4TextConfig
    from sharpinference_amd.models.llama4 import build_llama4

    def build(cfg):
        m = build_llama4(cfg)
        m.schedule = [Run(0, 0), Run(1, 1), Run(0, 2), Run(1, 1, write=False)]
        m._check_schedule()
        return m

    register_architecture("LoopedLlama4ForTest", Llama4TextConfig, build, replace=True)
    try:
        d = make_model_dir(tmp_path, "A", std=0.1)
        cfg = load_config(d)
        cfg.architecture = "LoopedLlama4ForTest"
        import json, os
        json.dump(cfg.to_dict(), open(os.path.join(d, "config.json"), "w"))
        eng = Engine(d, dtype="float32", kv_tokens=256, max_num_seqs=2)
        assert len(eng.cache.slot_specs) == 3
        toks = H.random_tokens(45, 256, 3)
        got = H.run_cut(eng, "x", toks, [20, 1, 1, 13, 10])
        c, W = P.read_config(d), {k: v.float() for k, v in P.load_weights(d).items()}
        eps, pos = c["rms_norm_eps"], torch.arange(45)
        h = W["model.embed_tokens.weight"][torch.tensor(toks)]
        kv1 = []
        for lay, kv_out, kv_in in ((0, None, None), (1, kv1, None), (0, None, None), (1, None, "shared")):
            p = f"model.layers.{lay}."
            n = P.rms_norm(h, W[p + "input_layernorm.weight"], eps)
            h = h + P.attention_layer(c, W, lay, n, pos, kv_out=kv_out, kv_in=kv1[0] if kv_in else None)
            n = P.rms_norm(h, W[p + "post_attention_layernorm.weight"], eps)
            h = h + P.moe_layer(c, W, lay, n)
        want = P.rms_norm(h, W["model.norm.weight"], eps) @ W["lm_head.weight"].T
        H.assert_close_fp32(got, want, "looped schedule")
    finally:
        unregister_architecture("LoopedLlama4ForTest")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_scale_and_logit_scale_and_cap_are_arguments_of_the_model(tmp_path, dtype):
    """An architecture that scales its embeddings, scales its logits or caps them softly gives the
    decoder model three numbers; nothing else changes.  Against the plain functions: the embedding
    rows times the scale before the first layer, and cap * tanh(scale * logits / cap) behind the head
    (reference: src/SharpInference.Engine/ForwardPass.cs:1482-1483, src/SharpInference.Cpu/SimdKernels.cs:4490-4530)."""
    from sharpinference_amd import load_config
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.registry import register_architecture, unregister_architecture
    from sharpinference_amd.config.llama4 import Llama4TextConfig
    from sharpinference_amd.models.llama4 import build_llama4

    SCALE, LSCALE, CAP = 3.5, 1.5, 2.0

    def build(cfg):
        m = build_llama4(cfg)
        m.embedding_scale, m.logit_scale, m.logit_softcap = SCALE, LSCALE, CAP
        return m

    register_architecture("ScaledLlama4ForTest", Llama4TextConfig, build, replace=True)
    try:
        d = make_model_dir(tmp_path, "A", std=0.1)
        cfg = load_config(d)
        cfg.architecture = "ScaledLlama4ForTest"
        import json, os
        json.dump(cfg.to_dict(), open(os.path.join(d, "config.json"), "w"))
        eng = Engine(d, dtype=dtype, kv_tokens=256, max_num_seqs=2)
        toks = H.random_tokens(40, 256, 5)
        got = H.run_cut(eng, "x", toks, [25, 1, 1, 13])
        c, W = P.read_config(d), {k: v.float() for k, v in P.load_weights(d).items()}
        store = P.store_bf16 if dtype == "bfloat16" else P._same
        eps, pos = c["rms_norm_eps"], torch.arange(40)
        h = W["model.embed_tokens.weight"][torch.tensor(toks)] * SCALE
        for lay in range(c["num_hidden_layers"]):
            p = f"model.layers.{lay}."
            n = store(P.rms_norm(h, W[p + "input_layernorm.weight"], eps))
            h = h + P.attention_layer(c, W, lay, n, pos, store)
            n = store(P.rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))
            h = h + P.moe_layer(c, W, lay, n, store=store)
        raw = store(P.rms_norm(h, W["model.norm.weight"], eps)) @ W["lm_head.weight"].T
        want = CAP * torch.tanh(raw * LSCALE / CAP)
        assert float(raw.abs().max()) * LSCALE > 0.5 * CAP        # the cap bites
        if dtype == "float32":
            H.assert_close_fp32(got, want, "scaled model")
        else:
            H.assert_close_bf16(got, want, "scaled model", *H.bounds_of(d))
        # ... and they do something: the same folder as the plain architecture gives other logits
        plain_eng = H.make_engine(make_model_dir(tmp_path / "plain", "A", std=0.1), dtype, kv_tokens=256, max_num_seqs=2)
        assert float((H.run_cut(plain_eng, "y", toks, [40]) - got).abs().max()) > 0.1
    finally:
        unregister_architecture("ScaledLlama4ForTest")


def test_toy_mixer_with_state_needs_no_change_to_the_framework():
    """A mixer defined here, with per-request state of fixed size (a running sum and a count),
    is registered, built and stepped through the ordinary engine."""
    from sharpinference_amd.cache.spec import StateSpec
    from sharpinference_amd.config.base import ModelConfig
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.parts.base import Part
    from sharpinference_amd.parts.block import PreNormBlock
    from sharpinference_amd.parts.feedforward import DenseSwiGLU
    from sharpinference_amd.parts.model import DecoderModel
    from sharpinference_amd.parts.norm import RMSNorm
    from sharpinference_amd.registry import register_architecture, unregister_architecture

    @dataclass
    class ToyConfig(ModelConfig):
        architecture: str = "ToyRunningMean"
        hidden_size: int = 32
        layers: int = 2
        vocab_size: int = 50
        max_position_embeddings: int = 256

        @classmethod
        def from_dict(cls, d):
            return cls(hidden_size=d["hidden_size"], layers=d["layers"], vocab_size=d["vocab_size"])

        def to_dict(self):
            return {"architectures": [self.architecture], "hidden_size": self.hidden_size, "layers": self.layers,
                    "vocab_size": self.vocab_size}

    class RunningMean(Part):
        """out[t] = mean of the inputs of positions 0..t; state per request: [sum (H), count]."""

        def __init__(self, hidden):
            self.hidden = hidden

        def cache_spec(self):
            return StateSpec((self.hidden + 1,), torch.float32)

        def forward(self, x, ctx, cache):
            out = torch.empty_like(x)
            o = 0
            slots = ctx.state_slots.cpu().tolist()
            for e, n in enumerate(ctx.entry_lens):
                st = cache.state[slots[e]]
                cs = torch.cumsum(x[o:o + n].float(), 0) + st[:-1]
                cnt = st[-1] + torch.arange(1, n + 1, device=x.device)
                out[o:o + n] = (cs / cnt[:, None]).to(x.dtype)
                st[:-1] = cs[-1]
                st[-1] = cnt[-1]
                o += n
            return out

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(cfg.hidden_size, 1e-5), RunningMean(cfg.hidden_size), RMSNorm(cfg.hidden_size, 1e-5),
                               DenseSwiGLU(cfg.hidden_size, 48), names={"norm1": "n1.", "mixer": "mix.", "norm2": "n2.", "ffn": "ff."})
                  for _ in range(cfg.layers)]
        return DecoderModel(cfg.vocab_size, cfg.hidden_size, blocks, RMSNorm(cfg.hidden_size, 1e-5), config=cfg)

    register_architecture("ToyRunningMean", ToyConfig, build, replace=True)
    try:
        eng = Engine(config=ToyConfig(), weight_seed=7, dtype="float32", kv_tokens=64, max_num_seqs=3, weight_std=0.3)
        assert eng.cache.groups == [] and eng.cache.state[0].shape == (3 + 1, 33)      # a slot per request and the scratch slot
        a, b = H.random_tokens(40, 50, 1), H.random_tokens(25, 50, 2)
        whole_a = H.run_cut(eng, "a", a, [40])
        whole_b = H.run_cut(eng, "b", b, [25])
        # the same two requests interleaved, in portions and single tokens; a third takes and frees a slot between
        steps = H.mixed_trace({"a": a, "b": b, "c": H.random_tokens(9, 50, 3)}, seed=2, max_live=3, tail=6)
        got = H.replay(eng, steps)
        assert float((got["a"] - whole_a).abs().max()) <= 1e-4 and float((got["b"] - whole_b).abs().max()) <= 1e-4
        # and against the formula itself
        m = eng.model
        h = m.embed[torch.tensor(a, device=DEV)].float()
        for blk in m.blocks:
            n = P.rms_norm(h, blk.norm1.weight, 1e-5)
            h = h + torch.cumsum(n, 0) / torch.arange(1, 41, device=DEV)[:, None]
            n = P.rms_norm(h, blk.norm2.weight, 1e-5)
            gu = n @ blk.ffn.w_gate_up.T
            h = h + (P.silu(gu[:, :48]) * gu[:, 48:]) @ blk.ffn.w_down.T
        want = P.rms_norm(h, m.final_norm.weight, 1e-5) @ m.head.T
        assert float((whole_a - want.cpu()).abs().max()) <= 1e-4
    finally:
        unregister_architecture("ToyRunningMean")


def test_toy_position_encoding_and_routed_feed_forward_need_no_change_to_the_framework():
    """Two more parts defined here: a learned absolute position encoding (added to the mixer's
    input, around an attention without rotation) and a feed-forward that routes by position
    (expert = position mod E, no router weights), built from the framework's routing and
    grouped-product operations.  Registered, built, stepped whole, cut and mixed."""
    from sharpinference_amd import ops
    from sharpinference_amd.config.base import ModelConfig
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.parts.attention import Attention
    from sharpinference_amd.parts.base import ParamSpec, Part
    from sharpinference_amd.parts.block import PreNormBlock
    from sharpinference_amd.parts.model import DecoderModel
    from sharpinference_amd.parts.norm import RMSNorm
    from sharpinference_amd.registry import register_architecture, unregister_architecture

    HID, NH, NKV, HD, E, INTER, MAXPOS, VOCAB = 32, 2, 1, 16, 3, 40, 128, 60

    @dataclass
    class ToyConfig(ModelConfig):
        architecture: str = "ToyLearnedPositions"
        vocab_size: int = VOCAB
        max_position_embeddings: int = MAXPOS

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": [self.architecture]}

    class LearnedPositions(Part):
        """mixer(x + table[position]): a position encoding as a part around any mixer."""

        def __init__(self, inner, hidden, max_pos):
            self.inner, self.hidden, self.max_pos = inner, hidden, max_pos

        def param_specs(self, prefix):
            out = {prefix + "positions.weight": ParamSpec((self.max_pos, self.hidden))}
            out.update(self.inner.param_specs(prefix))
            return out

        def load(self, prefix, source):
            self.table = source.get(prefix + "positions.weight")
            self.inner.load(prefix, source)

        def cache_spec(self):
            return self.inner.cache_spec()

        def forward(self, x, ctx, cache):
            return self.inner.forward((x + self.table[ctx.positions.long()].to(x.dtype)), ctx, cache)

    class RoutedByPosition(Part):
        """Expert (position mod E) of E SwiGLU experts: routing without a router."""

        def param_specs(self, prefix):
            return {prefix + "gate_up": ParamSpec((E, 2 * INTER, HID)), prefix + "down": ParamSpec((E, HID, INTER))}

        def load(self, prefix, source):
            self.w_gate_up, self.w_down = source.get(prefix + "gate_up"), source.get(prefix + "down")

        def forward(self, x, ctx):
            T = x.shape[0]
            ids = (ctx.positions % E).to(torch.int32).view(T, 1)
            rt = ops.moe_permute(ids, torch.ones(T, 1, device=x.device), E)
            act = ops.grouped_swiglu(x, self.w_gate_up, rt, ctx.act_dtype)
            y = ops.grouped_linear(act, self.w_down, rt, False, ctx.act_dtype)
            return ops.moe_combine(y, rt.inv_pos, None, T, 1)

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(HID, 1e-5), LearnedPositions(Attention(HID, NH, NKV, HD), HID, MAXPOS),
                               RMSNorm(HID, 1e-5), RoutedByPosition(),
                               names={"norm1": "n1.", "mixer": "mix.", "norm2": "n2.", "ffn": "ff."}) for _ in range(2)]
        return DecoderModel(VOCAB, HID, blocks, RMSNorm(HID, 1e-5), config=cfg)

    register_architecture("ToyLearnedPositions", ToyConfig, build, replace=True)
    try:
        eng = Engine(config=ToyConfig(), weight_seed=11, dtype="float32", kv_tokens=128, max_num_seqs=3, weight_std=0.3)
        a, b = H.random_tokens(50, VOCAB, 1), H.random_tokens(33, VOCAB, 2)
        whole_a = H.run_cut(eng, "a", a, [50])
        whole_b = H.run_cut(eng, "b", b, [33])
        assert float((H.run_cut(eng, "a2", a, H.changing_portions(50, 4)) - whole_a).abs().max()) <= 1e-4
        steps = H.mixed_trace({"a": a, "b": b, "c": H.random_tokens(7, VOCAB, 3)}, seed=1, max_live=3, tail=5)
        got = H.replay(eng, steps)
        assert float((got["a"] - whole_a).abs().max()) <= 1e-4 and float((got["b"] - whole_b).abs().max()) <= 1e-4
        # and against the formulas
        m = eng.model
        pos = torch.arange(50, device=DEV)
        h = m.embed[torch.tensor(a, device=DEV)].float()
        causal = torch.tril(torch.ones(50, 50, device=DEV, dtype=torch.bool))
        for blk in m.blocks:
            n = P.rms_norm(h, blk.norm1.weight, 1e-5) + blk.mixer.table[pos]
            att = blk.mixer.inner
            qkv = n @ att.w_qkv.T
            q, k, v = qkv[:, :NH * HD].view(50, NH, HD), qkv[:, NH * HD:(NH + NKV) * HD].view(50, NKV, HD), \
                qkv[:, (NH + NKV) * HD:].view(50, NKV, HD)
            outs = []
            for hh in range(NH):
                sc = (q[:, hh] @ k[:, hh // (NH // NKV)].T) / math.sqrt(HD)
                outs.append(torch.softmax(sc.masked_fill(~causal, float("-inf")), -1) @ v[:, hh // (NH // NKV)])
            h = h + torch.cat(outs, -1) @ att.w_o.T
            n = P.rms_norm(h, blk.norm2.weight, 1e-5)
            y = torch.empty_like(n)
            for e in range(E):
                rows = pos % E == e
                gu = n[rows] @ blk.ffn.w_gate_up[e].T
                y[rows] = (P.silu(gu[:, :INTER]) * gu[:, INTER:]) @ blk.ffn.w_down[e].T
            h = h + y
        want = P.rms_norm(h, m.final_norm.weight, 1e-5) @ m.head.T
        assert float((whole_a - want.cpu()).abs().max()) <= 1e-4
    finally:
        unregister_architecture("ToyLearnedPositions")



@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_with_half_split_partial_rotary_and_scores_on_the_experts_outputs(dtype):
    """An architecture defined here from the framework's own parts with other arguments than
    Llama 4 gives them: rotary on half-split pairs over the first half of each head only, with its
    own base per layer, and a softmax router with renormalised top-2 whose scores multiply the
    experts' OUTPUTS.  No file of the framework knows of it."""
    from sharpinference_amd.cache.spec import WINDOW_SLIDING
    from sharpinference_amd.config.base import ModelConfig
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.parts.attention import Attention
    from sharpinference_amd.parts.block import PreNormBlock
    from sharpinference_amd.parts.feedforward import MoESwiGLU
    from sharpinference_amd.parts.model import DecoderModel
    from sharpinference_amd.parts.norm import RMSNorm
    from sharpinference_amd.parts.position import Rotary
    from sharpinference_amd.registry import register_architecture, unregister_architecture

    HID, NH, NKV, HD, RD, E, K, INTER, VOCAB, WIN = 128, 4, 2, 32, 16, 5, 2, 128, 70, 24
    THETAS = (10000.0, 300.0)

    @dataclass
    class ToyConfig(ModelConfig):
        architecture: str = "ToyHalfSplit"
        vocab_size: int = VOCAB
        max_position_embeddings: int = 256

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": [self.architecture]}

    def build(cfg):
        blocks = []
        for theta in THETAS:
            att = Attention(HID, NH, NKV, HD, rotary=Rotary(HD, theta, None, pair_layout="half", rotary_dim=RD),
                            window_kind=WINDOW_SLIDING, window=WIN)
            ffn = MoESwiGLU(HID, E, K, INTER, shared_intermediate=None, gate="softmax", renormalise=True, score_on_input=False)
            blocks.append(PreNormBlock(RMSNorm(HID, 1e-5), att, RMSNorm(HID, 1e-5), ffn))
        return DecoderModel(VOCAB, HID, blocks, RMSNorm(HID, 1e-5), config=cfg)

    register_architecture("ToyHalfSplit", ToyConfig, build, replace=True)
    try:
        eng = Engine(config=ToyConfig(), weight_seed=5, dtype=dtype, kv_tokens=256, max_num_seqs=3, weight_std=0.2)
        a, b = H.random_tokens(60, VOCAB, 1), H.random_tokens(41, VOCAB, 2)
        whole_a = H.run_cut(eng, "a", a, [60])
        whole_b = H.run_cut(eng, "b", b, [41])
        cut_tol = 1e-4 if dtype == "float32" else 0.15
        assert float((H.run_cut(eng, "a2", a, H.last_decoded(60, 20)) - whole_a).abs().max()) <= cut_tol * float(whole_a.abs().max())
        steps = H.mixed_trace({"a": a, "b": b, "c": H.random_tokens(9, VOCAB, 3)}, seed=3, max_live=3, tail=5)
        got = H.replay(eng, steps)
        assert float((got["a"] - whole_a).abs().max()) <= cut_tol * float(whole_a.abs().max())
        assert float((got["b"] - whole_b).abs().max()) <= cut_tol * float(whole_b.abs().max())
        if dtype != "float32":
            return
        # against the formulas, written out here
        m = eng.model
        n_tok = 60
        pos = torch.arange(n_tok, device=DEV)
        h = m.embed[torch.tensor(a, device=DEV)].float()
        visible = (pos[None, :] <= pos[:, None]) & (pos[None, :] > pos[:, None] - WIN)
        for blk, theta in zip(m.blocks, THETAS):
            n = P.rms_norm(h, blk.norm1.weight, 1e-5)
            att = blk.mixer
            qkv = n @ att.w_qkv.T
            q, k, v = (qkv[:, :NH * HD].view(n_tok, NH, HD).clone(), qkv[:, NH * HD:(NH + NKV) * HD].view(n_tok, NKV, HD).clone(),
                       qkv[:, (NH + NKV) * HD:].view(n_tok, NKV, HD))
            freq = torch.tensor([theta ** (-2.0 * i / RD) for i in range(RD // 2)], device=DEV, dtype=torch.float32)
            ang = pos.float()[:, None] * freq[None, :]
            cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            for t in (q, k):
                x0, x1 = t[..., :RD // 2].clone(), t[..., RD // 2:RD].clone()
                t[..., :RD // 2], t[..., RD // 2:RD] = x0 * cos - x1 * sin, x0 * sin + x1 * cos
            outs = []
            for hh in range(NH):
                sc = (q[:, hh] @ k[:, hh // (NH // NKV)].T) / math.sqrt(HD)
                outs.append(torch.softmax(sc.masked_fill(~visible, float("-inf")), -1) @ v[:, hh // (NH // NKV)])
            h = h + torch.cat(outs, -1) @ att.w_o.T
            n = P.rms_norm(h, blk.norm2.weight, 1e-5)
            ffn = blk.ffn
            gates = torch.softmax(n @ ffn.w_router.T.float(), -1)
            top = gates.topk(K, dim=-1)
            wts = top.values / top.values.sum(-1, keepdim=True)
            y = torch.zeros_like(n)
            for t in range(n_tok):
                for j in range(K):
                    e = int(top.indices[t, j])
                    gu = ffn.w_gate_up[e] @ n[t]
                    y[t] += wts[t, j] * (ffn.w_down[e] @ (P.silu(gu[:INTER]) * gu[INTER:]))
            h = h + y
        want = P.rms_norm(h, m.final_norm.weight, 1e-5) @ m.head.T
        assert float((whole_a - want.cpu()).abs().max()) <= 1e-4 * max(1.0, float(want.abs().max()))
    finally:
        unregister_architecture("ToyHalfSplit")


@pytest.mark.parametrize("graphs", [True, False])
def test_a_stateful_mixer_that_can_be_captured_decodes_from_graphs(graphs):
    """A mixer with state of its own that walks the entries through the context's device tensors
    (no copy to the host) declares ``graph_safe``: its decode steps are then replayed from graphs.
    The capture's trial run works on the scratch state slot, so no request's state moves; every
    replay gives what the same step gives when launched part by part."""
    from sharpinference_amd.cache.spec import StateSpec
    from sharpinference_amd.config.base import ModelConfig
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.parts.base import Part
    from sharpinference_amd.parts.block import PreNormBlock
    from sharpinference_amd.parts.feedforward import DenseSwiGLU
    from sharpinference_amd.parts.model import DecoderModel
    from sharpinference_amd.parts.norm import RMSNorm
    from sharpinference_amd.registry import register_architecture, unregister_architecture

    @dataclass
    class ToyConfig(ModelConfig):
        architecture: str = "ToyDecay"
        vocab_size: int = 50
        max_position_embeddings: int = 256

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": [self.architecture]}

    class Decay(Part):
        """out[t] = s[t], s[t] = 0.5 * s[t-1] + x[t]: a state of fixed size per request."""
        graph_safe = True

        def cache_spec(self):
            return StateSpec((32,), torch.float32)

        def forward(self, x, ctx, cache):
            slots = ctx.state_slots.long()                  # device tensor: no host copy
            s = cache.state.index_select(0, slots)          # [entries, H]
            out = torch.empty_like(x)
            o, last = 0, []
            for e, n in enumerate(ctx.entry_lens):          # lengths are the host's plan of the step
                cur = s[e]
                for t in range(n):
                    cur = 0.5 * cur + x[o + t].float()
                    out[o + t] = cur.to(x.dtype)
                last.append(cur)
                o += n
            cache.state.index_copy_(0, slots, torch.stack(last))
            return out

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(32, 1e-5), Decay(), RMSNorm(32, 1e-5), DenseSwiGLU(32, 48),
                               names={"norm1": "n1.", "mixer": "mix.", "norm2": "n2.", "ffn": "ff."}) for _ in range(2)]
        return DecoderModel(cfg.vocab_size, 32, blocks, RMSNorm(32, 1e-5), config=cfg)

    register_architecture("ToyDecay", ToyConfig, build, replace=True)
    try:
        eng = Engine(config=ToyConfig(), weight_seed=3, dtype="float32", kv_tokens=64, max_num_seqs=3, weight_std=0.3,
                     decode_graphs=graphs)
        assert eng.runner.decode_graphs == graphs
        a, b = H.random_tokens(30, 50, 1), H.random_tokens(22, 50, 2)
        steps = [{"entries": [{"id": "a", "tokens": a[:20], "want": [19]}], "end": []},
                 {"entries": [{"id": "b", "tokens": b[:12], "want": [11]}], "end": []}]
        steps += [{"entries": [{"id": "a", "tokens": [a[20 + i]], "want": [0]}, {"id": "b", "tokens": [b[12 + i]], "want": [0]}],
                   "end": []} for i in range(10)]
        steps[-1]["end"] = ["a", "b"]
        for i, st in enumerate(steps):
            st["step"] = i
        got = H.replay(eng, steps)
        assert eng.runner.graph_replays == (10 if graphs else 0)
        whole_a, whole_b = H.run_cut(eng, "wa", a, [30]), H.run_cut(eng, "wb", b, [22])
        assert float((got["a"] - whole_a[19:]).abs().max()) <= 1e-5 and float((got["b"] - whole_b[11:]).abs().max()) <= 1e-5
        # A capture's trial run works on the slot behind the requests' own (it is the only one a
        # trial may change); requests have left their state in their slots, and the next request
        # that takes a slot finds it zeroed.
        scratch = eng.cache.scratch_state_slot
        assert scratch == 3 and eng.cache.state[0].shape[0] == 4
        assert bool(eng.cache.state[0][scratch].any()) == graphs
        assert bool(eng.cache.state[0][:scratch].any())
        eng.add_request("fresh")
        slot = eng.cache.requests["fresh"].state_slot
        assert 0 <= slot < scratch and not bool(eng.cache.state[0][slot].any()) and not bool(eng.cache.state[1][slot].any())
        eng.free_request("fresh")
    finally:
        unregister_architecture("ToyDecay")


@pytest.mark.parametrize("graphs", [True, False])
def test_a_part_declares_the_index_arrays_it_wants_made_once_a_step(graphs, tmp_path):
    """A mixer asks for index arrays of its own through a step planner (here: the row of each
    entry's last token); the step function uploads them with its own arrays, in eager steps and
    in replayed graphs, without knowing what they mean.  A model without attention gets no
    attention work lists."""
    import numpy as np
    from sharpinference_amd.cache.spec import StateSpec
    from sharpinference_amd.config.base import ModelConfig
    from sharpinference_amd.engine import Engine
    from sharpinference_amd.parts.base import Part, StepPlanner
    from sharpinference_amd.parts.block import PreNormBlock
    from sharpinference_amd.parts.feedforward import DenseSwiGLU
    from sharpinference_amd.parts.model import DecoderModel
    from sharpinference_amd.parts.norm import RMSNorm
    from sharpinference_amd.registry import register_architecture, unregister_architecture

    @dataclass
    class ToyConfig(ModelConfig):
        architecture: str = "ToyLastRow"
        vocab_size: int = 50
        max_position_embeddings: int = 256

        @classmethod
        def from_dict(cls, d):
            return cls()

        def to_dict(self):
            return {"architectures": [self.architecture]}

    calls = {"plan": 0, "attach": 0}

    class LastRows(StepPlanner):
        key = "last_rows"

        def plan(self, host):
            calls["plan"] += 1
            return [host.cu_tokens[1:] - 1], {"entries": host.n_entries}

        def null(self, host, arrays):
            return [np.arange(arrays[0].size, dtype=np.int32)]

        def attach(self, ctx, views, facts):
            calls["attach"] += 1
            assert views[0].shape == (facts["entries"],) and views[0].dtype == torch.int32 and views[0].is_cuda
            ctx.extras["last_rows"] = views[0]

    planner = LastRows()

    class Decay(Part):
        """out[t] = s[t], s[t] = 0.5 * s[t-1] + x[t]; the state an entry leaves is the row of its last
        token, found through the planner's list."""
        graph_safe = True

        def step_planners(self):
            return (planner,)

        def cache_spec(self):
            return StateSpec((32,), torch.float32)

        def forward(self, x, ctx, cache):
            slots = ctx.state_slots.long()
            s = cache.state.index_select(0, slots)
            out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            o = 0
            for e, n in enumerate(ctx.entry_lens):
                cur = s[e]
                for t in range(n):
                    cur = 0.5 * cur + x[o + t].float()
                    out[o + t] = cur
                o += n
            cache.state.index_copy_(0, slots, out.index_select(0, ctx.extras["last_rows"].long()))
            return out.to(x.dtype)

    def build(cfg):
        blocks = [PreNormBlock(RMSNorm(32, 1e-5), Decay(), RMSNorm(32, 1e-5), DenseSwiGLU(32, 48),
                               names={"norm1": "n1.", "mixer": "mix.", "norm2": "n2.", "ffn": "ff."}) for _ in range(2)]
        return DecoderModel(cfg.vocab_size, 32, blocks, RMSNorm(32, 1e-5), config=cfg)

    register_architecture("ToyLastRow", ToyConfig, build, replace=True)
    try:
        eng = Engine(config=ToyConfig(), weight_seed=3, dtype="float32", kv_tokens=64, max_num_seqs=3, weight_std=0.3,
                     decode_graphs=graphs)
        assert [pl.key for pl in eng.runner.planners] == ["last_rows"]      # one per key, and no attention lists
        a, b = H.random_tokens(30, 50, 1), H.random_tokens(22, 50, 2)
        steps = [{"entries": [{"id": "a", "tokens": a[:20], "want": [19]}], "end": []},
                 {"entries": [{"id": "b", "tokens": b[:12], "want": [11]}, {"id": "a", "tokens": [a[20]], "want": [0]}], "end": []}]
        steps += [{"entries": [{"id": "a", "tokens": [a[21 + i]], "want": [0]}, {"id": "b", "tokens": [b[12 + i]], "want": [0]}],
                   "end": []} for i in range(9)]
        steps[-1]["end"] = ["a", "b"]
        for i, st in enumerate(steps):
            st["step"] = i
        got = H.replay(eng, steps)
        assert eng.runner.graph_replays == (9 if graphs else 0)
        assert calls["plan"] >= len(steps) and calls["attach"] >= (3 if graphs else len(steps))
        whole_a, whole_b = H.run_cut(eng, "wa", a, [30]), H.run_cut(eng, "wb", b[:21], [21])
        assert float((got["a"] - whole_a[19:]).abs().max()) <= 1e-5 and float((got["b"] - whole_b[11:]).abs().max()) <= 1e-5
    finally:
        unregister_architecture("ToyLastRow")
    # the architecture's own model asks for the attention kernels' work lists, once for all its layers
    eng = Engine(make_model_dir(tmp_path, "A"), dtype="float32", kv_tokens=128, max_num_seqs=2)
    assert [pl.key for pl in eng.runner.planners] == ["attention"]
