"""A plain, slow Llama 4 text decoder: whole sequences, no cache, one function a part.

This file is the yardstick of the tests.  It shares no code with the package: it
reads ``config.json`` as a raw dict, takes weights as a ``{name: tensor}`` dict and
computes everything with ordinary dense tensor arithmetic on the CPU.  Each function
cites the place in the reference (paths from the root of pekkah/SharpInference) whose
formula it follows; where the reference has no such code the formula is stated in full.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# ----------------------------------------------------------------------------
# configuration (raw dict -> the handful of derived per-layer facts)
# ----------------------------------------------------------------------------
def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        d = json.load(f)
    c = dict(d.get("text_config") or {})
    for k, v in d.items():
        if k != "text_config":
            c.setdefault(k, v)
    # the rotary base and its scaling may come in one object instead of two keys
    rp = c.get("rope_parameters")
    if rp:
        c["rope_theta"] = rp["rope_theta"]
        rest = {k: v for k, v in rp.items() if k != "rope_theta"}
        c["rope_scaling"] = rest if rest.get("rope_type", "default") != "default" else None
    if not c.get("no_rope_layers") and c.get("no_rope_layer_interval"):
        step = int(c["no_rope_layer_interval"])
        c["no_rope_layers"] = [int((l + 1) % step != 0) for l in range(int(c["num_hidden_layers"]))]
    return c


def layer_uses_rope(c: dict, layer: int) -> bool:
    """src/SharpInference.Engine/ForwardPass.cs:1617-1618: rotary unless (layer+1) % 4 == 0;
    a ``no_rope_layers`` list in config.json (non-zero = rotary) takes the rule's place."""
    lst = c.get("no_rope_layers") or []
    if lst:
        return lst[layer] != 0
    return (layer + 1) % 4 != 0


def layer_is_moe(c: dict, layer: int) -> bool:
    """The reference is all-or-nothing (ForwardPass.cs:353-371); with
    ``interleave_moe_layer_step`` = s layer L has experts iff (L+1) % s == 0."""
    if c.get("moe_layers") is not None:
        return layer in c["moe_layers"]
    s = int(c.get("interleave_moe_layer_step", 1))
    return s > 0 and (layer + 1) % s == 0


def head_dim_of(c: dict) -> int:
    return int(c.get("head_dim") or c["hidden_size"] // c["num_attention_heads"])


# ----------------------------------------------------------------------------
# norms
# ----------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """src/SharpInference.Cpu/SimdKernels.cs:4209-4246: s = 1/sqrt(mean(x^2) + eps);
    out = (x * s) * w; eps inside the root, scale first, weight second."""
    s = 1.0 / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    y = x * s
    return y if w is None else y * w


def l2_head_norm(x: torch.Tensor, eps: float) -> torch.Tensor:
    """SimdKernels.cs:4252-4283 (PureRmsNorm), used per head at ForwardPass.cs:2401-2405:
    the same as rms_norm without a weight, over the head's width."""
    return rms_norm(x, None, eps)


# ----------------------------------------------------------------------------
# position encoding
# ----------------------------------------------------------------------------
def rope_inv_freq(head_dim: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """SimdKernels.cs:4789-4811 (BuildRopeTable): freq_i = theta^(-2i/head_dim), i < head_dim/2.

    llama3 scaling is not in the reference (it only divides by an optional table,
    ForwardPass.cs:259-276).  Its rule: wavelength L_i = 2*pi/freq_i, o = original
    context; L_i < o/high: unchanged; L_i > o/low: freq_i/factor; between:
    s = (o/L_i - low)/(high - low), freq_i <- (1-s)*freq_i/factor + s*freq_i.
    Computed in double, rounded once to float."""
    half = head_dim // 2
    out = []
    for i in range(half):
        f = theta ** (-2.0 * i / head_dim)
        if scaling:
            factor = float(scaling["factor"])
            low = float(scaling.get("low_freq_factor", 1.0))
            high = float(scaling.get("high_freq_factor", 4.0))
            o = float(scaling["original_max_position_embeddings"])
            wavelen = 2.0 * math.pi / f
            if wavelen < o / high:
                pass
            elif wavelen > o / low:
                f = f / factor
            else:
                s = (o / wavelen - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


def apply_rope_interleaved(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """SimdKernels.cs:4591-4629 (ApplyRoPECached): pairs (2i, 2i+1) of each head rotate by
    a = pos * freq_i: (x0, x1) -> (x0 cos a - x1 sin a, x0 sin a + x1 cos a).
    x: [T, heads, head_dim]; positions: [T]. The angle is a float32 product, as the
    reference's table builder multiplies in single precision."""
    dt = x.dtype
    ang = positions.to(torch.float32)[:, None] * inv_freq.to(positions.device)[None, :]      # [T, hd/2] float32
    cos = torch.cos(ang).to(dt)[:, None, :]
    sin = torch.sin(ang).to(dt)[:, None, :]
    x0 = x[..., 0::2]
    x1 = x[..., 1::2]
    y0 = x0 * cos - x1 * sin
    y1 = x0 * sin + x1 * cos
    return torch.stack((y0, y1), dim=-1).reshape(x.shape)


def query_temperature(positions: torch.Tensor, floor_scale: float, attn_scale: float) -> torch.Tensor:
    """Not in the reference.  Queries of layers without rotary are multiplied by
    1 + attn_scale * ln(floor((p + 1) / floor_scale) + 1), p the absolute position."""
    p = positions.to(torch.float32)
    return 1.0 + attn_scale * torch.log(torch.floor((p + 1.0) / floor_scale) + 1.0)


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------
def attention_mask(positions: torch.Tensor, chunk: Optional[int]) -> torch.Tensor:
    """Causal (ForwardPass.cs:1850-1851 visits keys 0..p only); with a chunk C a key t is
    visible from p iff t <= p and floor(t/C) == floor(p/C).  [T, T] bool, True = visible."""
    q = positions[:, None]
    k = positions[None, :]
    m = k <= q
    if chunk:
        m = m & ((k // chunk) == (q // chunk))
    return m


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """ForwardPass.cs:1838-1912: head h reads kv head h // G; score = q.k * head_dim^-0.5;
    softmax over visible keys; out = sum w_t v_t.  q: [T, nh, hd]; k, v: [T, nkv, hd]."""
    T, nh, hd = q.shape
    nkv = k.shape[1]
    g = nh // nkv
    out = torch.empty_like(q)
    scale = 1.0 / math.sqrt(hd)
    for h in range(nh):
        kh = k[:, h // g, :]
        vh = v[:, h // g, :]
        s = (q[:, h, :] @ kh.T) * scale                  # [T, T]
        s = s.masked_fill(~mask, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values           # SimdKernels.cs:4289-4343
        e = torch.exp(s - m)
        w = e / e.sum(dim=-1, keepdim=True)
        out[:, h, :] = w @ vh
    return out


def _same(t: torch.Tensor) -> torch.Tensor:
    return t


def store_bf16(t: torch.Tensor) -> torch.Tensor:
    """Round to bfloat16 and back: what the engine's bfloat16 path does wherever a tensor is
    handed from one kernel to the next or kept in the cache.  The residual sum, norm
    statistics, angles, scores and router values stay in float there and are not rounded here."""
    return t.to(torch.bfloat16).to(t.dtype)


def attention_layer(c: dict, W: Dict[str, torch.Tensor], layer: int, n: torch.Tensor,
                    positions: torch.Tensor, store=_same, kv_out: Optional[list] = None, kv_in=None) -> torch.Tensor:
    """ForwardPass.cs:1576-1690 for one layer on normed input n [T, H]: projections
    without bias, rotary then weightless norm on rotary layers (1635-1648), temperature
    on the others, attention, output projection.  `store` marks where the engine stores a
    tensor (identity in the 32-bit case)."""
    p = f"model.layers.{layer}.self_attn."
    nh, nkv, hd = c["num_attention_heads"], c.get("num_key_value_heads", c["num_attention_heads"]), head_dim_of(c)
    T = n.shape[0]
    q, k, v = (store(n @ W[p + f"{name}_proj.weight"].T) for name in "qkv")
    if c.get("attention_bias", False):       # ForwardPass.cs:1605-1613: biases right after the products
        q, k, v = (t + W[p + f"{name}_proj.bias"].to(t.dtype) for t, name in zip((q, k, v), "qkv"))
        v = store(v)                         # values go to the cache as they are
    q, k, v = q.view(T, nh, hd), k.view(T, nkv, hd), v.view(T, nkv, hd)
    eps = float(c.get("rms_norm_eps", 1e-5))
    if layer_uses_rope(c, layer):
        inv = rope_inv_freq(hd, float(c.get("rope_theta", 500000.0)), c.get("rope_scaling"))
        q = apply_rope_interleaved(q, positions, inv)
        k = apply_rope_interleaved(k, positions, inv)
        if c.get("use_qk_norm", True):
            q = l2_head_norm(q, eps)
            k = l2_head_norm(k, eps)
        mask = attention_mask(positions, int(c.get("attention_chunk_size", 8192)))
    else:
        if c.get("attn_temperature_tuning", True):
            t = query_temperature(positions, float(c.get("floor_scale", 8192)), float(c.get("attn_scale", 0.1)))
            q = q * t.to(q.dtype)[:, None, None]
        mask = attention_mask(positions, None)
    q, k = store(q), store(k)
    if kv_out is not None:       # hand the keys and values out (a later layer may read this layer's cache)
        kv_out.append((k, v))
    if kv_in is not None:        # read another layer's keys and values instead of this layer's own
        k, v = kv_in
    o = store(attention(q, k, v, mask)).reshape(T, nh * hd)
    out = store(o @ W[p + "o_proj.weight"].T)
    if c.get("attention_bias", False):       # ForwardPass.cs:893 (the output projection's bias)
        out = store(out + W[p + "o_proj.bias"].to(out.dtype))
    return out


# ----------------------------------------------------------------------------
# feed-forward
# ----------------------------------------------------------------------------
def silu(x: torch.Tensor) -> torch.Tensor:
    """SimdKernels.cs:4377-4408: g / (1 + exp(-g))."""
    return x / (1.0 + torch.exp(-x))


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """SimdKernels.cs:4474-4484 (the scalar form): 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))."""
    return 0.5 * x * (1.0 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)))


def activation_of(c: dict):
    """The gated unit's activation by the name config.json gives it (``hidden_act``): SiLU unless the
    file names the tanh form of GELU."""
    name = c.get("hidden_act", "silu")
    if name in ("silu", "swish"):
        return silu
    if name in ("gelu_pytorch_tanh", "gelu_tanh"):
        return gelu_tanh
    raise ValueError(f"hidden_act {name!r}")


def swiglu(n: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor, wd: torch.Tensor, store=_same, act=silu) -> torch.Tensor:
    """ForwardPass.cs:2006-2015: down( act(gate n) * (up n) ), act = SiLU for this architecture."""
    return store(store(act(store(n @ wg.T)) * store(n @ wu.T)) @ wd.T)


def router_gates(n: torch.Tensor, wr: torch.Tensor) -> torch.Tensor:
    """ForwardPass.cs:2028-2032: logits = Wr n, then a sigmoid over every expert."""
    return 1.0 / (1.0 + torch.exp(-(n @ wr.T)))


def router_topk(n: torch.Tensor, wr: torch.Tensor, k: int):
    """ForwardPass.cs:2028-2040 and 2132-2150: k picks by gate value, strict > so the lowest
    index wins a tie; weight = that gate value.  No renormalisation of the k weights (the
    reference would renormalise for k > 1, 2156-2162; this engine does not, by decision)."""
    dev = n.device
    sig = router_gates(n, wr).cpu()                      # [T, E]; the scan below runs on the host
    T, E = sig.shape
    ids = torch.zeros(T, k, dtype=torch.long)
    wts = torch.zeros(T, k, dtype=sig.dtype)
    rows = sig.tolist()
    for t in range(T):
        taken: List[int] = []
        for j in range(k):
            best, bv = 0, -float("inf")
            for e in range(E):
                if e in taken:
                    continue
                if rows[t][e] > bv:
                    bv, best = rows[t][e], e
            taken.append(best)
            ids[t, j] = best
            wts[t, j] = sig[t, best]
    return ids.to(dev), wts.to(dev)


def router_margin(n: torch.Tensor, wr: torch.Tensor, k: int) -> torch.Tensor:
    """Per token: router logit of the k-th pick minus that of the best expert left out,
    relative to the rms of the token's logits (inf if no expert is left out).  Where it is
    tiny, rounding decides the route; tests use it to tell which positions of a
    reduced-precision run can be compared with a 32-bit one."""
    r = n @ wr.T
    srt = torch.sort(r, dim=-1, descending=True).values
    if srt.shape[1] <= k:
        return torch.full((n.shape[0],), float("inf"), device=n.device)
    return (srt[:, k - 1] - srt[:, k]) / r.pow(2).mean(dim=-1).sqrt().clamp_min(1e-30)


def moe_layer(c: dict, W: Dict[str, torch.Tensor], layer: int, n: torch.Tensor, trace: Optional[dict] = None,
              store=_same, routes: Optional[dict] = None) -> torch.Tensor:
    """ForwardPass.cs:2021-2098: shared expert on the unscaled input (2060-2066); each chosen
    expert's gate and up products are multiplied by its score before the SiLU (2083-2089);
    sum of experts plus shared (2096-2097)."""
    p = f"model.layers.{layer}.feed_forward."
    k = int(c.get("num_experts_per_tok", 1))
    ids, wts = router_topk(n, W[p + "router.weight"], k)
    if routes is not None:
        # Picks given from outside (a reduced-precision run's own): take them, with this
        # implementation's gate values as weights, and record how far each lies below the
        # pick made here, relative to the rms of the token's router logits.
        r = n @ W[p + "router.weight"].T
        forced = routes[layer].to(torch.long).to(n.device)
        own = torch.gather(r, 1, ids)
        got = torch.gather(r, 1, forced)
        regret = (own.sort(dim=1).values - got.sort(dim=1).values).abs().max(dim=1).values
        regret = regret / r.pow(2).mean(dim=-1).sqrt().clamp_min(1e-30)
        if trace is not None:
            trace["route_regret"] = max(float(regret.max()), trace.get("route_regret", 0.0))
        ids = forced
        wts = torch.gather(router_gates(n, W[p + "router.weight"]), 1, forced)
    if trace is not None:
        trace.setdefault("picks", {})[layer] = ids      # the picks this run made (or was given), layer by layer
        m = router_margin(n, W[p + "router.weight"], k)
        trace["router_margin"] = torch.minimum(trace["router_margin"], m) if "router_margin" in trace else m
    act = activation_of(c)
    out = swiglu(n, W[p + "shared_expert.gate_proj.weight"], W[p + "shared_expert.up_proj.weight"],
                 W[p + "shared_expert.down_proj.weight"], store, act)
    Wg, Wu, Wd = W[p + "experts.gate_proj"], W[p + "experts.up_proj"], W[p + "experts.down_proj"]
    routed = torch.zeros_like(out)
    for e in range(Wg.shape[0]):                 # expert by expert, over the (token, pick) pairs that chose it
        t_idx, j_idx = (ids == e).nonzero(as_tuple=True)
        if t_idx.numel() == 0:
            continue
        w = wts[t_idx, j_idx][:, None]
        g = store(n[t_idx] @ Wg[e].T) * w
        u = store(n[t_idx] @ Wu[e].T) * w
        routed.index_add_(0, t_idx, store(store(act(g) * u) @ Wd[e].T))
    return store(routed + out)


def dense_layer(c: dict, W: Dict[str, torch.Tensor], layer: int, n: torch.Tensor, store=_same) -> torch.Tensor:
    p = f"model.layers.{layer}.feed_forward."
    return swiglu(n, W[p + "gate_proj.weight"], W[p + "up_proj.weight"], W[p + "down_proj.weight"], store, activation_of(c))


# ----------------------------------------------------------------------------
# whole model
# ----------------------------------------------------------------------------
def forward(c: dict, W: Dict[str, torch.Tensor], tokens: Sequence[int], start_pos: int = 0,
            dtype: torch.dtype = torch.float32, trace: Optional[dict] = None, store=_same,
            routes: Optional[dict] = None) -> torch.Tensor:
    """ForwardPass.cs:1474-1757 (Forward / RunTrunk) for a whole sequence at once:
    embed (no scale, 1478-1483); per layer norm -> attention -> +residual (1557-1690),
    norm -> feed-forward -> +residual (1695-1714); final norm and head (1741-1747).
    Returns logits [T, vocab].  With store=store_bf16 every tensor the engine's bfloat16 path
    stores is rounded as it is there; the arithmetic stays float.  `routes` ({layer: ids [T, k]})
    replaces the router's picks (see moe_layer)."""
    W = {k: v.to(dtype) if v.is_floating_point() else v for k, v in W.items()}
    eps = float(c.get("rms_norm_eps", 1e-5))
    dev = W["model.embed_tokens.weight"].device          # the run follows its weights' device
    ids = torch.tensor(list(tokens), dtype=torch.long, device=dev)
    positions = torch.arange(start_pos, start_pos + len(ids), device=dev)
    h = W["model.embed_tokens.weight"][ids]
    for l in range(int(c["num_hidden_layers"])):
        p = f"model.layers.{l}."
        n = store(rms_norm(h, W[p + "input_layernorm.weight"], eps))
        h = h + attention_layer(c, W, l, n, positions, store)
        n = store(rms_norm(h, W[p + "post_attention_layernorm.weight"], eps))
        h = h + (moe_layer(c, W, l, n, trace, store, routes) if layer_is_moe(c, l) else dense_layer(c, W, l, n, store))
    h = store(rms_norm(h, W["model.norm.weight"], eps))
    head = W["model.embed_tokens.weight"] if c.get("tie_word_embeddings", False) else W["lm_head.weight"]
    return h @ head.T


def load_weights(model_dir: str) -> Dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return load_file(os.path.join(model_dir, "model.safetensors"))


# ----------------------------------------------------------------------------
# sampling
# ----------------------------------------------------------------------------
def greedy(logits: torch.Tensor) -> int:
    """src/SharpInference.Engine/Sampler.cs:436-449: first maximum wins."""
    best, bv = 0, float(logits[0])
    for i in range(1, logits.numel()):
        if float(logits[i]) > bv:
            best, bv = i, float(logits[i])
    return best


def softmax_f32(x: torch.Tensor) -> torch.Tensor:
    """Sampler.cs:451-467."""
    e = torch.exp(x - x.max())
    return e * (1.0 / e.sum())


def sample(logits: torch.Tensor, u: float, temperature: float, top_k: int = 0, top_p: float = 1.0,
           min_p: float = 0.0) -> int:
    """Sampler.cs:15-107 (the full-vocabulary path) and 564-576: logits / T -> softmax ->
    top-k (zero what lies below the k-th value, renormalise) -> min-p (zero what lies below
    min_p * max) -> top-p (smallest prefix of the descending order whose sum reaches p) ->
    renormalise -> first index whose running sum reaches u; the last index if none does."""
    if temperature <= 0:
        return greedy(logits)
    x = logits.to(torch.float32).clone()
    if temperature != 1.0:
        x = x * (1.0 / temperature)
    p = softmax_f32(x)
    V = p.numel()
    if 0 < top_k < V:
        kth = torch.sort(p, descending=True).values[top_k - 1]
        p = torch.where(p < kth, torch.zeros_like(p), p)
        p = p / p.sum()
    if min_p > 0:
        p = torch.where(p < min_p * p.max(), torch.zeros_like(p), p)
    if 0 < top_p < 1:
        order = torch.sort(p, descending=True, stable=True)
        cum, cutoff = 0.0, V
        for i in range(V):
            cum += float(order.values[i])
            if cum >= top_p:
                cutoff = i + 1
                break
        keep = torch.zeros(V, dtype=torch.bool)
        keep[order.indices[:cutoff]] = True
        p = torch.where(keep, p, torch.zeros_like(p))
    s = p.sum()
    if float(s) > 0:
        p = p / s
    cum = torch.cumsum(p.to(torch.float32), 0)
    hit = (torch.tensor(u, dtype=torch.float32) <= cum).nonzero()
    return int(hit[0]) if hit.numel() else V - 1


def uniform_stream(seed: int, n: int) -> List[float]:
    """The engine's stated generator of sampling uniforms: draw i of a request with seed s is
    mix(s * 0x9E3779B97F4A7C15 + (i + 1) * 0xBF58476D1CE4E5B9) >> 40 scaled by 2^-24, with
    mix the splitmix64 finaliser.  (The reference uses .NET's Random, Sampler.cs:564-566;
    only the use of one uniform per token is taken from it.)"""
    M = (1 << 64) - 1
    out = []
    for i in range(n):
        z = ((seed & M) * 0x9E3779B97F4A7C15 + (i + 1) * 0xBF58476D1CE4E5B9) & M
        z ^= z >> 30
        z = (z * 0xBF58476D1CE4E5B9) & M
        z ^= z >> 27
        z = (z * 0x94D049BB133111EB) & M
        z ^= z >> 31
        out.append((z >> 40) / float(1 << 24))
    return out


def generate(c: dict, W: Dict[str, torch.Tensor], prompt: Sequence[int], max_new: int,
             temperature: float = 0.0, seed: int = 0, stop: Sequence[int] = ()) -> List[int]:
    """src/SharpInference.Cli/RunCommand.cs:2227-2299 (DecodeLoop): sample from the last
    logits, stop before emitting a stop token, feed the token back.  Recomputes the whole
    sequence each step (no cache)."""
    toks = list(prompt)
    us = uniform_stream(seed, max_new)
    out: List[int] = []
    for i in range(max_new):
        logits = forward(c, W, toks)[-1]
        nxt = greedy(logits) if temperature <= 0 else sample(logits, us[i], temperature)
        if nxt in stop:
            break
        out.append(nxt)
        toks.append(nxt)
    return out
