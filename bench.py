#!/usr/bin/env python3
"""Serving benchmark on one MI355X: Llama 4 Scout-shaped layers, random bfloat16 weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of a batch of B requests, each with a 2,048-token prompt already in
the cache.  Prints ONE JSON line: decoded tokens per second at the default batch, the prefill of
one 2,048-token prompt, the decode step's HBM roofline, and decode at batch 1 and 64.
"""
from __future__ import annotations

import argparse
import json
import os
import random
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# published peaks of MI355X
PEAK_HBM_GBS = 8000.0
PEAK_DENSE_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp8": 5000.0, "fp32": 157.3}

SCOUT = {
    "architectures": ["Llama4ForCausalLM"],
    "hidden_size": 5120, "num_hidden_layers": 48, "num_attention_heads": 40, "num_key_value_heads": 8,
    "head_dim": 128, "vocab_size": 202048,
    "intermediate_size": 8192, "intermediate_size_mlp": 16384,
    "num_local_experts": 16, "num_experts_per_tok": 1, "interleave_moe_layer_step": 1,
    "attention_chunk_size": 8192, "use_qk_norm": True, "attn_temperature_tuning": True,
    "floor_scale": 8192, "attn_scale": 0.1, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "tie_word_embeddings": False, "max_position_embeddings": 4096, "torch_dtype": "bfloat16",
}
FULL_LAYERS = 48
PROMPT_LEN = 2048
GEN_LEN = 256
CONTEXT = 4096


def log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def build_engine(layers: int, max_batch: int, page_size: int, graphs: bool = True, gen_len: int = GEN_LEN,
                 prompt_len: int = PROMPT_LEN):
    from sharpinference_amd.engine import Engine

    cfg = dict(SCOUT)
    cfg["num_hidden_layers"] = layers
    cfg["no_rope_layers"] = [0 if (l + 1) % 4 == 0 else 1 for l in range(layers)]
    per_req = (prompt_len + gen_len + page_size - 1) // page_size * page_size
    context = max(CONTEXT, per_req)
    cfg["max_position_embeddings"] = context
    t0 = time.time()
    eng = Engine(config=cfg, weight_seed=2, dtype="bfloat16", device="cuda:0", max_model_len=context,
                 max_num_seqs=max_batch, max_tokens_per_step=8192, kv_tokens=max_batch * per_req,
                 page_size=page_size, decode_graphs=graphs)
    log(f"engine with {layers} layers ready in {time.time() - t0:.1f}s")
    return eng


def layer_bytes(cfg) -> dict:
    """Bytes of the weights one decode step reads, by class (bfloat16)."""
    H, hd = cfg.hidden_size, cfg.head_dim
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd
    attn = 2 * ((q + 2 * kv) * H + H * q)
    expert = 2 * 3 * H * cfg.intermediate_size
    router = 2 * cfg.num_local_experts * H
    norms = 2 * 2 * H
    head = 2 * cfg.vocab_size * H
    return {"attn": attn, "expert": expert, "router": router, "norms": norms, "head": head,
            "kv_per_token": 2 * 2 * kv}


def visible_keys(cfg, layer: int, position: int) -> int:
    """Keys the query at `position` sees in a layer: all before it, or those of its chunk."""
    if cfg.no_rope_layers[layer] == 0:
        return position + 1
    return position % cfg.attention_chunk_size + 1


def prefill_flops(cfg, T: int, layers: int) -> float:
    H, hd = cfg.hidden_size, cfg.head_dim
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd
    lin = (q + 2 * kv) * H + H * q + cfg.num_local_experts * H + 2 * 3 * H * cfg.intermediate_size
    C = cfg.attention_chunk_size
    whole, rest = divmod(T, C)
    pairs_chunked = whole * (C * (C + 1) / 2) + rest * (rest + 1) / 2       # (query, key) pairs, causal inside a chunk
    pairs = sum(T * (T + 1) / 2 if cfg.no_rope_layers[l] == 0 else pairs_chunked for l in range(layers))
    attn = 2 * 2 * cfg.num_attention_heads * hd * pairs                     # QK^T and PV
    return layers * 2.0 * T * lin + attn + 2.0 * cfg.vocab_size * H        # one row through the head


def run_prefill(eng, rid, prompt):
    import torch
    from sharpinference_amd.engine import StepEntry

    eng.add_request(rid)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = eng.step([StepEntry(rid, prompt, (len(prompt) - 1,))])
    torch.cuda.synchronize()
    return time.perf_counter() - t0, logits


def decode_run(eng, batch: int, steps: int, warmup: int, rng: random.Random, count_experts: bool = False,
               prompt_len: int = PROMPT_LEN):
    """Prefill `batch` prompts, then time `steps` decode steps.  Returns seconds, the mean
    number of distinct experts a step used per layer (if asked) and the length the requests reached."""
    import torch
    from sharpinference_amd import ops
    from sharpinference_amd.engine import StepEntry

    vocab = eng.config.vocab_size
    ids = [f"b{batch}_{i}" for i in range(batch)]
    last = []
    per_step = max(1, eng.max_tokens_per_step // prompt_len)
    for i in range(0, batch, per_step):
        group = ids[i:i + per_step]
        for r in group:
            eng.add_request(r)
        prompts = [[rng.randrange(vocab) for _ in range(prompt_len)] for _ in group]
        lg = eng.step([StepEntry(r, p, (prompt_len - 1,)) for r, p in zip(group, prompts)])
        last += ops.argmax_rows(lg).cpu().tolist()
        log(f"  prefilled {min(i + per_step, batch)}/{batch}")

    def one_step(tokens, trace=None):
        lg = eng.step([StepEntry(r, (t,), (0,)) for r, t in zip(ids, tokens)], router_trace=trace)
        return ops.argmax_rows(lg).cpu().tolist()

    for _ in range(warmup):
        last = one_step(last)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        last = one_step(last)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    distinct = None
    if count_experts:
        trace: list = []
        last = one_step(last, trace)
        distinct = sum(len(set(p.flatten().cpu().tolist())) for p, _, _ in trace) / max(1, len(trace))
    ctx = eng.cache.length(ids[0])
    for r in ids:
        eng.free_request(r)
    return dt, distinct, ctx


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=GEN_LEN - 8, help="timed decode steps (default: with the warm-up, the 256 generated tokens of the baseline's run)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=FULL_LAYERS)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="tokens of every prompt (the contract's run: 2,048)")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--no-graphs", action="store_true", help="launch decode steps kernel by kernel instead of replaying a HIP graph")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this engine has no multi-GPU path (N=1 only)")
        return 2

    import torch  # noqa: F401

    rng = random.Random(2)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    gen_len = max(GEN_LEN, args.warmup + args.steps + 2)      # warm-up, timed steps and the one traced step
    P = args.prompt_len
    eng = build_engine(args.layers, max_batch, args.page_size, graphs=not args.no_graphs, gen_len=gen_len, prompt_len=P)
    cfg = eng.config

    # prefill: one prompt (2,048 tokens) alone, once to warm up, then three times timed
    prompt = [rng.randrange(cfg.vocab_size) for _ in range(P)]
    run_prefill(eng, "warm", prompt)
    eng.free_request("warm")
    times = []
    for i in range(3):                                   # the median of three: a single run varies by a per cent or two
        t, _ = run_prefill(eng, f"timed{i}", prompt)
        eng.free_request(f"timed{i}")
        times.append(t)
    pre_s = sorted(times)[1]
    log(f"prefill {P} tokens: {pre_s * 1e3:.1f} ms")
    flops = prefill_flops(cfg, P, args.layers)
    prefill = {"value": P / pre_s, "tokens": P, "ms": pre_s * 1e3,
               "frac": flops / pre_s / (PEAK_DENSE_TFLOPS["bf16"] * 1e12)}

    dt, distinct, ctx = decode_run(eng, args.batch, args.steps, args.warmup, rng, count_experts=True, prompt_len=P)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    b = layer_bytes(cfg)
    shared_and_routed = b["expert"] * (1 + distinct)
    step_bytes = args.layers * (b["attn"] + b["router"] + b["norms"] + shared_and_routed) + b["head"] \
        + args.batch * b["kv_per_token"] * sum(visible_keys(cfg, l, ctx - 1) for l in range(args.layers))
    achieved = step_bytes / (ms_step * 1e-3) / 1e9
    log(f"decode b{args.batch}: {ms_step:.2f} ms/step, {value:.1f} tok/s, {achieved:.0f} GB/s "
        f"({distinct:.2f} experts per layer)")

    points = {}
    if not args.no_points:
        for pb in (1, 64):
            k = max(8, args.steps // 2)
            pdt, _, _ = decode_run(eng, pb, k, max(2, args.warmup // 2), rng, prompt_len=P)
            points[f"decode_b{pb}"] = pb * k / pdt
            log(f"decode b{pb}: {pdt / k * 1e3:.2f} ms/step, {points[f'decode_b{pb}']:.1f} tok/s")

    out = {
        "metric": f"decode tok/s at batch {args.batch} (Scout-shaped, {P:,}-token prompts)",
        "value": value, "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "model": "llama4-scout-shaped-random", "global_batch": args.batch, "seq_len": eng.max_model_len,
            "parallelism": "single-gpu", "layers": args.layers, "layers_of_full_model": FULL_LAYERS,
            "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
            "head_dim": cfg.head_dim, "experts": cfg.num_local_experts, "experts_per_tok": cfg.num_experts_per_tok,
            "expert_ffn": cfg.intermediate_size, "shared_ffn": cfg.intermediate_size, "vocab": cfg.vocab_size,
            "attention_chunk": cfg.attention_chunk_size, "prompt_len": P, "generated": args.warmup + args.steps,
            "page_size": args.page_size,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": achieved / PEAK_HBM_GBS},
        "points": points,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
