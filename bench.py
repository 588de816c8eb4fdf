#!/usr/bin/env python3
"""Serving benchmark on one MI355X: Llama 4 Scout-shaped layers, random bfloat16 weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B]

A step is one decode step of a batch of B requests, each with a 2,048-token prompt already in
the cache.  Prints ONE JSON line: decoded tokens per second at the default batch, the prefill of
one 2,048-token prompt, the decode step's HBM roofline, and decode at batch 1 and 64 (with the
roofline fraction of each point), beside the peaks two measuring kernels of the library reach on
this GPU.  ``--profile`` adds, on stderr, milliseconds / bytes / GB/s per kernel class of one
prefill and one decode step, from event pairs.  ``--shape maverick8`` and ``--shape long16`` run
two other workloads instead (128 experts alternating with dense layers at batch 64; 32,768-token
prompts read in 4,096-token portions beside decoding requests) and print a JSON line of their own.
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
                 prompt_len: int = PROMPT_LEN, overrides: dict = None, max_tokens_per_step: int = 8192, **engine_kw):
    from sharpinference_amd.engine import Engine

    cfg = dict(SCOUT)
    cfg.update(overrides or {})
    cfg["num_hidden_layers"] = layers
    cfg["no_rope_layers"] = [0 if (l + 1) % 4 == 0 else 1 for l in range(layers)]
    per_req = (prompt_len + gen_len + page_size - 1) // page_size * page_size + 2 * page_size   # (room for the run-ahead's own warm-up and the traced step)
    context = max(CONTEXT, per_req)
    cfg["max_position_embeddings"] = context
    t0 = time.time()
    eng = Engine(config=cfg, weight_seed=2, dtype="bfloat16", device="cuda:0", max_model_len=context,
                 max_num_seqs=max_batch, max_tokens_per_step=max_tokens_per_step, kv_tokens=max_batch * per_req,
                 page_size=page_size, decode_graphs=graphs, **engine_kw)
    log(f"engine with {layers} layers ready in {time.time() - t0:.1f}s")
    return eng


def layer_bytes(cfg) -> dict:
    """Bytes of the weights one decode step reads, by class (bfloat16)."""
    H, hd = cfg.hidden_size, cfg.head_dim
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd
    attn = 2 * ((q + 2 * kv) * H + H * q)
    expert = 2 * 3 * H * cfg.intermediate_size
    dense = 2 * 3 * H * cfg.intermediate_size_mlp
    router = 2 * cfg.num_local_experts * H
    norms = 2 * 2 * H
    head = 2 * cfg.vocab_size * H
    return {"attn": attn, "expert": expert, "dense": dense, "router": router, "norms": norms, "head": head,
            "kv_per_token": 2 * 2 * kv}


def decode_step_bytes(cfg, layers: int, batch: int, context: int, distinct: float) -> float:
    """Bytes one decode step has to read: every weight it uses once (the shared expert and
    `distinct` routed experts on a routed layer, the dense feed-forward on the others) and the
    cache of the live requests (what each layer's window lets the query at `context - 1` see)."""
    b = layer_bytes(cfg)
    total = b["head"]
    for l in range(layers):
        ffn = b["router"] + b["expert"] * (1 + distinct) if cfg.is_moe_layer(l) else b["dense"]
        total += b["attn"] + b["norms"] + ffn + batch * b["kv_per_token"] * visible_keys(cfg, l, context - 1)
    return total


def visible_keys(cfg, layer: int, position: int) -> int:
    """Keys the query at `position` sees in a layer: all before it, or those of its chunk."""
    if cfg.no_rope_layers[layer] == 0:
        return position + 1
    return position % cfg.attention_chunk_size + 1


def prefill_flops(cfg, T: int, layers: int) -> float:
    H, hd = cfg.hidden_size, cfg.head_dim
    q, kv = cfg.num_attention_heads * hd, cfg.num_key_value_heads * hd
    attn_lin = (q + 2 * kv) * H + H * q
    moe = cfg.num_local_experts * H + 2 * 3 * H * cfg.intermediate_size       # router, one routed expert, the shared one
    dense = 3 * H * cfg.intermediate_size_mlp
    lin = sum(attn_lin + (moe if cfg.is_moe_layer(l) else dense) for l in range(layers))
    C = cfg.attention_chunk_size
    whole, rest = divmod(T, C)
    pairs_chunked = whole * (C * (C + 1) / 2) + rest * (rest + 1) / 2       # (query, key) pairs, causal inside a chunk
    pairs = sum(T * (T + 1) / 2 if cfg.no_rope_layers[l] == 0 else pairs_chunked for l in range(layers))
    attn = 2 * 2 * cfg.num_attention_heads * hd * pairs                     # QK^T and PV
    return 2.0 * T * lin + attn + 2.0 * cfg.vocab_size * H                 # one row through the head


def prefill_bytes(cfg, layers: int, experts_used=None) -> float:
    """Weights a prompt of thousands of tokens has to read once: every expert of every routed layer
    (or `experts_used` of them a layer, where a prompt does not reach them all)."""
    b = layer_bytes(cfg)
    total = b["head"]
    used = cfg.num_local_experts if experts_used is None else experts_used
    for l in range(layers):
        total += b["attn"] + b["norms"] + (b["router"] + b["expert"] * (1 + used) if cfg.is_moe_layer(l) else b["dense"])
    return total


def run_prefill(eng, rid, prompt):
    import torch
    from sharpinference_amd.engine import StepEntry

    eng.add_request(rid)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = None
    for o in range(0, len(prompt), eng.max_tokens_per_step):     # a prompt longer than a step goes in portions
        part = prompt[o:o + eng.max_tokens_per_step]
        logits = eng.step([StepEntry(rid, part, (len(part) - 1,) if o + len(part) == len(prompt) else ())])
    torch.cuda.synchronize()
    return time.perf_counter() - t0, logits


def decode_run(eng, batch: int, steps: int, warmup: int, rng: random.Random, count_experts: bool = False,
               prompt_len: int = PROMPT_LEN):
    """Prefill `batch` prompts, then time `steps` decode steps.  Returns seconds, the mean
    number of distinct experts a step used per layer (if asked), the length the requests reached and
    the host's milliseconds per step."""
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
        if prompt_len <= eng.max_tokens_per_step:
            lg = eng.step([StepEntry(r, p, (prompt_len - 1,)) for r, p in zip(group, prompts)])
        else:                                                # one prompt at a time, in portions of a step
            for o in range(0, prompt_len, eng.max_tokens_per_step):
                part = prompts[0][o:o + eng.max_tokens_per_step]
                lg = eng.step([StepEntry(group[0], part, (len(part) - 1,) if o + len(part) == prompt_len else ())])
        last += ops.argmax_rows(lg).cpu().tolist()
        log(f"  prefilled {min(i + per_step, batch)}/{batch}")

    host = [0.0]

    def one_step(tokens, trace=None):
        # greedy decoding as the engine serves it: the choice is made on the device behind the head.
        # The host's share of a step is what passes inside `step` (bookkeeping, the index arrays, the
        # launch); the wait for the chosen tokens after it is the GPU's.
        h0 = time.perf_counter()
        chosen = eng.step([StepEntry(r, (t,), (0,)) for r, t in zip(ids, tokens)], router_trace=trace, select="argmax")
        host[0] += time.perf_counter() - h0
        return chosen.cpu().tolist()

    def steps_on_end(tokens, n):
        # as the engine generates while every request decodes greedily: `decode_run_ahead` steps are
        # launched on end, each on what the one before chose, and their tokens read back together
        done = 0
        while done < n:
            chosen = eng.decode_steps([StepEntry(r, (t,), (0,)) for r, t in zip(ids, tokens)],
                                      min(eng.decode_run_ahead, n - done)).cpu().tolist()
            tokens = chosen[-1]
            done += len(chosen)
        return tokens

    for _ in range(warmup):
        last = one_step(last)
    if eng.decode_run_ahead > 1:
        last = steps_on_end(last, eng.decode_run_ahead)     # (the step's graph and buffers exist before the clock starts)
    host[0] = 0.0                            # two more, one by one, where the host's share of a step is measured
    for _ in range(2):
        last = one_step(last)
    host_ms = host[0] / 2 * 1e3
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if eng.decode_run_ahead > 1:
        last = steps_on_end(last, steps)
    else:
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
    return dt, distinct, ctx, host_ms


def profile_report(eng, batch: int, prompt_len: int, rng: random.Random) -> None:
    """ms / bytes / GB/s / TFLOP/s per kernel class of one prefill and one decode step (stderr)."""
    from sharpinference_amd.engine import StepEntry
    from sharpinference_amd.ops.profile import Profiler, format_table

    vocab = eng.config.vocab_size
    ids = [f"prof{i}" for i in range(batch)]
    prof = Profiler()
    for n, r in enumerate(ids):
        eng.add_request(r)
        entry = [StepEntry(r, [rng.randrange(vocab) for _ in range(prompt_len)], (prompt_len - 1,))]
        if n == 0:
            eng.profiled_step(entry, prof)
        else:
            eng.step(entry)
    log("\n" + format_table(prof.table(), f"prefill of one prompt of {prompt_len} tokens, by kernel class (event pairs):"))
    decode = [StepEntry(r, (rng.randrange(vocab),), (0,)) for r in ids]
    eng.step(decode, select="argmax")                       # warm
    prof = Profiler()
    decode = [StepEntry(r, (rng.randrange(vocab),), (0,)) for r in ids]
    eng.profiled_step(decode, prof, select="argmax", filler_ms=40.0)
    log("\n" + format_table(prof.table(), f"one decode step at batch {batch}, contexts of {prompt_len + 2} tokens, launched part by "
                                          "part behind filler work, by kernel class (event pairs):"))
    for r in ids:
        eng.free_request(r)


def host_report(eng, prompt_len: int, rng: random.Random, batch: int = 64) -> dict:
    """What the host does in steps where nothing hides it (no steps launched on end, no choice on
    the device): a sampled batch (temperature alone; with top-k / top-p / min-p; with the window
    penalties) and a mixed step (one prompt-sized portion beside the others' decode tokens).
    Per case: milliseconds inside `Engine.step` (index arrays, launches), milliseconds of the
    sampler on an idle GPU (packing the rows' settings, two copies, the kernels, the read-back),
    and the wall time of a whole step.  stderr, and returned for the JSON line."""
    import torch
    from sharpinference_amd import SamplingParams
    from sharpinference_amd.engine import StepEntry
    from sharpinference_amd.sampling.sampler import penalty_window

    vocab = eng.config.vocab_size
    batch = min(batch, eng.max_num_seqs)
    ids = [f"host{i}" for i in range(batch)]
    history = {}
    per_step = max(1, eng.max_tokens_per_step // prompt_len)
    for i in range(0, batch, per_step):
        group = ids[i:i + per_step]
        entries = []
        for r in group:
            eng.add_request(r)
            history[r] = [rng.randrange(vocab) for _ in range(prompt_len)]
            entries.append(StepEntry(r, history[r], ()))
        eng.step(entries)
    cases = {
        "temperature": SamplingParams(temperature=0.8, top_k=0, top_p=1.0, min_p=0.0),
        "filters": SamplingParams(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05),
        "penalties": SamplingParams(temperature=0.8, top_k=40, top_p=0.95, min_p=0.05, repetition_penalty=1.1,
                                    frequency_penalty=0.1, presence_penalty=0.1, penalty_last_n=64),
    }
    out = {}
    tokens = [rng.randrange(vocab) for _ in ids]
    for name, sp in cases.items():
        params = [SamplingParams(**{**sp.__dict__, "seed": 100 + i}) for i in range(batch)]
        t_step = t_sample = t_wall = 0.0
        n, warm = 6, 5       # (a wide batch's graph is captured when its shape has been met four times: within the warm-up)
        for it in range(n + warm):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = eng.step([StepEntry(r, (t,), (0,)) for r, t in zip(ids, tokens)])
            t1 = time.perf_counter()
            hist = [penalty_window(p, history[r][:prompt_len], history[r][prompt_len:]) if p.edits_logits else ()
                    for p, r in zip(params, ids)]
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            tokens = eng.sampler.sample(logits, params, [it] * batch, hist)
            t3 = time.perf_counter()
            for r, t in zip(ids, tokens):
                history[r].append(t)
            if it >= warm:
                t_step += t1 - t0
                t_sample += t3 - t2
                t_wall += t3 - t0
        out[name] = {"step_host_ms": t_step / n * 1e3, "sampler_ms": t_sample / n * 1e3, "step_ms": t_wall / n * 1e3}
        log(f"host, {batch} sampled rows ({name}): {out[name]['step_host_ms']:.2f} ms inside the step function, "
            f"{out[name]['sampler_ms']:.2f} ms in the sampler, of a step of {out[name]['step_ms']:.2f} ms")
    # a mixed step: one request leaves, a new prompt's portion comes in beside the others' decode tokens
    eng.free_request(ids[-1])
    portion = min(prompt_len, eng.max_tokens_per_step - (batch - 1))
    t_step = t_wall = 0.0
    n = 3
    for it in range(n + 1):
        rid = f"hostmix{it}"
        eng.add_request(rid)
        entries = [StepEntry(r, (t,), (0,)) for r, t in zip(ids[:-1], tokens[:-1])]
        entries.append(StepEntry(rid, [rng.randrange(vocab) for _ in range(portion)], (portion - 1,)))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        picked = eng.step(entries, select="argmax")
        t1 = time.perf_counter()
        tokens = picked.cpu().tolist()[:batch - 1] + [0]
        t2 = time.perf_counter()
        eng.free_request(rid)
        if it >= 1:
            t_step += t1 - t0
            t_wall += t2 - t0
    out["mixed"] = {"step_host_ms": t_step / n * 1e3, "step_ms": t_wall / n * 1e3, "portion_tokens": portion,
                    "decode_tokens": batch - 1}
    log(f"host, mixed step ({portion} prompt tokens beside {batch - 1} decode tokens): {out['mixed']['step_host_ms']:.2f} ms "
        f"inside the step function (launches run ahead of the GPU), of a step of {out['mixed']['step_ms']:.2f} ms")
    for r in ids[:-1]:
        eng.free_request(r)
    return out


def run_maverick8(args) -> int:
    """Eight Maverick-shaped layers: dense feed-forward (16,384) alternating with 128 experts
    top-1 + shared, no rotary scaling, no QK norm; router weights drawn so that router logits are
    about N(0, 1) and the experts' load is uneven.  Batch 64 of 1,024-token prompts, 128 decode steps."""
    import torch
    from sharpinference_amd.engine import StepEntry

    layers, batch, P, steps, warm = 8, 64, 1024, args.steps if args.steps != GEN_LEN - 8 else 120, 8
    over = {"num_local_experts": 128, "interleave_moe_layer_step": 2, "rope_scaling": None, "use_qk_norm": False}
    eng = build_engine(layers, batch, args.page_size, gen_len=steps + warm + 2, prompt_len=P, overrides=over,
                       weight_std_by_suffix={"router.weight": 5120 ** -0.5})
    cfg = eng.config
    rng = random.Random(3)
    prompt = [rng.randrange(cfg.vocab_size) for _ in range(P)]
    run_prefill(eng, "warm", prompt)
    eng.free_request("warm")
    eng.add_request("load")
    trace: list = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.step([StepEntry("load", prompt, (P - 1,))], router_trace=trace)
    torch.cuda.synchronize()
    pre_s = time.perf_counter() - t0
    eng.free_request("load")
    hist = torch.bincount(trace[0][0].flatten().long().cpu(), minlength=cfg.num_local_experts).tolist()
    log(f"prefill {P} tokens: {pre_s * 1e3:.1f} ms; tokens per expert in the first routed layer: min {min(hist)}, "
        f"median {sorted(hist)[len(hist) // 2]}, max {max(hist)}, unused {hist.count(0)} of {len(hist)}")
    dt, distinct, ctx, _ = decode_run(eng, batch, steps, warm, rng, count_experts=True, prompt_len=P)
    ms_step = dt / steps * 1e3
    step_bytes = decode_step_bytes(cfg, layers, batch, ctx, distinct)
    achieved = step_bytes / (ms_step * 1e-3) / 1e9
    log(f"decode b{batch}: {ms_step:.2f} ms/step, {batch * steps / dt:.1f} tok/s, {achieved:.0f} GB/s ({distinct:.1f} experts per routed layer)")
    out = {"metric": "decode tok/s at batch 64 (8 Maverick-shaped layers, 1,024-token prompts)", "value": batch * steps / dt,
           "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": ms_step, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"model": "llama4-maverick-shaped-random", "global_batch": batch, "seq_len": eng.max_model_len,
                      "parallelism": "single-gpu", "layers": layers, "layers_of_full_model": 48, "hidden_size": cfg.hidden_size,
                      "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                      "experts": cfg.num_local_experts, "moe_every": cfg.interleave_moe_layer_step,
                      "expert_ffn": cfg.intermediate_size, "dense_ffn": cfg.intermediate_size_mlp, "vocab": cfg.vocab_size,
                      "prompt_len": P, "generated": steps + warm, "page_size": args.page_size},
           "prefill": {"value": P / pre_s, "tokens": P, "ms": pre_s * 1e3,
                       "frac": prefill_flops(cfg, P, layers) / pre_s / (PEAK_DENSE_TFLOPS["bf16"] * 1e12),
                       # with 8 tokens an expert the prompt is a stream of the weights it touches
                       "hbm_frac": prefill_bytes(cfg, layers, experts_used=len(hist) - hist.count(0)) / pre_s / 1e9 / PEAK_HBM_GBS},
           "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS},
           "expert_load": {"min": min(hist), "median": sorted(hist)[len(hist) // 2], "max": max(hist), "unused": hist.count(0),
                           "distinct_per_decode_step": distinct}}
    print(json.dumps(out), flush=True)
    return 0


def run_long16(args) -> int:
    """Sixteen Scout-shaped layers, 8 prompts of 32,768 tokens read in portions of 4,096 beside the
    decoded tokens of the requests that are already through (the scheduler mixes them), then
    decoding alone; 512 generated tokens a request.  Four chunk edges of 8,192 are crossed, the
    windowed layers give pages back behind them, and the query temperature works at long positions."""
    import torch
    from sharpinference_amd.engine import StepEntry
    from sharpinference_amd.engine.scheduler import Request, Scheduler
    from sharpinference_amd.sampling.params import SamplingParams

    layers, batch, P, portion = 16, 8, 32768, 4096
    gen = args.steps if args.steps != GEN_LEN - 8 else 512
    eng = build_engine(layers, batch, args.page_size, gen_len=gen + 8, prompt_len=P, max_tokens_per_step=portion + batch)
    cfg = eng.config
    rng = random.Random(4)
    sched = Scheduler(eng.cache, batch, portion + batch, eng.max_model_len)
    reqs = [Request(("long", i), [rng.randrange(cfg.vocab_size) for _ in range(P)],
                    SamplingParams(temperature=0.0, max_new_tokens=gen, stop_token_ids=())) for i in range(batch)]
    for r in reqs:
        sched.add(r)
    phases = {"mixed": [0.0, 0, 0, 0], "decode": [0.0, 0, 0, 0]}        # seconds, steps, prompt tokens, decoded tokens
    pools = {g.key: g.pool.num_pages for g in eng.cache.groups}
    distinct = None
    while sched.has_work():
        b = sched.schedule()
        if not b:
            break
        entries = [StepEntry(s.request.req_id, s.tokens, (len(s.tokens) - 1,) if s.samples else ()) for s in b]
        n_prompt = sum(len(s.tokens) for s in b if s.request.in_prefill)
        n_dec = sum(1 for s in b if not s.request.in_prefill)
        trace = [] if (not n_prompt and distinct is None) else None   # the first step of decoding alone says how many experts a step uses
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        picked = eng.step(entries, select="argmax", router_trace=trace)
        picked = picked.cpu().tolist() if picked is not None else []
        dt = time.perf_counter() - t0
        if trace:
            distinct = sum(len(set(p.flatten().cpu().tolist())) for p, _, _ in trace) / len(trace)
        it = iter(picked)
        sched.update(b, [next(it) if s.samples else None for s in b])
        ph = phases["mixed" if n_prompt else "decode"]
        ph[0] += dt; ph[1] += 1; ph[2] += n_prompt; ph[3] += n_dec
        if ph[1] % 64 == 0:
            log(f"  {ph[1]} {'mixed' if n_prompt else 'decode'} steps")
    mixed, dec = phases["mixed"], phases["decode"]
    assert all(r.finish_reason == "length" and len(r.output) == gen for r in reqs)
    ms_step = dec[0] / max(1, dec[1]) * 1e3
    ctx = P + gen
    # bytes of a decode step in the middle of the decoding phase
    from_trace = distinct if distinct is not None else 0.0
    step_bytes = decode_step_bytes(cfg, layers, dec[3] / max(1, dec[1]), ctx - gen // 2, from_trace)
    achieved = step_bytes / (ms_step * 1e-3) / 1e9
    log(f"mixed phase: {mixed[1]} steps, {mixed[2]} prompt tokens beside {mixed[3]} decoded tokens in {mixed[0]:.2f} s "
        f"({mixed[2] / mixed[0]:.0f} prompt tok/s); decode alone: {dec[1]} steps, {dec[3] / dec[0]:.1f} tok/s, {ms_step:.2f} ms/step")
    out = {"metric": "decode tok/s at batch 8 after 32,768-token prompts (16 Scout-shaped layers)", "value": dec[3] / dec[0],
           "unit": "tok/s", "n_gpus": 1, "steps": dec[1], "warmup": 0, "ms_per_step": ms_step, "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"model": "llama4-scout-shaped-random", "global_batch": batch, "seq_len": eng.max_model_len,
                      "parallelism": "single-gpu", "layers": layers, "layers_of_full_model": FULL_LAYERS,
                      "hidden_size": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                      "head_dim": cfg.head_dim, "experts": cfg.num_local_experts, "expert_ffn": cfg.intermediate_size,
                      "vocab": cfg.vocab_size, "attention_chunk": cfg.attention_chunk_size, "prompt_len": P,
                      "portion": portion, "generated": gen, "page_size": args.page_size},
           "prefill": {"value": mixed[2] / mixed[0], "tokens": mixed[2], "ms": mixed[0] * 1e3,
                       "frac": batch * prefill_flops(cfg, P, layers) / mixed[0] / (PEAK_DENSE_TFLOPS["bf16"] * 1e12),
                       "steps": mixed[1], "decoded_beside": mixed[3]},
           "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": achieved / PEAK_HBM_GBS,
                        "experts_per_step": from_trace},
           "pools": {f"window_{k[1]}_{k[2]}": v for k, v in pools.items()}}
    print(json.dumps(out), flush=True)
    return 0


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
    ap.add_argument("--no-peaks", action="store_true", help="skip the two measuring kernels (pure read, matrix-core loop)")
    ap.add_argument("--profile", action="store_true", help="also print ms / bytes / GB/s per kernel class of one prefill and one decode step")
    ap.add_argument("--shape", default="scout", choices=["scout", "maverick8", "long16"],
                    help="scout: the headline run; maverick8 / long16: two other workloads, each printing a JSON line of its own")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this engine has no multi-GPU path (N=1 only)")
        return 2
    if args.shape == "maverick8":
        return run_maverick8(args)
    if args.shape == "long16":
        return run_long16(args)

    import torch  # noqa: F401

    rng = random.Random(2)
    max_batch = args.batch if args.no_points else max(args.batch, 64)
    gen_len = max(GEN_LEN, args.warmup + args.steps + 2)      # warm-up, timed steps and the one traced step
    P = args.prompt_len
    eng = build_engine(args.layers, max_batch, args.page_size, graphs=not args.no_graphs, gen_len=gen_len, prompt_len=P)
    cfg = eng.config
    measured = None
    if not args.no_peaks:
        from sharpinference_amd import ops

        measured = ops.measured_peaks("cuda:0", read_bytes=2 << 30)
        log(f"measured on this GPU: pure read {measured['hbm_gbs']:.0f} GB/s (published {PEAK_HBM_GBS:.0f}), "
            f"matrix-core loop {measured['bf16_tflops']:.0f} TFLOP/s bf16 (published {PEAK_DENSE_TFLOPS['bf16']:.0f})")

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
               "frac": flops / pre_s / (PEAK_DENSE_TFLOPS["bf16"] * 1e12),
               "hbm_frac": prefill_bytes(cfg, args.layers) / pre_s / 1e9 / PEAK_HBM_GBS}

    dt, distinct, ctx, host_ms = decode_run(eng, args.batch, args.steps, args.warmup, rng, count_experts=True, prompt_len=P)
    ms_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = decode_step_bytes(cfg, args.layers, args.batch, ctx, distinct)
    achieved = step_bytes / (ms_step * 1e-3) / 1e9
    log(f"decode b{args.batch}: {ms_step:.2f} ms/step ({host_ms:.2f} ms of it on the host), {value:.1f} tok/s, {achieved:.0f} GB/s "
        f"({distinct:.2f} experts per layer)")

    points, points_roofline, points_host = {}, {}, {}
    if not args.no_points:
        for pb in (1, 64):
            k = max(8, args.steps // 2)
            pdt, pdist, pctx, phost = decode_run(eng, pb, k, max(2, args.warmup // 2), rng, count_experts=True, prompt_len=P)
            points[f"decode_b{pb}"] = pb * k / pdt
            gbs = decode_step_bytes(cfg, args.layers, pb, pctx, pdist) / (pdt / k) / 1e9
            points_roofline[f"decode_b{pb}"] = gbs / PEAK_HBM_GBS
            points_host[f"decode_b{pb}"] = phost
            log(f"decode b{pb}: {pdt / k * 1e3:.2f} ms/step ({phost:.2f} ms on the host), "
                f"{points[f'decode_b{pb}']:.1f} tok/s, {gbs:.0f} GB/s "
                f"({gbs / PEAK_HBM_GBS:.3f} of the roofline; {pdist:.2f} experts per layer)")
    host_cases = None
    if args.profile:
        profile_report(eng, args.batch, P, rng)
        host_cases = host_report(eng, P, rng, batch=max_batch)

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
            "attention_chunk": cfg.attention_chunk_size, "prompt_len": P,
            # decoded tokens a request: warm-up, the two steps that time the host, the run-ahead's own warm-up, the
            # timed steps and the traced one
            "generated": args.warmup + 2 + (eng.decode_run_ahead if eng.decode_run_ahead > 1 else 0) + args.steps + 1,
            "page_size": args.page_size,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": achieved / PEAK_HBM_GBS},
        "points": points,
        "points_roofline": points_roofline,
        "host_ms_per_step": host_ms,
        "points_host_ms_per_step": points_host,
    }
    if host_cases is not None:
        out["host_unhidden"] = {k: {a: round(b, 3) for a, b in v.items()} for k, v in host_cases.items()}
    if measured is not None:
        out["measured_peaks"] = {"hbm_gbs": measured["hbm_gbs"], "bf16_tflops": measured["bf16_tflops"],
                                 "roofline_frac_of_measured": achieved / measured["hbm_gbs"]}
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
