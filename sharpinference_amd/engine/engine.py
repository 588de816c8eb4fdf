"""The engine: a model folder (or a configuration and a seed) turned into something that steps
and generates.  This is the Python entry point; the command line and trace replay are thin
layers over it.

The reference's library API streams chunks from ``GenerateChunksAsync(prompt, SamplingParams)``
(reference: src/SharpInference.Engine/IInferenceEngine.cs:60-64); there is no tokenizer here, so
prompts are lists of token ids and results are lists of token ids.
"""
from __future__ import annotations

import sys
import time
from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, Iterator, List, Optional, Sequence, Union

import torch

from ..cache.manager import CacheManager, pool_sizes
from ..cache.spec import KVSpec
from ..config.base import ModelConfig, load_config
from ..registry import build_model
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler, penalty_window
from ..weights.loader import RandomSource, SafetensorsSource, load_model_weights
from .runner import ModelRunner, StepEntry
from .scheduler import Request, Scheduler

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype {dtype!r} is not supported (bfloat16 or float32)") from None


@dataclass
class GenerationResult:
    token_ids: List[int]
    finish_reason: str
    prompt_tokens: int


@dataclass
class GenerateChunk:
    """One event of a generation (reference: src/SharpInference.Engine/GenerateChunk.cs:52-53)."""
    kind: str                         # "usage" | "token" | "stop"
    index: int                        # which prompt of the call
    token_id: int = -1
    prompt_tokens: int = 0
    finish_reason: Optional[str] = None
    truncated_by_max_tokens: bool = False


@dataclass
class GenerationStats:
    prefill_tokens: int = 0
    decode_tokens: int = 0
    prefill_seconds: float = 0.0
    decode_seconds: float = 0.0
    steps: int = 0


class Engine:
    def __init__(self, model_dir: Optional[str] = None, *, config: Union[ModelConfig, dict, None] = None,
                 weight_seed: Optional[int] = None, dtype="bfloat16", device="cuda:0",
                 max_model_len: Optional[int] = None, max_num_seqs: int = 8, max_tokens_per_step: int = 2048,
                 kv_tokens: Optional[int] = None, page_size: int = 16, weight_std: float = 0.02,
                 weight_std_by_suffix: Optional[Dict[str, float]] = None, verbose: bool = False,
                 decode_graphs: bool = True, past_position_limit: bool = False, row_major_copies: bool = True,
                 decode_run_ahead: int = 4):
        """max_model_len: the longest sequence a request may reach (default: the configuration's
        max_position_embeddings, 4096 if it names none); beyond max_position_embeddings only with
        past_position_limit (replaying given tokens needs no trained positions).
        row_major_copies=False keeps the attention, dense feed-forward and head matrices only in
        the packed order of the decode kernels (about a tenth less weight memory; prompt-sized
        products then run in this library's own kernels instead of the library product, slower).
        decode_run_ahead: while every running request decodes greedily and none waits, generation
        launches this many steps on end, each on what the step before chose (on the device), and
        reads the tokens back together: the host's part of a step then passes while the GPU works
        (1: every step waits for its tokens)."""
        self.decode_run_ahead = max(1, int(decode_run_ahead))
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError("the engine runs on the GPU only (device must be cuda:N)")
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU is visible: the engine has no CPU path")
        from ..ops import lib as _kernel_lib

        _kernel_lib.load(verbose=True)                      # fails loudly if the kernels are missing
        torch.cuda.set_device(self.device)
        if model_dir is not None:
            self.config = load_config(model_dir)
        elif isinstance(config, dict):
            self.config = load_config(config)
        elif config is not None:
            self.config = config
            self.config.validate()
        else:
            raise ValueError("give a model folder or a configuration")
        self.model = build_model(self.config)
        if model_dir is not None:
            source = SafetensorsSource(model_dir, self.dtype, self.device)
        else:
            if weight_seed is None:
                raise ValueError("a configuration without a model folder needs weight_seed (random weights)")
            source = RandomSource(self.model.param_specs(), weight_seed, self.dtype, self.device,
                                  stored_dtype=torch.bfloat16, std=weight_std, std_by_suffix=weight_std_by_suffix,
                                  generate_on_device=True)
        t0 = time.time()
        from .. import ops as _ops

        _ops.keep_row_major_copies(row_major_copies)
        try:
            load_model_weights(self.model, source)
        finally:
            _ops.keep_row_major_copies(True)
        if verbose:
            print(f"[engine] weights ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
        limit = getattr(self.config, "max_position_embeddings", 0) or 0
        self.max_model_len = int(max_model_len or limit or 4096)
        if limit and self.max_model_len > limit and not past_position_limit:
            raise ValueError(f"max_model_len {self.max_model_len} exceeds the model's max_position_embeddings {limit}")
        self.max_num_seqs = int(max_num_seqs)
        self.max_tokens_per_step = int(max_tokens_per_step)
        self.page_size = int(page_size)
        specs = self.model.cache_specs()
        # Pages per group.  kv_tokens is the number of tokens the pools are made for (default: every
        # request at full length, or what four fifths of the free memory hold if that is less); a
        # group without a window gets that many, a windowed group only what its windows can ever
        # hold at once (window + one step, per request), however long the requests grow.
        width = torch.empty(0, dtype=self.dtype).element_size()
        kv_specs = [s for s in specs if isinstance(s, KVSpec)]
        full_len = (self.max_model_len + page_size - 1) // page_size * page_size
        sizes = pool_sizes(specs, page_size, self.max_num_seqs, full_len, self.max_tokens_per_step,
                           None if kv_tokens is None else max(1, (int(kv_tokens) + page_size - 1) // page_size))
        if kv_tokens is None and kv_specs:
            def total_bytes(sz):
                return sum(sz[s.group_key()] * s.num_kv_heads * (s.head_dim + s.value_dim) * page_size * width for s in kv_specs)
            budget = int(torch.cuda.mem_get_info(self.device)[0] * 0.8)
            while total_bytes(sizes) > budget and max(sizes.values()) > 1:
                big = max(sizes, key=lambda k: sizes[k])       # the largest pools give way first
                sizes[big] = max(1, int(sizes[big] * 0.9))
        self.cache = CacheManager(specs, page_size, sizes if sizes else 1, self.max_num_seqs, self.dtype, self.device)
        self.runner = ModelRunner(self.model, self.cache, self.dtype, self.device, decode_graphs=decode_graphs,
                                  max_context=self.max_model_len)
        self.sampler = Sampler(self.device)
        self.last_stats = GenerationStats()
        self._sched: Optional[Scheduler] = None            # the generation that is running, if one is

    # -- the low level: requests and steps ------------------------------------
    def add_request(self, req_id: Hashable) -> None:
        self.cache.add_request(req_id)

    def free_request(self, req_id: Hashable) -> None:
        self.cache.free_request(req_id)

    def step(self, entries: Sequence[StepEntry], router_trace: Optional[list] = None,
             select: Optional[str] = None, device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        return self.runner.step(entries, router_trace, select, device_tokens)

    def decode_steps(self, entries: Sequence[StepEntry], steps: int) -> torch.Tensor:
        """Greedy decode steps run ahead of the host (see ModelRunner.decode_steps): int32
        [steps run, entries] on the device."""
        return self.runner.decode_steps(entries, steps)

    def profiled_step(self, entries: Sequence[StepEntry], profiler, select: Optional[str] = None,
                      filler_ms: float = 0.0) -> Optional[torch.Tensor]:
        """One step launched part by part with `profiler` (ops.profile.Profiler) active: its table
        then holds milliseconds, bytes and flops per kernel class.  `filler_ms` of filler work is
        queued first, so that the host's launch latency does not land inside the spans of short
        kernels (wanted for decode steps)."""
        graphs, self.runner.decode_graphs = self.runner.decode_graphs, False
        try:
            return profiler.run(lambda: self.runner.step(entries, select=select), filler_ms, self.device)
        finally:
            self.runner.decode_graphs = graphs

    # -- generation -------------------------------------------------------------
    def _sampling_params(self, n: int, params, max_new_tokens, temperature, seeds, stop_token_ids) -> List[SamplingParams]:
        plist: List[SamplingParams] = []
        for i in range(n):
            if isinstance(params, SamplingParams):
                p = SamplingParams(**{**params.__dict__})
            elif params is not None:
                p = params[i]
            else:
                p = SamplingParams(temperature=0.0)
            if max_new_tokens is not None:
                p.max_new_tokens = int(max_new_tokens)
            if temperature is not None:
                p.temperature = float(temperature)
            if seeds is not None:
                p.seed = int(seeds[i])
            if stop_token_ids is not None:
                p.stop_token_ids = tuple(int(t) for t in stop_token_ids)
            plist.append(p)
        return plist

    @property
    def queue_depth(self) -> int:
        """Requests waiting to be admitted (reference: IInferenceEngine.cs:15)."""
        return len(self._sched.waiting) if self._sched is not None else 0

    @property
    def active_requests(self) -> int:
        """Requests being generated (reference: IInferenceEngine.cs:18)."""
        return len(self._sched.running) if self._sched is not None else 0

    def generate_chunks(self, prompts: Sequence[Sequence[int]],
                        params: Union[SamplingParams, Sequence[SamplingParams], None] = None, *,
                        max_new_tokens: Optional[int] = None, temperature: Optional[float] = None,
                        seeds: Optional[Sequence[int]] = None, stop_token_ids: Optional[Sequence[int]] = None,
                        should_cancel: Optional[Callable[[int], bool]] = None) -> Iterator[GenerateChunk]:
        """Generate for a list of prompts (token ids) under continuous batching and yield what
        happens as it happens, in the reference's typed chunks
        (reference: src/SharpInference.Engine/GenerateChunk.cs:9-53): per prompt one ``usage``
        chunk with its number of prompt tokens before anything else of it, a ``token`` chunk per
        generated token (the reference's text chunk; there is no tokenizer here), and one ``stop``
        chunk when it ends.  ``should_cancel(index)`` is asked before every step, as the
        reference's cancellation token is; a cancelled prompt ends with reason "abort".  A request
        stops at the configuration's end-of-generation tokens unless its ``stop_token_ids``
        (or the argument here) replace them, as in the reference (Sampler.cs:724-741).  Closing
        the generator early gives every page back."""
        if self._sched is not None:
            raise RuntimeError("a generation is running on this engine: requests are admitted by one loop at a time")
        plist = self._sampling_params(len(prompts), params, max_new_tokens, temperature, seeds, stop_token_ids)
        sched = Scheduler(self.cache, self.max_num_seqs, self.max_tokens_per_step, self.max_model_len,
                          end_of_generation=self.config.eos_token_ids)
        reqs = [Request(("gen", i), [int(t) for t in prompt], plist[i]) for i, prompt in enumerate(prompts)]
        for r in reqs:
            sched.add(r)
        stats = GenerationStats()
        self.last_stats = stats
        self._sched = sched
        reported = 0                                       # finished requests already told of
        try:
            for i, r in enumerate(reqs):
                yield GenerateChunk("usage", i, prompt_tokens=len(r.prompt))
            while sched.has_work():
                if should_cancel is not None:
                    for i, r in enumerate(reqs):
                        if not r.finished and not r.cancelled and should_cancel(i):
                            r.cancelled = True
                batch = sched.schedule()
                if batch:
                    t0 = time.perf_counter()
                    entries = [StepEntry(s.request.req_id, s.tokens, (len(s.tokens) - 1,) if s.samples else ())
                               for s in batch]
                    sampling = [s for s in batch if s.samples]
                    tokens: List[Optional[int]] = [None] * len(batch)
                    ahead = self._steps_ahead(sched, batch, should_cancel)
                    if ahead > 1:
                        # Every request decodes greedily and nobody waits: several steps on end, each
                        # launched on what the one before chose; the scheduler is then told of them
                        # step by step, exactly as if each had been waited for.
                        rows = self.runner.decode_steps(entries, ahead).cpu().tolist()
                        col = {s.request.req_id: j for j, s in enumerate(batch)}
                        dt = (time.perf_counter() - t0) / len(rows)
                        for i, row in enumerate(rows):
                            if i > 0:
                                batch = sched.schedule()       # the requests that are still running, in their order
                                if not batch:
                                    break
                            stats.decode_tokens += len(batch)
                            stats.decode_seconds += dt
                            stats.steps += 1
                            had = [len(s.request.output) for s in batch]
                            sched.update(batch, [row[col[s.request.req_id]] for s in batch])
                            for s, n0 in zip(batch, had):
                                if len(s.request.output) > n0:
                                    yield GenerateChunk("token", s.request.req_id[1], token_id=s.request.output[-1])
                            for r in sched.finished[reported:]:
                                yield GenerateChunk("stop", r.req_id[1], finish_reason=r.finish_reason,
                                                    truncated_by_max_tokens=r.finish_reason == "length")
                            reported = len(sched.finished)
                        continue
                    if sampling and all(s.request.params.greedy for s in sampling):
                        # every row greedy: the choice is made on the device behind the head, and only
                        # the token ids come back (reference: ContinuousBatchingEngine.cs:332-347)
                        picked = self.runner.step(entries, select="argmax").cpu().tolist()
                    else:
                        logits = self.runner.step(entries)
                        picked = []
                        if sampling:
                            hist = [penalty_window(s.request.params, s.request.prompt, s.request.output)
                                    if s.request.params.edits_logits else () for s in sampling]
                            picked = self.sampler.sample(logits, [s.request.params for s in sampling],
                                                         [s.request.draws for s in sampling], hist)
                    if sampling:
                        it = iter(picked)
                        tokens = [next(it) if s.samples else None for s in batch]
                    dt = time.perf_counter() - t0
                    n_prefill = sum(len(s.tokens) for s in batch if s.request.in_prefill)
                    n_decode = sum(1 for s in batch if not s.request.in_prefill)
                    if n_prefill:
                        stats.prefill_tokens += n_prefill
                        stats.prefill_seconds += dt * n_prefill / (n_prefill + n_decode)
                    if n_decode:
                        stats.decode_tokens += n_decode
                        stats.decode_seconds += dt * n_decode / (n_prefill + n_decode)
                    stats.steps += 1
                    had = [len(s.request.output) for s in batch]
                    sched.update(batch, tokens)
                    for s, n0 in zip(batch, had):
                        if len(s.request.output) > n0:
                            yield GenerateChunk("token", s.request.req_id[1], token_id=s.request.output[-1])
                elif sched.has_work() and len(sched.finished) == reported:
                    raise RuntimeError("scheduler has work but nothing can run")
                for r in sched.finished[reported:]:
                    yield GenerateChunk("stop", r.req_id[1], finish_reason=r.finish_reason,
                                        truncated_by_max_tokens=r.finish_reason == "length")
                reported = len(sched.finished)
            for r in sched.finished[reported:]:            # what the last scheduling pass ended without a step
                yield GenerateChunk("stop", r.req_id[1], finish_reason=r.finish_reason,
                                    truncated_by_max_tokens=r.finish_reason == "length")
        finally:
            self._sched = None
            for r in list(sched.running):                  # an error or an early close: give everything back
                if self.cache.has_request(r.req_id):
                    self.cache.free_request(r.req_id)

    def _steps_ahead(self, sched: Scheduler, batch, should_cancel) -> int:
        """How many decode steps may be launched on end for this batch: more than one only while
        the batch holds every running request and each of them decodes greedily, nobody waits to
        be admitted or can be cancelled in between, and no request would pass its own limit (a
        request that meets a stop token on the way is ended there; the steps run past it are
        dropped with its pages).  With a token budget below the number of running requests the
        batch changes from step to step, so every step is scheduled on its own."""
        if self.decode_run_ahead <= 1 or should_cancel is not None or sched.waiting or not batch:
            return 1
        if len(batch) != len(sched.running):
            return 1
        steps = self.decode_run_ahead
        for s in batch:
            r = s.request
            if r.in_prefill or not s.samples or len(s.tokens) != 1 or not r.params.greedy:
                return 1
            steps = min(steps, r.params.max_new_tokens - len(r.output),
                        self.max_model_len - (len(r.prompt) + len(r.output)))
        return max(1, steps)

    def generate(self, prompts: Sequence[Sequence[int]], params: Union[SamplingParams, Sequence[SamplingParams], None] = None,
                 *, max_new_tokens: Optional[int] = None, temperature: Optional[float] = None,
                 seeds: Optional[Sequence[int]] = None, stop_token_ids: Optional[Sequence[int]] = None) -> List[GenerationResult]:
        """Generate for a list of prompts (token ids) under continuous batching; the chunks of
        ``generate_chunks`` gathered per prompt."""
        out = [GenerationResult([], "abort", len(p)) for p in prompts]
        for c in self.generate_chunks(prompts, params, max_new_tokens=max_new_tokens, temperature=temperature,
                                      seeds=seeds, stop_token_ids=stop_token_ids):
            if c.kind == "token":
                out[c.index].token_ids.append(c.token_id)
            elif c.kind == "stop":
                out[c.index].finish_reason = c.finish_reason
        return out
