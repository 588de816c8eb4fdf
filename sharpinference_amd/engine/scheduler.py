"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.

Shape of the reference's batcher (reference: src/SharpInference.Engine/ContinuousBatchingEngine.cs):
FIFO admission that reserves the request's whole need of cache up front and stops at the first
request that does not fit while others run (511-580); a per-iteration token budget spread over
the prompts still being read (625-645); the first token sampled from the prompt's last logits,
a stop token ending the request before anything is emitted (722-827, and
src/SharpInference.Cli/RunCommand.cs:2276); a request ends on a stop token or at its token limit
and its cache goes back at once (394-407, 697-714).

Unlike the reference, one step carries decode tokens and prompt portions together: every
decoding request first gets its one token, what is left of the budget goes to prompts in
arrival order.  The reference decodes every active sequence in every iteration (314-347);
where the token budget is smaller than the number of requests that want a token, the ones
that have waited longest go first with one token each, so that all of them advance within
one step of each other.

When pages run out: they cannot for a running request, because admission reserved the pages it
can ever hold.  A waiting request waits until enough reservations are returned.  A request
that would not fit even with the pools to itself is finished at once with reason "too_long"
rather than admitted to fail later (the reference admits it alone, 505-510).

The scheduler owns no device memory and calls no kernel: it can be driven with a scripted
step function.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Hashable, List, Optional, Sequence

from ..cache.manager import CacheManager
from ..sampling.params import SamplingParams

FINISH_STOP, FINISH_LENGTH, FINISH_TOO_LONG, FINISH_ABORT = "stop", "length", "too_long", "abort"


@dataclass
class Request:
    req_id: Hashable
    prompt: List[int]
    params: SamplingParams
    output: List[int] = field(default_factory=list)
    num_computed: int = 0             # tokens of prompt + output that have been through the model
    finish_reason: Optional[str] = None
    cancelled: bool = False
    draws: int = 0                    # uniforms used so far
    stops: frozenset = frozenset()    # tokens that end it (its own and the model's), set on admission to the queue
    last_step: int = -1               # ticket of the scheduling pass that last gave it tokens

    @property
    def finished(self) -> bool:
        return self.finish_reason is not None

    @property
    def in_prefill(self) -> bool:
        return self.num_computed < len(self.prompt)


@dataclass
class Scheduled:
    request: Request
    tokens: List[int]
    samples: bool                     # this entry's last token yields the request's next token


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_tokens_per_step: int, max_model_len: int,
                 end_of_generation: Sequence[int] = ()):
        if max_tokens_per_step < 1 or max_num_seqs < 1:
            raise ValueError("max_tokens_per_step and max_num_seqs must be positive")
        if max_num_seqs > cache.max_requests:
            raise ValueError(f"max_num_seqs {max_num_seqs} exceeds the cache's {cache.max_requests} state slots")
        self.cache = cache
        self.max_num_seqs = max_num_seqs
        self.max_tokens_per_step = max_tokens_per_step
        self.max_model_len = max_model_len
        self.end_of_generation = tuple(int(t) for t in end_of_generation)   # the model's own stop tokens
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self.finished: List[Request] = []
        self._tickets = 0                                # one per request and scheduling pass, in the order served

    # ------------------------------------------------------------------
    def add(self, request: Request) -> None:
        if not request.prompt:
            raise ValueError(f"request {request.req_id!r} has an empty prompt")
        request.stops = request.params.stop_set(self.end_of_generation)
        self.waiting.append(request)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _need(self, r: Request) -> int:
        return min(len(r.prompt) + r.params.max_new_tokens, self.max_model_len)

    def _finish(self, r: Request, reason: str, held: bool) -> None:
        r.finish_reason = reason
        if held:
            self.cache.free_request(r.req_id)
            self.running.remove(r)
        self.finished.append(r)

    def _admit(self) -> None:
        while self.waiting and len(self.running) < self.max_num_seqs:
            r = self.waiting[0]
            if r.cancelled:
                self.waiting.popleft()
                self._finish(r, FINISH_ABORT, held=False)
                continue
            need = self._need(r)
            if len(r.prompt) >= self.max_model_len or not self.cache.fits_alone(need, self.max_tokens_per_step):
                self.waiting.popleft()
                self._finish(r, FINISH_TOO_LONG, held=False)
                continue
            if r.params.max_new_tokens == 0:
                self.waiting.popleft()
                self._finish(r, FINISH_LENGTH, held=False)
                continue
            if not self.cache.can_admit(need, self.max_tokens_per_step):
                break                                    # FIFO: nobody overtakes the head of the line
            self.waiting.popleft()
            self.cache.add_request(r.req_id, reserve_tokens=need, max_step_tokens=self.max_tokens_per_step)
            self.running.append(r)

    def schedule(self) -> List[Scheduled]:
        """The next step's batch (empty if nothing can run)."""
        for r in [r for r in self.running if r.cancelled]:
            self._finish(r, FINISH_ABORT, held=True)
        self._admit()
        budget = self.max_tokens_per_step
        batch: List[Scheduled] = []
        decoders = [r for r in self.running if not r.in_prefill]
        prompts = [r for r in self.running if r.in_prefill]
        if len(decoders) > budget or (prompts and len(decoders) == budget):
            # fewer tokens than requests that want one: one token each to those left out longest
            # (the sort is stable, so equals keep their arrival order); the batch keeps the running
            # order, and a prompt advances by a one-token portion
            turn = sorted(self.running, key=lambda r: r.last_step)[:budget]
            chosen = set(id(r) for r in turn)
            decoders = [r for r in decoders if id(r) in chosen]
            prompts = [r for r in prompts if id(r) in chosen]
            share = 1
        else:
            share, turn = None, None
        for r in decoders:                               # decoding requests first: one token each
            batch.append(Scheduled(r, [r.output[-1]], True))
            budget -= 1
        for r in prompts:                                # then prompts, in arrival order
            if budget > 0:
                take = min(len(r.prompt) - r.num_computed, share or budget)
                toks = r.prompt[r.num_computed:r.num_computed + take]
                batch.append(Scheduled(r, toks, r.num_computed + take == len(r.prompt)))
                budget -= take
        for r in turn if turn is not None else [s.request for s in batch]:
            r.last_step = self._tickets                  # strictly increasing: a round robin, no ties
            self._tickets += 1
        return batch

    def update(self, batch: Sequence[Scheduled], sampled: Sequence[Optional[int]]) -> List[Request]:
        """After the step: `sampled[i]` is the token drawn for batch[i] (None if it did not
        sample).  Returns the requests that finished."""
        done: List[Request] = []
        for s, tok in zip(batch, sampled):
            r = s.request
            r.num_computed += len(s.tokens)
            if not s.samples:
                continue
            assert tok is not None
            r.draws += 0 if r.params.greedy else 1
            if tok in r.stops:
                self._finish(r, FINISH_STOP, held=True)   # the stop token is not emitted
                done.append(r)
                continue
            r.output.append(int(tok))
            if len(r.output) >= r.params.max_new_tokens or len(r.prompt) + len(r.output) >= self.max_model_len:
                self._finish(r, FINISH_LENGTH, held=True)
                done.append(r)
        return done
