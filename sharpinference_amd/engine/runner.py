"""The step function: one batch of (request, its next tokens) through the model, from the cache.

The reference has three batched entry points that never mix prompt portions with decoded
tokens (reference: src/SharpInference.Engine/IBatchedForwardPass.cs:27-69;
src/SharpInference.Engine/ContinuousBatchingEngine.cs:306-347).  Here there is one: a step takes
any number of entries, each a request with one or more next tokens, runs exactly those tokens
as one flat batch against what earlier steps left in the cache, and returns float32 logits at
the wanted places.  Lengths advance only when the step has run (the reference is transactional
in the same way, src/SharpInference.Engine/CudaForwardPass.cs:4894, 4985-4986).
"""
from __future__ import annotations

import gc
import sys
from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheError, CacheManager
from ..parts.base import GroupView, HostStep, LayerCache, StepContext


MAX_GRAPH_BATCH = 64   # decode steps of up to this many requests are replayed from a HIP graph (at 64 the host's part of an eager step is still a tenth of the step)
GRAPH_AT_ONCE = 16     # up to this many requests a graph is captured when its shape is first met; wider ones once the
GRAPH_AFTER_ASKS = 4   # shape has been met this often (a graph per width costs capture time and memory of its own)
MAX_GRAPHS = 48        # graphs kept at a time; beyond, the one replayed longest ago is dropped (and captured again if its shape returns)
GRAPH_CONTEXT_MIN = 4096   # a graph is captured for a bound on the contexts of its requests: this, or 4, 16, 64 ... times it
N_OWN = 7              # index arrays of the step function's own, first in the upload (tokens ... logit rows)


class CacheExhausted(CacheError):
    """A step needed more pages than the pools hold; nothing was changed."""


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)   # places among `tokens` whose logits are asked for


class ModelRunner:
    def __init__(self, model, cache: CacheManager, act_dtype: torch.dtype, device, decode_graphs: bool = False,
                 max_context: int = 0):
        self.model = model
        self.cache = cache
        self.act_dtype = act_dtype
        self.device = torch.device(device)
        self.steps_run = 0
        # Steps made of single decoded tokens only are launch-bound: they are captured once per
        # batch size into a HIP graph over fixed index buffers and replayed.  A mixer with state of
        # its own must say that its step can be captured (``graph_safe``: it walks the entries
        # through the context's device tensors, without a copy to the host); the capture's trial
        # run then works on the cache manager's scratch state slot, so that no request's state moves.
        safe = getattr(model, "decode_graph_safe", None)
        self.decode_graphs = bool(decode_graphs) and max_context > 0 and (
            all(t is None for t in cache.state) or bool(safe and safe()))
        self.max_context = int(max_context)
        # what the model's parts want made once a step beside the step's own index arrays (attention: its
        # kernels' work lists); the step function uploads them and knows nothing of their meaning
        self.planners = list(getattr(model, "step_planners", list)())
        self._graphs: dict = {}
        self._graph_pool = None      # one memory pool for every graph of this runner (made with the first capture)
        self._graph_asks: dict = {}
        self.graph_replays = 0

    # ------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        seen = set()
        vocab = self.model.vocab_size
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if not self.cache.has_request(e.req_id):
                raise ValueError(f"request {e.req_id!r} is not in the cache (add_request first)")
            if len(e.tokens) == 0:
                raise ValueError(f"request {e.req_id!r} brings no tokens")
            for t in e.tokens:
                if not 0 <= int(t) < vocab:
                    raise ValueError(f"request {e.req_id!r}: token id {t} outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} outside its {len(e.tokens)} tokens")

    def _host_arrays(self, entries: Sequence[StepEntry], static_blocks: Optional[int] = None):
        """Host side of a step: lay the batch out flat.  Returns the index arrays in upload order
        and what the context needs to know about them."""
        cache = self.cache
        ps = cache.page_size
        n = len(entries)
        lens = [len(e.tokens) for e in entries]
        starts = [cache.length(e.req_id) for e in entries]
        T = sum(lens)
        if T == n:
            # single tokens only (a decode step): no loop over the entries' tokens
            token_ids = np.fromiter((e.tokens[0] for e in entries), dtype=np.int32, count=n)
            positions = np.asarray(starts, dtype=np.int32)
            entry_of = np.arange(n, dtype=np.int32)
            cu = np.arange(n + 1, dtype=np.int32)
            rows = [i for i, e in enumerate(entries) for _ in e.want]
        else:
            token_ids = np.empty(T, dtype=np.int32)
            positions = np.empty(T, dtype=np.int32)
            entry_of = np.empty(T, dtype=np.int32)
            cu = np.zeros(n + 1, dtype=np.int32)
            rows = []
            o = 0
            for i, e in enumerate(entries):
                L = lens[i]
                token_ids[o:o + L] = np.asarray(e.tokens, dtype=np.int32)
                positions[o:o + L] = np.arange(starts[i], starts[i] + L, dtype=np.int32)
                entry_of[o:o + L] = i
                rows.extend(o + int(w) for w in e.want)
                o += L
                cu[i + 1] = o
        state_slots = np.asarray([cache.requests[e.req_id].state_slot for e in entries], dtype=np.int32)
        group_tables, group_slots = [], []
        block_of = positions // ps
        for g in range(len(cache.groups)):
            tables = [cache.block_table_array(e.req_id, g) for e in entries]
            if static_blocks is not None:
                maxb = static_blocks
            else:
                maxb = max(1, max(t.size for t in tables))
                maxb = (maxb + 3) // 4 * 4
            bt = np.full((n, maxb), -1, dtype=np.int32)
            for i, t in enumerate(tables):
                bt[i, :t.size] = t
            pages = bt[entry_of, block_of]          # every token's page, at once
            if T and int(pages.min()) < 0:
                i = int(entry_of[int(np.argmin(pages))])
                raise CacheError(f"request {entries[i].req_id!r}: a new position has no page in group {g}")
            sm = (pages * ps + positions % ps).astype(np.int32, copy=False)
            group_tables.append(bt)
            group_slots.append(sm)
        rows_np = np.asarray(rows, dtype=np.int32)
        # what the parts' planners want, then the groups' block tables and slots
        host = HostStep(n_entries=n, n_tokens=T, lens=lens, starts=starts, cu_tokens=cu)
        pieces = [token_ids, positions, entry_of, cu, state_slots, np.full(T, -1, dtype=np.int32), rows_np]
        planned = []                                  # per planner: (number of arrays, host facts)
        for pl in self.planners:
            arrays, facts = pl.plan(host)
            arrays = [np.ascontiguousarray(a, dtype=np.int32).reshape(-1) for a in arrays]
            planned.append((len(arrays), facts))
            pieces += arrays
        n_planned = len(pieces) - N_OWN
        for bt, sm in zip(group_tables, group_slots):
            pieces += [bt.reshape(-1), sm]
        info = dict(n=n, T=T, lens=lens, starts=starts, n_rows=len(rows), planned=planned, n_planned=n_planned, host=host,
                    max_blocks=[bt.shape[1] for bt in group_tables],
                    max_context=int(positions.max()) + 1 if T else 0)
        return pieces, info

    def _context_from(self, dev: torch.Tensor, sizes: Sequence[int], info: dict):
        """The step's context over one device tensor that holds the index arrays back to back."""
        views, off = [], 0
        for size in sizes:
            views.append(dev[off:off + size])
            off += size
        d_tok, d_pos, d_ent, d_cu, d_state, d_nostore, d_rows = views[:N_OWN]
        n, T = info["n"], info["T"]
        first_group = N_OWN + info["n_planned"]
        groups = []
        for g in range(len(self.cache.groups)):
            bt = views[first_group + 2 * g].view(n, info["max_blocks"][g])
            groups.append(GroupView(bt, views[first_group + 1 + 2 * g], self.cache.page_size, max_context=info["max_context"]))
        ctx = StepContext(n_tokens=T, n_entries=n, token_ids=d_tok, positions=d_pos, entry_of_token=d_ent,
                          cu_tokens=d_cu, state_slots=d_state, groups=groups, act_dtype=self.act_dtype,
                          no_store_slots=d_nostore, entry_lens=info["lens"], entry_starts=info["starts"],
                          max_entry_len=max(info["lens"]) if info["lens"] else 1)
        at = N_OWN
        for pl, (count, facts) in zip(self.planners, info["planned"]):
            pl.attach(ctx, views[at:at + count], facts)
            at += count
        return ctx, (d_rows if info["n_rows"] else None)

    def build_context(self, entries: Sequence[StepEntry]):
        """Index arrays of a step packed into ONE upload, and the context over them."""
        pieces, info = self._host_arrays(entries)
        flat = np.concatenate(pieces) if pieces else np.zeros(0, dtype=np.int32)
        dev = torch.from_numpy(flat).to(self.device)
        return self._context_from(dev, [p.size for p in pieces], info)

    def layer_caches(self, ctx: StepContext) -> List[LayerCache]:
        cache = self.cache
        out = []
        for i in range(len(cache.slot_specs)):
            g = cache.group_of_slot[i]
            out.append(LayerCache(group=ctx.groups[g] if g >= 0 else None, k=cache.k[i], v=cache.v[i],
                                  state=cache.state[i], write=True))
        return out

    # ------------------------------------------------------------------
    def _decode_graph_step(self, entries: Sequence[StepEntry], router_trace: Optional[list] = None,
                           select: Optional[str] = None, device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Replay the captured graph of this batch size if the step qualifies: every entry one
        token whose logits are wanted, all contexts within the captured bound.  None otherwise."""
        n = len(entries)
        if not self.decode_graphs or n > MAX_GRAPH_BATCH:
            return None
        longest = 0
        for e in entries:
            if len(e.tokens) != 1 or len(e.want) != 1 or int(e.want[0]) != 0:
                return None
            longest = max(longest, self.cache.length(e.req_id) + 1)
        if longest > self.max_context:
            return None
        # The graph's shapes are fixed at a bound on the contexts (block table width, runs of the
        # decode kernel); a bound far above the contexts costs time, so bounds grow in steps of 4
        bound = GRAPH_CONTEXT_MIN
        while bound < longest:
            bound *= 4
        bound = min(bound, self.max_context)
        key = (n, bound) if select is None else (n, bound, select)
        graph = self._graphs.get(key)
        if graph is False:
            return None
        if graph is None and n > GRAPH_AT_ONCE:
            asks = self._graph_asks.get(key, 0) + 1
            self._graph_asks[key] = asks
            if asks < GRAPH_AFTER_ASKS:
                return None
        static_blocks = (bound + self.cache.page_size - 1) // self.cache.page_size
        pieces, info = self._host_arrays(entries, static_blocks=static_blocks)
        if graph is None:
            try:
                if self._graph_pool is None:
                    self._graph_pool = torch.cuda.graph_pool_handle()
                graph = _DecodeGraph(self, pieces, info, bound, select, pool=self._graph_pool)
            except Exception as e:  # noqa: BLE001 - capture is an optimisation: report once, go on eagerly
                print(f"[sharpi] decode graph for batch {n}, contexts to {bound} not captured ({type(e).__name__}: {e}); "
                      "running eagerly", file=sys.stderr, flush=True)
                self._graphs[key] = False
                return None
            self._graphs[key] = graph
            live = [k for k, g in self._graphs.items() if g is not False]
            if len(live) > MAX_GRAPHS:          # (the dict keeps the order of last use: see below)
                del self._graphs[live[0]]
                self._graph_asks.pop(live[0], None)
        else:
            self._graphs[key] = self._graphs.pop(key)     # moved to the end: the most recently used
        self.graph_replays += 1
        return graph.replay(pieces, router_trace, device_tokens)

    def step(self, entries: Sequence[StepEntry], router_trace: Optional[list] = None,
             select: Optional[str] = None, device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Run one batch.  Returns float32 logits [wanted, vocab] in the order of the entries and
        of their ``want`` lists, or None when nothing is wanted; with ``select="argmax"`` the index
        of each wanted row's largest logit instead (int32 [wanted]), so that only token ids leave
        the device.  ``device_tokens`` (int32 [entries], on the device; every entry one token):
        the token ids are taken from there instead of from the entries, whose own are then only
        placeholders: a step can be launched on what the step before chose before the host has
        seen it.  A list given as ``router_trace``
        receives, per routed layer run, the (expert ids, weights, router input) of the step's tokens,
        as the reference can print its router picks (src/SharpInference.Engine/ForwardPass.cs:2042-2056)."""
        if not entries:
            return None
        self._validate(entries)
        appended = []
        try:
            for e in entries:
                if not self.cache.append(e.req_id, len(e.tokens)):
                    raise CacheExhausted(f"no pages left for request {e.req_id!r} ({len(e.tokens)} more tokens)")
                appended.append(e.req_id)
            if device_tokens is not None:
                if any(len(e.tokens) != 1 for e in entries) or device_tokens.shape != (len(entries),) \
                        or device_tokens.dtype != torch.int32 or not device_tokens.is_cuda:
                    raise ValueError("device_tokens: one int32 token per single-token entry, on the engine's device")
            logits = self._decode_graph_step(entries, router_trace, select, device_tokens)
            if logits is None:
                ctx, rows = self.build_context(entries)
                if device_tokens is not None:
                    ctx.token_ids.copy_(device_tokens)
                if router_trace is not None:
                    ctx.extras["router_trace"] = router_trace
                logits = self.model.forward(ctx, self.layer_caches(ctx), rows, select) if select else \
                    self.model.forward(ctx, self.layer_caches(ctx), rows)
        except BaseException:
            for r in appended:
                self.cache.rollback(r)
            raise
        for e in entries:
            self.cache.commit(e.req_id)
        self.steps_run += 1
        return logits


    def decode_steps(self, entries: Sequence[StepEntry], steps: int) -> torch.Tensor:
        """`steps` greedy decode steps of the same requests, run ahead of the host: the first takes
        the entries' own tokens, every later one what the step before chose, on the device, so
        that the host prepares and launches a step while the one before it still runs and reads
        nothing back in between.  Returns the chosen tokens, int32 [steps, entries], on the
        device.  Fewer steps are run if the pages do not reach (at least one, or CacheExhausted
        as in ``step``)."""
        if not entries or steps <= 0:
            raise ValueError("decode_steps needs entries and at least one step")
        if any(len(e.tokens) != 1 for e in entries):
            raise ValueError("decode_steps: every entry brings one token")
        chosen: List[torch.Tensor] = []
        ahead = [StepEntry(e.req_id, (0,), (0,)) for e in entries]
        for i in range(steps):
            try:
                out = self.step(entries if i == 0 else ahead, select="argmax",
                                device_tokens=None if i == 0 else chosen[-1])
            except CacheExhausted:
                if i == 0:
                    raise
                break
            chosen.append(out)
        return torch.stack(chosen)


class _DecodeGraph:
    """One captured decode step of a fixed batch size over fixed index buffers.

    The index arrays of a step are written into a pinned host buffer, copied into the device
    buffer the graph was captured over, and the graph is replayed; shapes that vary from step to
    step (block table width, context bound of the decode kernel) are fixed at ``max_context``.
    The logits tensor belongs to the graph: the caller gets a copy."""

    def __init__(self, runner: ModelRunner, pieces, info: dict, max_context: int, select: Optional[str] = None,
                 pool=None):
        self.sizes = [p.size for p in pieces]
        total = sum(self.sizes)
        self.host = torch.empty(total, dtype=torch.int32).pin_memory()
        self.host_np = self.host.numpy()
        self.dev = torch.empty(total, dtype=torch.int32, device=runner.device)
        self.copied = torch.cuda.Event()
        info = dict(info, max_context=max_context)
        # capture over harmless contents: nothing is stored (slots -1) and no key is visible (tables -1)
        null = [np.zeros_like(p) for p in pieces]
        n = info["n"]
        null[2] = np.arange(n, dtype=np.int32)            # entry of token
        null[3] = np.arange(n + 1, dtype=np.int32)        # cu_tokens
        null[4] = np.full_like(pieces[4], runner.cache.scratch_state_slot)   # state: the slot of no request
        null[5] = np.full(n, -1, dtype=np.int32)
        null[6] = np.arange(n, dtype=np.int32)            # logit rows
        at = N_OWN
        for pl, (count, _) in zip(runner.planners, info["planned"]):      # the planners' own harmless contents
            null[at:at + count] = [np.ascontiguousarray(a, dtype=np.int32).reshape(-1)
                                   for a in pl.null(info["host"], pieces[at:at + count])]
            at += count
        for i in range(at, len(null)):                    # block tables and slots
            null[i] = np.full_like(pieces[i], -1)
        self._upload(null)
        ctx, rows = runner._context_from(self.dev, self.sizes, info)
        caches = runner.layer_caches(ctx)
        side = torch.cuda.Stream(device=runner.device)
        side.wait_stream(torch.cuda.current_stream())
        args = (ctx, caches, rows, select) if select else (ctx, caches, rows)
        with torch.cuda.stream(side):                     # once eagerly: libraries initialise outside the capture
            runner.model.forward(*args)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        # A fresh context for the captured run: what the trial run's parts kept in the context (tensors
        # they make once a step) was made outside the graph and would never be made again.
        ctx, rows = runner._context_from(self.dev, self.sizes, info)
        caches = runner.layer_caches(ctx)
        args = (ctx, caches, rows, select) if select else (ctx, caches, rows)
        # the captured run also notes where its router picks lie (tensors of the graph's own memory,
        # filled anew by every replay), so that a replayed step can be traced like a launched one
        self.trace: list = []
        ctx.extras["router_trace"] = self.trace
        self.graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is capturing: a collector run that frees another
        # engine's graph (or anything else that calls into the runtime) in the middle of a capture
        # aborts the process.  (This object holds no reference to the runner, so that an engine
        # that is dropped frees its graphs at once, by reference count, not in some later collection.)
        collecting = gc.isenabled()
        gc.disable()
        try:
            # One pool for all of a runner's graphs: they are replayed one after the other on one
            # stream and their results are copied out before the next replay, so what one graph's
            # intermediate tensors held another's may hold; with a pool each, every shape a served
            # process meets would keep its own activations and logits for good.
            with torch.cuda.graph(self.graph, pool=pool):
                self.logits = runner.model.forward(*args)
        finally:
            if collecting:
                gc.enable()

    def _upload(self, pieces) -> None:
        self.copied.synchronize()                         # the previous copy has left the pinned buffer
        off = 0
        for p, size in zip(pieces, self.sizes):
            assert p.size == size
            self.host_np[off:off + size] = p.reshape(-1)
            off += size
        self.dev.copy_(self.host, non_blocking=True)
        self.copied.record()

    def replay(self, pieces, router_trace: Optional[list] = None,
               device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        self._upload(pieces)
        if device_tokens is not None:                    # the token ids lie first in the buffer
            self.dev[:self.sizes[0]].copy_(device_tokens)
        self.graph.replay()
        if router_trace is not None:
            router_trace.extend(tuple(t.clone() for t in item) for item in self.trace)
        return self.logits.clone()
