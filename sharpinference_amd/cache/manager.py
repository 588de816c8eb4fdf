"""The cache manager: pages with a block table per request, and slots of fixed-size state.

Layers are sorted into *groups* by what they need of the past (all keys; a chunk or a sliding
window of them).  A group has its own pool of pages and, per request, its own block table:
entry b names the page that holds positions [b * page_size, (b + 1) * page_size) or -1.  Every
layer of a group uses the same page ids in its own tensor, as the reference shares one slot
index across layers (reference: src/SharpInference.Engine/PagedKvCache.cs:34-44, 144-148); unlike the
reference, the pools are shared by all requests.  Pages return to the pool when a request ends
and, in a windowed group, as soon as no later query can see them; nothing is cleared on
release (lengths and block tables mask stale contents).  Requests also hold one *state slot*
each: an index into per-layer tensors of fixed size, zeroed at admission
(reference: src/SharpInference.Engine/GdnStateCache.cs:7-33).

All bookkeeping is host-side and independent of the device tensors, so it can be exercised
without a GPU (``allocate=False``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Union

import numpy as np
import torch

from .spec import KVSpec, StateSpec


class CacheError(RuntimeError):
    pass


def pages_to_hold(spec: KVSpec, page_size: int, total_tokens: int, max_step_tokens: int) -> int:
    """Upper bound of the pages a request of `total_tokens` holds at once under `spec` when no step
    brings more than `max_step_tokens` of it: all of them without a window; with one, the window,
    the step that is being appended before the pages behind the window are given back, and one
    page for the edges."""
    full = (total_tokens + page_size - 1) // page_size
    if spec.window_kind == 0:
        return full
    span = spec.window + max(1, max_step_tokens)
    return min(full, (span + page_size - 1) // page_size + 1)


def pool_sizes(slot_specs, page_size: int, max_requests: int, total_tokens: int, max_step_tokens: int,
               budget_pages: Optional[int] = None) -> Dict[tuple, int]:
    """Pages per group for `max_requests` requests of up to `total_tokens` each: a group without
    a window gets them all (or `budget_pages`, if that is less), a windowed group what its window
    can ever hold, which is what makes its memory bounded however long the requests grow."""
    out: Dict[tuple, int] = {}
    for spec in slot_specs:
        if not isinstance(spec, KVSpec) or spec.group_key() in out:
            continue
        n = max_requests * pages_to_hold(spec, page_size, total_tokens, max_step_tokens)
        if budget_pages is not None:
            n = min(n, budget_pages)
        out[spec.group_key()] = max(1, n)
    return out


class PagePool:
    """Free list of page ids 0..n-1; LIFO, so a page just released is the next handed out."""

    def __init__(self, num_pages: int):
        if num_pages <= 0:
            raise CacheError(f"a page pool needs at least one page (got {num_pages})")
        self.num_pages = num_pages
        self._free: List[int] = list(range(num_pages - 1, -1, -1))
        self._held = [False] * num_pages
        self.total_allocs = 0

    @property
    def num_free(self) -> int:
        return len(self._free)

    def alloc(self) -> Optional[int]:
        if not self._free:
            return None
        p = self._free.pop()
        self._held[p] = True
        self.total_allocs += 1
        return p

    def release(self, page: int) -> None:
        if not (0 <= page < self.num_pages) or not self._held[page]:
            raise CacheError(f"page {page} released but not held")
        self._held[page] = False
        self._free.append(page)

    def is_held(self, page: int) -> bool:
        return self._held[page]


@dataclass
class CacheGroup:
    key: tuple
    spec: KVSpec                      # the window that all layers of the group share
    pool: PagePool
    slots: List[int] = field(default_factory=list)   # cache slots (layers) that belong here


@dataclass
class RequestCache:
    req_id: Hashable
    length: int = 0                   # tokens committed
    pending: int = 0                  # tokens appended for the running step, not yet committed
    state_slot: int = -1
    tables: List[List[int]] = field(default_factory=list)      # per group: block index -> page or -1
    reserved: List[int] = field(default_factory=list)          # per group: pages promised at admission
    changed: List[int] = field(default_factory=list)           # per group: how often the table has changed
    arrays: List[Optional[tuple]] = field(default_factory=list)   # per group: (changed then, the table as int32 array)
    passed: List[int] = field(default_factory=list)            # per group: blocks below this one were given back


class CacheManager:
    def __init__(self, slot_specs: Sequence[Union[KVSpec, StateSpec, None]], page_size: int,
                 num_pages: Union[int, Dict[tuple, int]], max_requests: int, dtype: torch.dtype = torch.float32,
                 device="cpu", allocate: bool = True):
        if page_size <= 0 or page_size % 16 != 0:
            raise CacheError(f"page_size must be a positive multiple of 16 (got {page_size})")
        if max_requests <= 0:
            raise CacheError("max_requests must be positive")
        self.page_size = page_size
        self.max_requests = max_requests
        self.dtype = dtype
        self.device = torch.device(device)
        self.slot_specs = list(slot_specs)
        self.groups: List[CacheGroup] = []
        self.group_of_slot: List[int] = []
        by_key: Dict[tuple, int] = {}
        for i, spec in enumerate(self.slot_specs):
            if isinstance(spec, KVSpec):
                key = spec.group_key()
                if key not in by_key:
                    n = num_pages[key] if isinstance(num_pages, dict) else int(num_pages)
                    by_key[key] = len(self.groups)
                    self.groups.append(CacheGroup(key, KVSpec(0, 0, spec.window_kind, spec.window), PagePool(n)))
                g = by_key[key]
                self.groups[g].slots.append(i)
                self.group_of_slot.append(g)
            else:
                self.group_of_slot.append(-1)
        self._free_state_slots = list(range(max_requests - 1, -1, -1))
        # one more slot than requests: a slot that belongs to no request, for runs whose effects on
        # state must not count (the trial run of a graph capture)
        self.scratch_state_slot = max_requests
        self.requests: Dict[Hashable, RequestCache] = {}
        self._reserved_total = [0] * len(self.groups)
        # device tensors
        self.k: List[Optional[torch.Tensor]] = [None] * len(self.slot_specs)
        self.v: List[Optional[torch.Tensor]] = [None] * len(self.slot_specs)
        self.state: List[Optional[torch.Tensor]] = [None] * len(self.slot_specs)
        if allocate:
            for i, spec in enumerate(self.slot_specs):
                if isinstance(spec, KVSpec):
                    n = self.groups[self.group_of_slot[i]].pool.num_pages
                    # keys [page, kv head, position, head_dim]; values transposed inside the page,
                    # [page, kv head, head_dim, position], the layout the matrix-core kernels read
                    self.k[i] = torch.zeros((n, spec.num_kv_heads, page_size, spec.head_dim), dtype=dtype,
                                            device=self.device)
                    self.v[i] = torch.zeros((n, spec.num_kv_heads, spec.value_dim, page_size), dtype=dtype,
                                            device=self.device)
                elif isinstance(spec, StateSpec):
                    self.state[i] = torch.zeros((max_requests + 1, *spec.shape), dtype=spec.dtype, device=self.device)

    # ------------------------------------------------------------------ sizes
    def bytes_per_page(self) -> List[int]:
        """Per group: bytes of one page across all its layers (keys and values)."""
        width = torch.empty(0, dtype=self.dtype).element_size()
        out = []
        for g in self.groups:
            b = 0
            for s in g.slots:
                spec = self.slot_specs[s]
                b += spec.num_kv_heads * (spec.head_dim + spec.value_dim) * self.page_size * width
            out.append(b)
        return out

    def blocks_for(self, n_tokens: int) -> int:
        return (n_tokens + self.page_size - 1) // self.page_size

    def pages_to_hold(self, group: int, total_tokens: int, max_step_tokens: int) -> int:
        """Upper bound of the pages a request of `total_tokens` holds at once in a group when no
        step brings more than `max_step_tokens` of it."""
        return pages_to_hold(self.groups[group].spec, self.page_size, total_tokens, max_step_tokens)

    # ------------------------------------------------------------------ requests
    def has_request(self, req_id) -> bool:
        return req_id in self.requests

    def can_admit(self, total_tokens: int, max_step_tokens: int) -> bool:
        if not self._free_state_slots:
            return False
        for g, grp in enumerate(self.groups):
            need = self.pages_to_hold(g, total_tokens, max_step_tokens)
            if self._reserved_total[g] + need > grp.pool.num_pages:
                return False
        return True

    def fits_alone(self, total_tokens: int, max_step_tokens: int) -> bool:
        """Could the request ever run, with the pools to itself?"""
        return all(self.pages_to_hold(g, total_tokens, max_step_tokens) <= grp.pool.num_pages
                   for g, grp in enumerate(self.groups))

    def add_request(self, req_id, reserve_tokens: int = 0, max_step_tokens: int = 1) -> RequestCache:
        """Admit a request: a state slot, and (if reserve_tokens > 0) a promise of pages."""
        if req_id in self.requests:
            raise CacheError(f"request {req_id!r} is already in the cache")
        if not self._free_state_slots:
            raise CacheError("no state slot free: too many live requests")
        rc = RequestCache(req_id)
        rc.tables = [[] for _ in self.groups]
        rc.reserved = [0] * len(self.groups)
        rc.changed = [0] * len(self.groups)
        rc.arrays = [None] * len(self.groups)
        rc.passed = [0] * len(self.groups)
        if reserve_tokens > 0:
            if not self.can_admit(reserve_tokens, max_step_tokens):
                raise CacheError(f"request {req_id!r}: not enough pages to reserve {reserve_tokens} tokens")
            for g in range(len(self.groups)):
                rc.reserved[g] = self.pages_to_hold(g, reserve_tokens, max_step_tokens)
                self._reserved_total[g] += rc.reserved[g]
        rc.state_slot = self._free_state_slots.pop()
        for t in self.state:
            if t is not None:
                t[rc.state_slot].zero_()
        self.requests[req_id] = rc
        return rc

    def pages_needed(self, req_id, n_tokens: int) -> List[int]:
        rc = self.requests[req_id]
        start = rc.length + rc.pending
        end = start + n_tokens
        out = []
        for g in range(len(self.groups)):
            tbl = rc.tables[g]
            need = 0
            for b in range(start // self.page_size, self.blocks_for(end)):
                if b >= len(tbl) or tbl[b] < 0:
                    need += 1
            out.append(need)
        return out

    def can_append(self, req_id, n_tokens: int) -> bool:
        need = self.pages_needed(req_id, n_tokens)
        return all(need[g] <= self.groups[g].pool.num_free for g in range(len(self.groups)))

    def append(self, req_id, n_tokens: int) -> bool:
        """Make room for the next `n_tokens` positions in every group; all or nothing."""
        if n_tokens <= 0:
            raise CacheError("append needs at least one token")
        rc = self.requests[req_id]
        if n_tokens == 1:      # a decoded token that lands in a page the request already holds: nothing to find
            b = (rc.length + rc.pending) // self.page_size
            for tbl in rc.tables:
                if b >= len(tbl) or tbl[b] < 0:
                    break
            else:
                rc.pending += 1
                return True
        if not self.can_append(req_id, n_tokens):
            return False
        start = rc.length + rc.pending
        end = start + n_tokens
        for g, grp in enumerate(self.groups):
            tbl = rc.tables[g]
            first = start // self.page_size
            last = self.blocks_for(end)
            if len(tbl) < last:
                tbl.extend([-1] * (last - len(tbl)))
                rc.changed[g] += 1
            for b in range(first, last):
                if tbl[b] < 0:
                    page = grp.pool.alloc()
                    assert page is not None
                    tbl[b] = page
                    rc.changed[g] += 1
        rc.pending += n_tokens
        return True

    def commit(self, req_id) -> int:
        """The step that used the appended positions is done: lengths advance and pages that no
        later query can see go back to their pool.  Returns the number of pages released."""
        rc = self.requests[req_id]
        rc.length += rc.pending
        rc.pending = 0
        released = 0
        for g, grp in enumerate(self.groups):
            if grp.spec.window_kind == 0:
                continue
            first_needed = grp.spec.first_visible(rc.length)   # the next query sits at position `length`
            tbl = rc.tables[g]
            upto = min(first_needed // self.page_size, len(tbl))
            for b in range(rc.passed[g], upto):                # (blocks below `passed` went back in earlier steps)
                if tbl[b] >= 0:
                    grp.pool.release(tbl[b])
                    tbl[b] = -1
                    released += 1
                    rc.changed[g] += 1
            rc.passed[g] = max(rc.passed[g], upto)
        return released

    def rollback(self, req_id) -> None:
        """Forget appended-but-uncommitted positions (a step that failed)."""
        rc = self.requests[req_id]
        if rc.pending == 0:
            return
        keep_blocks = self.blocks_for(rc.length)
        for g, grp in enumerate(self.groups):
            tbl = rc.tables[g]
            for b in range(keep_blocks, len(tbl)):
                if tbl[b] >= 0:
                    grp.pool.release(tbl[b])
                    tbl[b] = -1
            del tbl[keep_blocks:]
            rc.changed[g] += 1
        rc.pending = 0

    def free_request(self, req_id) -> None:
        rc = self.requests.pop(req_id, None)
        if rc is None:
            raise CacheError(f"request {req_id!r} freed but not in the cache")
        for g, grp in enumerate(self.groups):
            for p in rc.tables[g]:
                if p >= 0:
                    grp.pool.release(p)
            self._reserved_total[g] -= rc.reserved[g]
        self._free_state_slots.append(rc.state_slot)

    # ------------------------------------------------------------------ views for a step
    def length(self, req_id) -> int:
        return self.requests[req_id].length

    def block_table(self, req_id, group: int) -> List[int]:
        return self.requests[req_id].tables[group]

    def block_table_array(self, req_id, group: int) -> np.ndarray:
        """The block table as an int32 array (not to be written to), made anew only when the
        table has changed since it was last asked for: a decoding request changes its table once
        a page, not once a step."""
        rc = self.requests[req_id]
        held = rc.arrays[group]
        if held is None or held[0] != rc.changed[group]:
            held = rc.arrays[group] = (rc.changed[group], np.asarray(rc.tables[group], dtype=np.int32))
        return held[1]

    def slots_for(self, req_id, group: int, start: int, n: int) -> List[int]:
        """Flat cache slots (page * page_size + offset) of positions start..start+n-1."""
        tbl = self.requests[req_id].tables[group]
        ps = self.page_size
        out = []
        for pos in range(start, start + n):
            page = tbl[pos // ps] if pos // ps < len(tbl) else -1
            if page < 0:
                raise CacheError(f"request {req_id!r}: position {pos} has no page in group {group}")
            out.append(page * ps + pos % ps)
        return out

    # ------------------------------------------------------------------ checks
    def check_invariants(self) -> None:
        """No page lost, none held twice, free lists and tables agree."""
        for g, grp in enumerate(self.groups):
            seen: Dict[int, Hashable] = {}
            for rc in self.requests.values():
                for p in rc.tables[g]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise CacheError(f"group {g}: page {p} held by {seen[p]!r} and {rc.req_id!r}")
                    if not grp.pool.is_held(p):
                        raise CacheError(f"group {g}: page {p} in a table but on the free list")
                    seen[p] = rc.req_id
            free = grp.pool._free
            if len(set(free)) != len(free):
                raise CacheError(f"group {g}: a page is on the free list twice")
            if len(seen) + len(free) != grp.pool.num_pages:
                raise CacheError(f"group {g}: {grp.pool.num_pages - len(seen) - len(free)} page(s) lost")
            if set(free) & set(seen):
                raise CacheError(f"group {g}: a page is both free and held")
        slots = [rc.state_slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_state_slots):
            raise CacheError("state slots held twice")
        if len(slots) + len(self._free_state_slots) != self.max_requests:
            raise CacheError("state slot lost")
