"""The cache manager: keys and values in pages, a block table per request, and slots
for fixed-size per-request state.

What the reference spreads over ``KVPagePool`` (/root/reference/src/pylon/kv/pool.py:19-75),
``PagedKVCache`` (/root/reference/src/pylon/kv/cache.py:20-135) and the page bookkeeping
of ``PackedBatchCache.prepare_packed`` (:381-408) lives here, with two generalisations:

* Runs of layers are put into *groups* by what they need (number of key/value heads,
  head size, window).  A group has its own page pool, its own storage and, per request,
  its own list of pages; the reference has exactly one such group.
* A group with a window gives a request's pages back as soon as no later token can see
  them, not only when the request ends.

Everything here is host-side bookkeeping plus the storage tensors; it runs unchanged
with CPU tensors, which is how the unit tests drive it.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence as Seq, Tuple

import numpy as np
import torch

from ..parts.base import KVRequirement, StateRequirement
from .pages import OutOfPages, PagePool
from .state import StateSlots

FREED = -1  # entry of a request's page list whose page has been given back


def pages_for(tokens: int, page_size: int) -> int:
    return (tokens + page_size - 1) // page_size


def bytes_per_token(requirements: Seq[object], dtype: torch.dtype) -> int:
    """Cache bytes one token takes over all runs that keep keys and values."""
    elem = torch.empty((), dtype=dtype).element_size()
    return sum(2 * r.n_kv_heads * r.head_dim * elem for r in requirements if isinstance(r, KVRequirement))


def group_requirements(requirements: Seq[object]):
    """Runs by what they keep: ``({KVRequirement: [run ids]}`` in order of first appearance,
    one entry per group of pages; ``{run id: StateRequirement})``."""
    by_need: Dict[KVRequirement, List[int]] = {}
    states: Dict[int, StateRequirement] = {}
    for cache_id, need in enumerate(requirements):
        if need is None:
            continue
        if isinstance(need, KVRequirement):
            by_need.setdefault(need, []).append(cache_id)
        elif isinstance(need, StateRequirement):
            states[cache_id] = need
        else:
            raise TypeError(f"run {cache_id} asks for an unknown kind of cache: {need!r}")
    return by_need, states


def plan_pool(budget_bytes: int, groups: Seq[object], *, page_size: int, max_requests: int,
              max_positions: Optional[int], chunk: int) -> List[int]:
    """Pages for each group of runs under a budget of bytes.  ``groups[g]`` has
    ``bytes_per_token`` (over the group's runs) and ``window``.

    Every group has to hold the same requests, so every group gets the same number of pages P,
    the largest the budget pays for, except that no group gets more than it can ever use: a
    group that keeps every token, ``max_requests`` requests of ``max_positions`` tokens; a group
    with a window, per request the pages of ``window + chunk`` tokens and one more (a step
    takes the pages of up to ``chunk`` new tokens before it gives back those the window has
    passed).  The reference's single group gets ``budget // bytes of a page``
    (/root/reference/src/pylon/engine.py:173-178), capped as above."""
    if not groups:
        return []
    full = pages_for(max_positions, page_size) * max_requests if max_positions else None
    caps: List[Optional[int]] = []
    for group in groups:
        cap = full
        if group.window is not None:
            own = (pages_for(group.window + chunk, page_size) + 1) * max_requests
            cap = own if cap is None else min(cap, own)
        caps.append(cap)

    def cost(pages: int) -> int:
        return sum((pages if cap is None else min(pages, cap)) * page_size * group.bytes_per_token
                   for group, cap in zip(groups, caps))

    high = max(budget_bytes, 0) // max(1, page_size * min(g.bytes_per_token for g in groups)) + 1
    if all(cap is not None for cap in caps):
        high = min(high, max(caps))
    low = 0  # the largest P known to fit
    while low < high:
        mid = (low + high + 1) // 2
        if cost(mid) <= budget_bytes:
            low = mid
        else:
            high = mid - 1
    if low < 1:
        raise RuntimeError("Not enough GPU memory remains for the KV cache and activations.")
    return [low if cap is None else min(low, cap) for cap in caps]


class KVGroup:
    """Runs with one key/value geometry: a pool of page ids and one K and V tensor per run."""

    def __init__(self, index: int, requirement: KVRequirement, cache_ids: List[int], num_pages: int,
                 page_size: int, dtype: torch.dtype, device, max_requests: int) -> None:
        self.index = index
        # table[slot, i] = id of the i-th page of the request in state slot `slot`; kept as
        # one array so that a step's block table and slot map are single gathers.
        self.table = np.zeros((max_requests, 8), dtype=np.int32)
        self.requirement = requirement
        self.cache_ids = list(cache_ids)
        self.page_size = page_size
        self.pool = PagePool(num_pages)
        shape = (num_pages, page_size, requirement.n_kv_heads, requirement.head_dim)
        # Same layout as the reference's pool (/root/reference/src/pylon/kv/pool.py:36-44):
        # page, slot in page, key/value head, element.  Zero-filled so that a slot no
        # token has written yet holds finite numbers.
        self.k: Dict[int, torch.Tensor] = {c: torch.zeros(shape, dtype=dtype, device=device) for c in cache_ids}
        self.v: Dict[int, torch.Tensor] = {c: torch.zeros(shape, dtype=dtype, device=device) for c in cache_ids}

    def record_pages(self, slot: int, first_index: int, pages: List[int]) -> None:
        end = first_index + len(pages)
        if end > self.table.shape[1]:
            width = self.table.shape[1]
            while width < end:
                width *= 2
            grown = np.zeros((self.table.shape[0], width), dtype=np.int32)
            grown[:, : self.table.shape[1]] = self.table
            self.table = grown
        self.table[slot, first_index:end] = pages

    @property
    def bytes_per_token(self) -> int:
        r = self.requirement
        elem = next(iter(self.k.values())).element_size() if self.k else 0
        return len(self.cache_ids) * 2 * r.n_kv_heads * r.head_dim * elem


class Sequence:
    """One request's hold on the cache: its pages in every group, its length, its slot."""

    __slots__ = ("request_id", "length", "capacity", "pages", "slot", "closed", "_pending")

    def __init__(self, request_id: Hashable, capacity: Optional[int], n_groups: int, slot: int) -> None:
        self.request_id = request_id
        self.length = 0
        self.capacity = capacity
        self.pages: List[List[int]] = [[] for _ in range(n_groups)]
        self.slot = slot
        self.closed = False
        self._pending: Optional[int] = None


@dataclass
class CacheView:
    """What a mixer sees of its run's cache during one step."""

    page_size: int = 0
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    block_table: Optional[torch.Tensor] = None  # int32 [rows, width]
    slot_map: Optional[torch.Tensor] = None  # int32 [tokens]: page * page_size + offset
    state: Optional[torch.Tensor] = None  # [max_slots, *shape] for stateful mixers
    group: int = -1


class CacheManager:
    def __init__(self, requirements: Seq[object], *, page_size: int, num_pages, max_requests: int,
                 dtype: torch.dtype, device="cpu") -> None:
        """``requirements[c]`` is what run ``c`` of the schedule needs: a
        :class:`KVRequirement`, a :class:`StateRequirement`, or None (it borrows, or keeps
        nothing).  ``num_pages``: pages (of ``page_size`` tokens) of every group, or one
        number per group in the order of :func:`group_requirements`."""
        if page_size < 1:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.dtype = dtype
        self.device = device
        self.n_caches = len(requirements)
        self.groups: List[KVGroup] = []
        self.group_of: Dict[int, int] = {}
        self.slots = StateSlots(max_requests)
        by_need, states = group_requirements(requirements)
        for cache_id, need in states.items():
            self.slots.add_state(cache_id, tuple(need.shape), need.dtype, device)
        if isinstance(num_pages, int):
            per_group = [num_pages] * len(by_need)
        else:
            per_group = [int(n) for n in num_pages]
            if len(per_group) != len(by_need):
                raise ValueError(f"{len(per_group)} page counts for {len(by_need)} groups of runs")
        # What admission counts with: the pages of the group that has most (one that keeps
        # every token, if there is one; a group with a window may have fewer and never lacks).
        self.num_pages = max(per_group) if per_group else (num_pages if isinstance(num_pages, int) else 0)
        for (need, cache_ids), pages in zip(by_need.items(), per_group):
            group = KVGroup(len(self.groups), need, cache_ids, pages, page_size, dtype, device,
                            max_requests)
            self.groups.append(group)
            for cache_id in cache_ids:
                self.group_of[cache_id] = group.index
        self._live: Dict[Hashable, Sequence] = {}

    # ---- sizes -------------------------------------------------------------------
    @property
    def bytes_per_token(self) -> int:
        """Cache bytes one token takes (/root/reference/src/pylon/kv/pool.py:47-55)."""
        return sum(g.bytes_per_token for g in self.groups)

    @property
    def free_pages(self) -> int:
        """Free pages of the tightest group."""
        return min((g.pool.free_pages for g in self.groups), default=self.num_pages)

    @property
    def capacity_tokens(self) -> int:
        return self.num_pages * self.page_size

    def live_sequences(self) -> Tuple[Sequence, ...]:
        return tuple(self._live.values())

    # ---- life of a request ---------------------------------------------------------
    def open(self, request_id: Hashable, capacity: Optional[int] = None) -> Sequence:
        if request_id in self._live:
            raise ValueError(f"request {request_id!r} already has a cache")
        if capacity is not None and capacity < 1:
            raise ValueError("capacity must be at least one token")
        slot = self.slots.acquire()
        seq = Sequence(request_id, capacity, len(self.groups), slot)
        self._live[request_id] = seq
        return seq

    def missing_pages(self, seq: Sequence, count: int) -> List[int]:
        """Pages each group still lacks to hold ``count`` more tokens of ``seq``."""
        end = seq.length + count
        return [max(0, pages_for(end, self.page_size) - len(seq.pages[g.index])) for g in self.groups]

    def reserve(self, entries: Seq[Tuple[Sequence, int]]) -> None:
        """Take the pages a step needs.  Every entry is checked before any page is
        taken (/root/reference/src/pylon/kv/cache.py:386-408), so a refused step leaves
        the cache as it was."""
        seen = set()
        totals = [0] * len(self.groups)
        plans = []
        for seq, count in entries:
            if seq.closed:
                raise ValueError(f"request {seq.request_id!r} has been closed")
            if id(seq) in seen:
                raise ValueError("Paged batches require distinct request caches.")
            seen.add(id(seq))
            if count < 1:
                raise ValueError("Each packed sequence needs at least one query token.")
            if seq._pending is not None:
                raise ValueError("Packed append exceeds capacity or an append is pending.")
            if seq.capacity is not None and seq.length + count > seq.capacity:
                raise ValueError("Packed append exceeds capacity or an append is pending.")
            missing = self.missing_pages(seq, count)
            plans.append((seq, count, missing))
            for g, n in enumerate(missing):
                totals[g] += n
        for group, total in zip(self.groups, totals):
            if total > group.pool.free_pages:
                raise OutOfPages(
                    f"Insufficient free pages for packed append: group {group.index} needs "
                    f"{total}, {group.pool.free_pages} are free."
                )
        for seq, count, missing in plans:
            for group, n in zip(self.groups, missing):
                if n:
                    held = seq.pages[group.index]
                    fresh = group.pool.acquire(n)
                    group.record_pages(seq.slot, len(held), fresh)
                    held.extend(fresh)
            seq._pending = count

    def cancel(self, entries: Seq[Tuple[Sequence, int]]) -> None:
        """Undo :meth:`reserve` after a step that failed: pages beyond the cached length
        go back, lengths stay."""
        for seq, _count in entries:
            if seq._pending is None:
                continue
            seq._pending = None
            keep = pages_for(seq.length, self.page_size)
            for group in self.groups:
                pages = seq.pages[group.index]
                while len(pages) > keep:
                    page = pages.pop()
                    if page != FREED:
                        group.pool.release(page)

    def commit(self, entries: Seq[Tuple[Sequence, int]]) -> None:
        """The step has run: lengths grow, and pages a window has passed go back."""
        for seq, count in entries:
            if seq._pending != count:
                raise RuntimeError("commit must match the reserved token count")
            seq.length += count
            seq._pending = None
            for group in self.groups:
                window = group.requirement.window
                if window is None:
                    continue
                # The next token sits at position `length`; it sees keys from
                # length - window + 1 on.  A page whose last slot lies before that is dead.
                first_needed = seq.length - window + 1
                pages = seq.pages[group.index]
                dead = min(max(0, first_needed // self.page_size), len(pages))
                for i in range(dead):
                    if pages[i] != FREED:
                        group.pool.release(pages[i])
                        pages[i] = FREED

    def close(self, seq: Sequence) -> None:
        """The request is over: all its pages and its slot go back."""
        if seq.closed:
            raise RuntimeError(f"request {seq.request_id!r} was closed twice")
        for group in self.groups:
            for page in seq.pages[group.index]:
                if page != FREED:
                    group.pool.release(page)
            seq.pages[group.index] = []
        self.slots.release(seq.slot)
        seq.closed = True
        seq._pending = None
        self._live.pop(seq.request_id, None)

    # ---- fixed-size state across a step that may fail ---------------------------------
    def snapshot_state(self, seqs: Seq[Sequence]):
        """A copy of the fixed-size state of these requests, to put back should the step
        fail after a mixer has overwritten it.  None when no run keeps such state (then
        nothing is copied: the case of every model of keys and values only)."""
        if not self.slots.tensors:
            return None
        index = torch.as_tensor([seq.slot for seq in seqs], dtype=torch.long, device=self.device)
        return index, {cache_id: tensor.index_select(0, index) for cache_id, tensor in self.slots.tensors.items()}

    def restore_state(self, saved) -> None:
        if saved is None:
            return
        index, copies = saved
        for cache_id, copy in copies.items():
            self.slots.tensors[cache_id].index_copy_(0, index, copy)

    # ---- what a step needs to know ---------------------------------------------------
    def table_width(self, seqs: Seq[Sequence], counts: Seq[int]) -> int:
        return max(pages_for(s.length + c, self.page_size) for s, c in zip(seqs, counts))

    def block_table(self, group: int, slots: np.ndarray, width: int, out: np.ndarray) -> None:
        """``out[r, :width]`` = page ids of the request in slot ``slots[r]``.  Entries past
        a request's pages, and pages already given back, are never visited by a kernel."""
        table = self.groups[group].table
        if width > table.shape[1]:
            out[:, : table.shape[1]] = table[slots]
            out[:, table.shape[1]:] = 0
        else:
            out[:, :] = table[slots, :width]

    def slot_map(self, group: int, token_slots: np.ndarray, positions: np.ndarray, out: np.ndarray) -> None:
        """Cache slot (page * page_size + offset) of every token of a step
        (/root/reference/src/pylon/kv/cache.py:440-449)."""
        table = self.groups[group].table
        page = table[token_slots, positions // self.page_size]
        out[:] = page * self.page_size + positions % self.page_size

    def view(self, cache_id: int) -> CacheView:
        """The storage side of a run's cache (tables and slot maps are added per step)."""
        if cache_id in self.group_of:
            group = self.groups[self.group_of[cache_id]]
            return CacheView(page_size=self.page_size, k=group.k[cache_id], v=group.v[cache_id],
                             group=group.index)
        if cache_id in self.slots.tensors:
            return CacheView(state=self.slots.tensors[cache_id])
        return CacheView()

    # ---- invariants ---------------------------------------------------------------------
    def check(self) -> None:
        """No page lost, held twice or freed twice; no slot lost."""
        for group in self.groups:
            group.pool.check()
            held: Dict[int, Hashable] = {}
            for seq in self._live.values():
                for page in seq.pages[group.index]:
                    if page == FREED:
                        continue
                    if page in held:
                        raise AssertionError(
                            f"page {page} of group {group.index} is held by {held[page]!r} "
                            f"and {seq.request_id!r}"
                        )
                    held[page] = seq.request_id
                    if group.pool.refcount(page) < 1:
                        raise AssertionError(f"page {page} is in use but marked free")
            if len(held) != group.pool.used_pages:
                raise AssertionError(
                    f"group {group.index}: {group.pool.used_pages} pages are out of the pool "
                    f"but requests hold {len(held)}"
                )
        self.slots.check()
        if self.slots.max_slots - self.slots.free_slots != len(self._live):
            raise AssertionError("state slots in use do not match the live requests")
