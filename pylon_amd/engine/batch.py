"""One step's batch: which tokens of which requests run, and everything the kernels
need to know about them, as one packed block of int32 that crosses to the device in a
single copy.

The vectors are the ones the reference builds in ``PackedBatchCache.prepare_packed``
(/root/reference/src/pylon/kv/cache.py:409-450): token ids, positions, the prefix sums
of the rows' token counts (its ``cu_seq_q``), the rows' lengths after the step (its
``seqused_k``), the block table, the cache slot of every token (its ``write_slots``) and
the indices whose logits are wanted (its ``last_indices``).  The reference fills them
with Python loops over every token; here they are numpy gathers.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence as Seq, Tuple

import numpy as np
import torch

from ..cache.manager import CacheManager, CacheView, Sequence


#: In place of a token id: "the token that the sampler chose for this request last, and
#: left on the device".  It lets a step be queued before the host has read that token.
PENDING = -1


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and which of them need logits."""

    seq: Sequence
    tokens: Seq[int]  # token ids; PENDING where the id is still on the device
    want: Seq[int] = ()  # indices into `tokens`


def _align4(n: int) -> int:
    return (n + 3) & ~3


class MetadataArena:
    """Pinned host buffers (used in rotation) and one device buffer for step metadata."""

    def __init__(self, device, capacity: int = 1 << 16, rotation: int = 4) -> None:
        self.device = torch.device(device)
        self.rotation = rotation
        self._cursor = 0
        self._capacity = 0
        self._host: List[torch.Tensor] = []
        self._events: List[Optional[torch.cuda.Event]] = []
        self._device_buf: Optional[torch.Tensor] = None
        self._grow(capacity)

    def _grow(self, capacity: int) -> None:
        pin = self.device.type == "cuda"
        if pin:
            torch.cuda.synchronize(self.device)
        self._capacity = capacity
        self._host = [torch.empty(capacity, dtype=torch.int32, pin_memory=pin) for _ in range(self.rotation)]
        self._events = [None] * self.rotation
        self._device_buf = torch.empty(capacity, dtype=torch.int32, device=self.device)

    def acquire(self, size: int) -> Tuple[np.ndarray, int]:
        """A host buffer of at least ``size`` ints that no pending copy still reads."""
        if size > self._capacity:
            self._grow(max(size, 2 * self._capacity))
        index = self._cursor
        self._cursor = (self._cursor + 1) % self.rotation
        event = self._events[index]
        if event is not None:
            event.synchronize()
        return self._host[index].numpy(), index

    def stage(self, values: np.ndarray) -> torch.Tensor:
        """A new int32 device tensor holding ``values``, copied through one of the pinned
        buffers without making the host wait for the device."""
        flat = np.ascontiguousarray(values, dtype=np.int32).reshape(-1)
        host, index = self.acquire(flat.size)
        host[: flat.size] = flat
        out = torch.empty(flat.size, dtype=torch.int32, device=self.device)
        self.upload(index, flat.size, into=out)
        return out.view(values.shape)

    def upload(self, index: int, size: int, into: Optional[torch.Tensor] = None) -> torch.Tensor:
        target = self._device_buf if into is None else into
        target[:size].copy_(self._host[index][:size], non_blocking=True)
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
            self._events[index] = event
        return target


@dataclass
class StepContext:
    """What parts see of the running step."""

    tokens: int
    rows: int
    token_ids: torch.Tensor  # int32 [tokens]
    positions: torch.Tensor  # int32 [tokens]: index of each token in its request
    tok_row: torch.Tensor  # int32 [tokens]: row (request of this step) of each token
    row_start: torch.Tensor  # int32 [rows + 1]: prefix sums of the rows' token counts
    seq_lens: torch.Tensor  # int32 [rows]: cached length of each row after this step
    row_slots: torch.Tensor  # int32 [rows]: state slot of each row's request
    row_first: torch.Tensor  # int32 [rows]: 1 where the row's tokens start its request
    logit_idx: Optional[torch.Tensor]  # int32 [n]: token indices whose logits are wanted
    n_logits: int
    views: Dict[int, CacheView]
    # host-side copies for parts that plan their launches on the host
    counts: np.ndarray = field(default=None)
    starts: np.ndarray = field(default=None)
    max_count: int = 0
    max_len: int = 0  # the longest row after this step; with fixed_shapes an upper bound on it
    decode_only: bool = False
    fixed_shapes: bool = False  # launches must not depend on lengths (graph capture)
    logit_slots: Optional[torch.Tensor] = None  # int32 [n]: state slot of each wanted row's request
    chosen: Optional[torch.Tensor] = None  # int32 [slots]: last sampled token per state slot
    logits_out: Optional[torch.Tensor] = None  # float32 [>= n_logits, vocab]: where the logits go, if given
    arena: Optional[MetadataArena] = None  # pinned staging for what parts put on the device themselves
    _tiles: Dict[Tuple[int, int, int], torch.Tensor] = field(default_factory=dict)

    def cache(self, cache_id: int) -> CacheView:
        return self.views[cache_id]

    @property
    def leading_singles(self) -> int:
        """How many rows at the head of the step bring exactly one token (the decoding
        requests, which the engine puts first): token t of them is row t."""
        more = np.nonzero(self.counts != 1)[0]
        return int(more[0]) if more.size else self.rows

    def token_tiles(self, tokens_per_tile: int, skip_rows: int = 0, fold: int = 0) -> torch.Tensor:
        """int32 ``[n, 4]`` on the device: the step's tokens (without those of the first
        ``skip_rows`` rows) cut into runs of at most ``tokens_per_tile`` consecutive tokens
        of one row, as (index of the first token, count, row, position of the first token),
        longest context first so that the heaviest tiles start first.  With ``fold`` (the
        number of tiles whose workgroups fill the chip once) every second run of ``fold``
        tiles is turned round: where two workgroups share a compute unit, the one that
        arrives second beside the heaviest of a round is the lightest of the next."""
        key = (tokens_per_tile, skip_rows, fold)
        tiles = self._tiles.get(key)
        if tiles is None:
            per_row = -(-self.counts // tokens_per_tile)
            per_row[:skip_rows] = 0
            row = np.repeat(np.arange(self.rows, dtype=np.int64), per_row)
            first_of_row = np.zeros(self.rows + 1, dtype=np.int64)
            np.cumsum(per_row, out=first_of_row[1:])
            within = (np.arange(int(per_row.sum()), dtype=np.int64) - first_of_row[row]) * tokens_per_tile
            count = np.minimum(tokens_per_tile, self.counts[row] - within)
            starts = np.zeros(self.rows + 1, dtype=np.int64)
            np.cumsum(self.counts, out=starts[1:])
            table = np.stack([starts[row] + within, count, row, self.starts[row] + within], axis=1)
            order = np.argsort(-(table[:, 3] + table[:, 1]), kind="stable")
            if fold > 0:
                for start in range(fold, len(order), 2 * fold):
                    order[start: start + fold] = order[start: start + fold][::-1].copy()
            ordered = table[order].astype(np.int32)
            if self.arena is not None:
                tiles = self.arena.stage(ordered)
            else:
                tiles = torch.from_numpy(np.ascontiguousarray(ordered)).to(self.token_ids.device)
            self._tiles[key] = tiles
        return tiles


def plan_layout(tokens: int, rows: int, n_logits: int, n_groups: int, width: int) -> Tuple[Dict[str, Tuple[int, int]], int]:
    """Offsets (in int32 units, each a multiple of 4) of every vector in the packed block."""
    layout: Dict[str, Tuple[int, int]] = {}
    cursor = 0

    def put(name: str, size: int) -> None:
        nonlocal cursor
        layout[name] = (cursor, size)
        cursor += _align4(max(size, 1))

    put("token_ids", tokens)
    put("positions", tokens)
    put("tok_row", tokens)
    put("row_start", rows + 1)
    put("seq_lens", rows)
    put("row_slots", rows)
    put("row_first", rows)
    put("logit_idx", n_logits)
    put("logit_slots", n_logits)
    for g in range(n_groups):
        put(f"slot_map{g}", tokens)
        put(f"block_table{g}", rows * width)
    return layout, cursor


def build_step(entries: Seq[StepEntry], manager: CacheManager, arena: MetadataArena, *,
               vocab_size: int, width: Optional[int] = None,
               device_block: Optional[torch.Tensor] = None, fixed_shapes: bool = False,
               chosen: Optional[torch.Tensor] = None, len_bound: Optional[int] = None) -> StepContext:
    """Check the entries, take the pages they need, and put the step's metadata on the
    device.  Raises before touching the cache if any entry is malformed; raises
    :class:`~pylon_amd.cache.pages.OutOfPages` (cache untouched) if pages run short.
    ``chosen`` is the table of last sampled tokens by state slot; only with it may an
    entry hold :data:`PENDING`.  ``len_bound``: what the parts are told instead of the
    longest row's length (a recorded step must not depend on the lengths themselves)."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    rows = len(entries)
    counts = np.fromiter((len(e.tokens) for e in entries), dtype=np.int64, count=rows)
    if (counts < 1).any():
        raise ValueError("Each packed sequence needs at least one query token.")
    tokens = int(counts.sum())
    flat = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
    pending = flat == PENDING
    if pending.any() and chosen is None:
        raise ValueError("A token left on the device needs the table of sampled tokens.")
    if flat.size and (flat[~pending].min(initial=0) < 0 or flat.max() >= vocab_size):
        raise ValueError(f"Token IDs must be between 0 and {vocab_size - 1:,}.")
    row_start = np.zeros(rows + 1, dtype=np.int64)
    np.cumsum(counts, out=row_start[1:])
    logit_list: List[int] = []
    for r, e in enumerate(entries):
        for w in e.want:
            if not 0 <= w < counts[r]:
                raise ValueError(f"wanted index {w} is outside the {counts[r]} tokens of its entry")
            logit_list.append(int(row_start[r]) + int(w))
    pairs = [(e.seq, int(c)) for e, c in zip(entries, counts)]
    manager.reserve(pairs)  # all-or-nothing

    # From here on pages are held for this step: whatever goes wrong before the step's
    # metadata is on the device gives them back.
    try:
        starts = np.fromiter((e.seq.length for e in entries), dtype=np.int64, count=rows)
        slots = np.fromiter((e.seq.slot for e in entries), dtype=np.int64, count=rows)
        tok_row = np.repeat(np.arange(rows, dtype=np.int64), counts)
        positions = starts[tok_row] + (np.arange(tokens, dtype=np.int64) - row_start[tok_row])
        seq_lens = starts + counts
        need_width = int(-(-seq_lens.max() // manager.page_size))
        if width is None:
            width = need_width
        elif need_width > width:
            raise ValueError(f"a request needs {need_width} pages but the block table holds {width}")

        n_groups = len(manager.groups)
        layout, size = plan_layout(tokens, rows, len(logit_list), n_groups, width)
        host, index = arena.acquire(size)

        def seg(name: str) -> np.ndarray:
            off, n = layout[name]
            return host[off: off + n]

        token_slots = slots[tok_row]
        if pending.any():
            flat = np.where(pending, -1 - token_slots, flat)  # the embedding reads chosen[slot]
        seg("token_ids")[:] = flat
        seg("positions")[:] = positions
        seg("tok_row")[:] = tok_row
        seg("row_start")[:] = row_start
        seg("seq_lens")[:] = seq_lens
        seg("row_slots")[:] = slots
        seg("row_first")[:] = starts == 0
        if logit_list:
            seg("logit_idx")[:] = logit_list
            seg("logit_slots")[:] = token_slots[logit_list]
        for g in range(n_groups):
            manager.slot_map(g, token_slots, positions, seg(f"slot_map{g}"))
            manager.block_table(g, slots, width, seg(f"block_table{g}").reshape(rows, width))
        block = arena.upload(index, size, into=device_block)

        def dev(name: str) -> torch.Tensor:
            off, n = layout[name]
            return block[off: off + n]

        views: Dict[int, CacheView] = {}
        for cache_id in range(manager.n_caches):
            view = manager.view(cache_id)
            if view.group >= 0:
                view.slot_map = dev(f"slot_map{view.group}")
                view.block_table = dev(f"block_table{view.group}").view(rows, width)
            views[cache_id] = view
        return StepContext(
            tokens=tokens, rows=rows,
            token_ids=dev("token_ids"), positions=dev("positions"), tok_row=dev("tok_row"),
            row_start=dev("row_start"), seq_lens=dev("seq_lens"), row_slots=dev("row_slots"),
            row_first=dev("row_first"),
            logit_idx=dev("logit_idx") if logit_list else None, n_logits=len(logit_list),
            logit_slots=dev("logit_slots") if logit_list else None, chosen=chosen,
            views=views, counts=counts, starts=starts, max_count=int(counts.max()),
            max_len=int(seq_lens.max()) if len_bound is None else int(len_bound),
            decode_only=bool((counts == 1).all()),
            fixed_shapes=fixed_shapes, arena=arena,
        )
    except BaseException:
        manager.cancel(pairs)
        raise
