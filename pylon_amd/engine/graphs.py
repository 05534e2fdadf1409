"""HIP graph replay of decode-only steps.

As in the reference (/root/reference/src/pylon/decode/graph.py:71-242) there is one graph
per batch size, captured over static buffers; a replay fills the buffers and launches the
graph; a batch size without a graph, or whose capture failed, runs kernel by kernel, and a
failed capture is not tried again.  Differences: the static buffers are one packed block
of metadata (filled by the same code that prepares any other step), a graph that was not
captured at start-up (``Runner.capture_graphs``) is captured the first time its batch size
is seen, and a batch is never padded to a larger captured size.

The launches recorded in a graph must not depend on the requests' lengths: the block
table has a fixed width, and what a mixer launches may depend on the batch size and on a
bound on the lengths only (the decode attention kernel shares a request's keys between
workgroups and waves by it).  That bound is a power of two of at least 512 tokens (up to
there one workgroup per token and head is fastest; beyond, the keys are cut).  A
mixer says through ``decode_signature(rows, bound)`` what of its launches depends on the
bound; bounds with equal signatures share one graph, and a mixer that does not say is taken
to depend on the bound itself.  There is one graph per (batch size, signature).
"""
from __future__ import annotations

import gc
import logging
from typing import Dict, Optional, Sequence as Seq, Tuple

import torch

from .batch import StepEntry, build_step, plan_layout

logger = logging.getLogger("pylon")

MIN_BOUND = 512  # the smallest bound on the requests' lengths a graph is captured for


class DecodeGraphs:
    def __init__(self, model, manager, arena, *, max_batch: int, max_pages_per_request: int,
                 chosen: Optional[torch.Tensor] = None) -> None:
        # The model, manager and arena are held directly, not through the runner that owns
        # this object: no reference cycle, so graphs are destroyed when the runner goes,
        # never by a garbage collection that happens to run inside a later capture.
        self.model = model
        self.manager = manager
        self.arena = arena
        self.chosen = chosen  # table of last sampled tokens, read by the recorded embedding
        self.last_logit_slots: Optional[torch.Tensor] = None
        self.max_batch = max_batch
        self.width = max_pages_per_request
        self.pool = torch.cuda.graph_pool_handle()
        # Every graph leaves its logits in the first rows of this one buffer: with a buffer per
        # graph, the graphs of a large vocabulary would hold gigabytes between them.
        self.logits = torch.empty((max_batch, model.spec.vocab_size), dtype=torch.float32, device=model.device)
        self.captured: Dict[Tuple[int, int], tuple] = {}
        self.failed = set()
        self.replays = 0

    def captured_sizes(self):
        return tuple(sorted({rows for rows, _signature in self.captured}))

    def key(self, rows: int, bound: int) -> tuple:
        """What names the graph of ``rows`` requests of at most ``bound`` tokens: the batch
        size and everything the model's recorded launches take from the bound."""
        describe = getattr(self.model, "decode_signature", None)
        return rows, (("bound", bound) if describe is None else describe(rows, bound))

    def _bound(self, entries: Seq[StepEntry]) -> int:
        """The power of two (from MIN_BOUND) that holds the longest request after this step."""
        need = max(e.seq.length for e in entries) + 1
        bound = MIN_BOUND
        while bound < need:
            bound *= 2
        return bound

    def bounds(self) -> Tuple[int, ...]:
        """Every bound a graph may be captured for: the powers of two from MIN_BOUND up to the
        one that holds the longest request the block table has room for."""
        longest = self.width * self.manager.page_size
        out = [MIN_BOUND]
        while out[-1] < longest:
            out.append(out[-1] * 2)
        return tuple(out)

    def wants(self, entries: Seq[StepEntry]) -> bool:
        """A decode-only step: one token per request, each wanting its logits."""
        rows = len(entries)
        if rows > self.max_batch or self.key(rows, self._bound(entries)) in self.failed:
            return False
        page = self.manager.page_size
        for e in entries:
            if len(e.tokens) != 1 or list(e.want) != [0]:
                return False
            if e.seq.length + 1 > self.width * page:
                return False  # longer than the captured block table: run kernel by kernel
        return True

    def run(self, entries: Seq[StepEntry], bound: Optional[int] = None) -> Optional[torch.Tensor]:
        """Replay (capturing first if need be).  Returns None if this batch size has no
        graph; the caller then runs the step kernel by kernel.  The cache is reserved and
        committed here exactly as an ordinary step does.  ``bound`` (capture at start-up)
        asks for the graph of a larger bound than these requests need: what a graph records
        depends on the bound, not on the lengths, so short requests can capture it."""
        rows = len(entries)
        manager, model, arena = self.manager, self.model, self.arena
        pairs = [(e.seq, 1) for e in entries]
        bound = max(bound or 0, self._bound(entries))
        key = self.key(rows, bound)
        entry = self.captured.get(key)
        if entry is None:
            _, size = plan_layout(rows, rows, rows, len(manager.groups), self.width)
            block = torch.empty(size, dtype=torch.int32, device=model.device)
            ctx = build_step(entries, manager, arena, vocab_size=model.spec.vocab_size,
                             width=self.width, device_block=block, fixed_shapes=True,
                             chosen=self.chosen, len_bound=bound)
            ctx.logits_out = self.logits
            # No garbage collection while the stream is capturing: a finalizer that frees a
            # device object (an event, another graph) is not allowed there and aborts.
            gc.collect()
            gc_was_enabled = gc.isenabled()
            gc.disable()
            try:
                torch.cuda.synchronize(model.device)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, pool=self.pool):
                    logits = model.step(ctx)
            except Exception:  # noqa: BLE001 - a failed capture leaves this size to eager steps
                logger.exception("decode_graph_capture_failed batch_size=%s bound=%s", rows, bound)
                self.failed.add(key)
                manager.cancel(pairs)
                return None
            finally:
                if gc_was_enabled:
                    gc.enable()
            self.captured[key] = (graph, block, logits, ctx.logit_slots)
            self.last_logit_slots = ctx.logit_slots
            try:
                graph.replay()  # capture records only; this runs the step
            except BaseException:
                manager.cancel(pairs)
                raise
        else:
            graph, block, logits, self.last_logit_slots = entry
            build_step(entries, manager, arena, vocab_size=model.spec.vocab_size,
                       width=self.width, device_block=block, fixed_shapes=True, chosen=self.chosen,
                       len_bound=bound)
            try:
                graph.replay()
            except BaseException:
                manager.cancel(pairs)  # the pages taken for this step go back
                raise
        self.replays += 1
        manager.commit(pairs)
        return logits
