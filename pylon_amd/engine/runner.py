"""The step executor: a model, its cache manager, and the one step function.

It plays the part of the reference's ``Decoder``
(/root/reference/src/pylon/decode/runner.py:58-302): it owns the page pool, opens and
releases request caches, and runs packed batches.  Unlike the reference there is one
step function for every kind of batch; a decode-only step differs only in that it may
be replayed from a HIP graph.
"""
from __future__ import annotations

import math
from pathlib import Path
from typing import Hashable, Optional, Sequence as Seq

import torch

from ..cache.manager import CacheManager, Sequence
from ..config.registry import load_model_config
from ..kernels import check_device
from ..weights.loader import load_weights
from .batch import MetadataArena, StepEntry, build_step
from .model import Model

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError("dtype must be bfloat16 or float32") from None


def weight_bytes(spec, dtype: torch.dtype) -> int:
    """Bytes of every parameter of a model of this spec, counted without allocating it."""
    model = Model(spec, dtype=dtype, device="meta")
    return sum(owner.params[name].numel() * owner.params[name].element_size()
               for _, owner, name in model.named_params())


def check_weights_fit(needed: int, free: int, total: int, config, what) -> None:
    """Refuse a model whose weights, with their headroom, do not fit under the utilisation
    limit (/root/reference/src/pylon/kv/budget.py:49-68, model/loader.py:59-72)."""
    required = int(needed * (1 + config.weight_headroom_ratio))
    available = max(0, math.floor(total * config.max_gpu_utilization) - (total - free))
    if required > available:
        raise RuntimeError(
            f"Refusing to load {what}: weights and headroom need {required:,} bytes; "
            f"{available:,} bytes are available under the GPU utilization limit.")


def pool_pages(free: int, total: int, bytes_per_token: int, config, max_positions: Optional[int]) -> int:
    """Pages of the cache pool from the device's memory once the weights are resident
    (/root/reference/src/pylon/kv/budget.py:70-113): the utilisation limit times the total,
    minus what is occupied, minus a headroom ``free - free / (1 + kv_cache_headroom_ratio)``
    that stays free for activations and graphs; no more than ``max_batch_size`` requests of
    the model's longest length could ever hold."""
    headroom = free - int(free / (1 + config.kv_cache_headroom_ratio))
    budget = math.floor(total * config.max_gpu_utilization) - (total - free) - headroom
    pages = budget // max(1, config.page_size * bytes_per_token)
    if max_positions:
        pages = min(pages, -(-max_positions // config.page_size) * config.max_batch_size)
    if pages < 1:
        raise RuntimeError("Not enough GPU memory remains for the KV cache and activations.")
    return int(pages)


class Runner:
    def __init__(self, model: Model, *, page_size: int, num_pages: int, max_requests: int) -> None:
        if model.device.type != "cuda":
            raise RuntimeError("A GPU is required: the step function has no CPU path.")
        check_device()
        self.model = model
        self.manager = CacheManager(
            model.cache_requirements(), page_size=page_size, num_pages=num_pages,
            max_requests=max_requests, dtype=model.dtype, device=model.device,
        )
        self.arena = MetadataArena(model.device)
        self.graphs = None
        # Per-request state of the sampler, by state slot: the token chosen last.  A step
        # may take a request's next token from here (StepEntry tokens = [PENDING]).
        self.chosen = torch.zeros(self.manager.slots.max_slots, dtype=torch.int32, device=model.device)
        self.logit_slots: Optional[torch.Tensor] = None  # state slot per row of the last step's logits

    # ---- construction ------------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder, *, dtype="bfloat16", device="cuda:0", page_size: int = 256,
                    num_pages: int, max_requests: int = 32) -> "Runner":
        """Load the model folder ``folder`` (config.json decides the model class)."""
        if not torch.cuda.is_available():
            raise RuntimeError("A GPU is required: the step function has no CPU path.")
        arch, config = load_model_config(folder)
        model = Model(arch.model_spec(config), dtype=resolve_dtype(dtype), device=device)
        load_weights(model, arch, config, Path(folder))
        runner = cls(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests)
        runner.config = config
        return runner

    @classmethod
    def from_config(cls, config, *, device="cuda:0") -> "Runner":
        """Load ``config.model_path`` and size the page pool: ``config.num_pages`` if given,
        else from the device memory that is free once the weights are resident
        (/root/reference/src/pylon/kv/budget.py:70-113: utilisation limit times total
        memory, minus what is occupied, minus a headroom share for activations)."""
        if not torch.cuda.is_available():
            raise RuntimeError("A GPU is required: the step function has no CPU path.")
        arch, model_config = load_model_config(config.model_path)
        spec = arch.model_spec(model_config)
        free, total = torch.cuda.mem_get_info(torch.device(device))
        check_weights_fit(weight_bytes(spec, resolve_dtype(config.dtype)), free, total, config, config.model_path)
        model = Model(spec, dtype=resolve_dtype(config.dtype), device=device)
        load_weights(model, arch, model_config, Path(config.model_path))
        num_pages = config.num_pages
        sizing = None
        if num_pages is None:
            from ..cache.manager import bytes_per_token

            per_token = bytes_per_token(model.cache_requirements(), model.dtype)
            free, total = torch.cuda.mem_get_info(model.device)
            num_pages = pool_pages(free, total, per_token, config, model.spec.max_positions)
            sizing = {"free": free, "total": total, "bytes_per_token": per_token, "num_pages": num_pages}
        runner = cls(model, page_size=config.page_size, num_pages=int(num_pages),
                     max_requests=config.max_batch_size)
        runner.config = model_config
        runner.pool_sizing = sizing  # what the pool was sized from (None: num_pages was given)
        if config.cuda_graphs:
            runner.enable_graphs(config.max_batch_size)
            runner.capture_graphs()
        return runner

    def enable_graphs(self, max_batch: Optional[int] = None, max_tokens_per_request: Optional[int] = None) -> None:
        """Replay decode-only steps of up to ``max_batch`` requests from HIP graphs.
        ``max_tokens_per_request`` bounds the lengths a graph serves (longer requests run
        kernel by kernel); by default whatever the page pool could hold."""
        from .graphs import DecodeGraphs

        page = self.manager.page_size
        limit = max_tokens_per_request or self.model.spec.max_positions or self.manager.capacity_tokens
        limit = min(limit, self.manager.capacity_tokens)
        self.graphs = DecodeGraphs(self.model, self.manager, self.arena,
                                   max_batch=max_batch or self.manager.slots.max_slots,
                                   max_pages_per_request=-(-limit // page), chosen=self.chosen)

    def capture_graphs(self, batch_sizes: Optional[Seq[int]] = None, bounds: Optional[Seq[int]] = None) -> tuple:
        """Capture decode graphs now instead of at their first use, as the reference does at
        start-up (/root/reference/src/pylon/decode/warmup.py:140-167): for these batch sizes
        (default: every size the graphs serve) and these bounds on the requests' lengths
        (default: the smallest, which serves requests of up to 1,024 tokens; the graphs of
        longer requests, see :meth:`DecodeGraphs.bounds`, are captured when such a request
        first decodes: a model of 262,144 positions has nine bounds, and start-up would
        capture nine graphs per batch size).  Throw-away requests of one
        token each take one decode step per graph and are closed again.  Sizes for which the
        pool has no free pages or slots are left to their first use.  Returns the batch sizes
        that have a graph."""
        if self.graphs is None:
            raise RuntimeError("capture_graphs needs enable_graphs first")
        from ..cache import OutOfPages

        sizes = sorted(set(batch_sizes or range(1, self.graphs.max_batch + 1)))
        bounds = sorted(set(bounds or self.graphs.bounds()[:1]))
        most = min(max(sizes), self.manager.free_pages, self.manager.slots.free_slots, self.graphs.max_batch)
        seqs = [self.open(("graph-warm-up", i)) for i in range(most)]
        limit = self.model.spec.max_positions
        try:
            if seqs:
                self.step([StepEntry(seq, [0], []) for seq in seqs])
            for bound in bounds:
                for rows in sizes:
                    if rows > most or (limit and seqs[0].length + 1 > limit):
                        break
                    entries = [StepEntry(seq, [0], [0]) for seq in seqs[:rows]]
                    if self.graphs.wants(entries) and (rows, bound) not in self.graphs.captured:
                        self.graphs.run(entries, bound=bound)
        except OutOfPages:
            pass  # a small pool: the remaining graphs are captured when they first occur
        finally:
            for seq in seqs:
                self.close(seq)
        self.synchronize()
        return self.graphs.captured_sizes()

    def synchronize(self) -> None:
        torch.cuda.synchronize(self.model.device)

    # ---- requests -------------------------------------------------------------------------
    def open(self, request_id: Hashable, capacity: Optional[int] = None) -> Sequence:
        max_positions = self.model.spec.max_positions
        if capacity is not None and max_positions and capacity > max_positions:
            raise ValueError(
                f"KV-cache capacity must be between 1 and {max_positions:,} tokens."
            )
        return self.manager.open(request_id, capacity)

    def close(self, seq: Sequence) -> None:
        self.manager.close(seq)

    # ---- the step ---------------------------------------------------------------------------
    def step(self, entries: Seq[StepEntry]) -> Optional[torch.Tensor]:
        """Run the given tokens of the given requests as one batch, from the cache that
        earlier steps left, and return float32 logits at the wanted places (in the order
        of the entries and of their ``want``), or None if nothing is wanted."""
        max_positions = self.model.spec.max_positions
        if max_positions:
            for e in entries:
                if e.seq.length + len(e.tokens) > max_positions:
                    raise ValueError(
                        f"The model supports at most {max_positions:,} tokens per request."
                    )
        if self.graphs is not None and self.graphs.wants(entries):
            logits = self.graphs.run(entries)
            if logits is not None:
                self.logit_slots = self.graphs.last_logit_slots
                return logits
        ctx = build_step(entries, self.manager, self.arena, vocab_size=self.model.spec.vocab_size,
                         chosen=self.chosen)
        self.logit_slots = ctx.logit_slots
        pairs = [(e.seq, len(e.tokens)) for e in entries]
        try:
            logits = self.model.step(ctx)
        except Exception:
            self.manager.cancel(pairs)
            raise
        self.manager.commit(pairs)
        return logits
