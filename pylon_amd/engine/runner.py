"""The step executor: a model, its cache manager, and the one step function.

It plays the part of the reference's ``Decoder``
(/root/reference/src/pylon/decode/runner.py:58-302): it owns the page pool, opens and
releases request caches, and runs packed batches.  Unlike the reference there is one
step function for every kind of batch; a decode-only step differs only in that it may
be replayed from a HIP graph.

Start-up (:meth:`Runner.from_config` for a model folder, :meth:`Runner.from_random` for
random weights drawn in place) is the reference's, in its order
(/root/reference/src/pylon/engine.py:129-239, kv/budget.py:49-113,
decode/warmup.py:33-167): refuse weights that do not fit, make them resident, run the
largest step the serving options allow once to measure what activations take, size the
page pool from what is left, capture the decode graphs.
"""
from __future__ import annotations

import logging
import math
import time
from pathlib import Path
from typing import Callable, Dict, Hashable, List, Mapping, Optional, Sequence as Seq

import torch

from ..cache.manager import CacheManager, Sequence, group_requirements, plan_pool
from ..config.registry import load_model_config, resolve
from ..kernels import check_device
from ..weights.loader import load_weights, stored_param_dtypes
from ..weights.random_init import fill_random_model
from .batch import MetadataArena, StepEntry, build_step
from .model import Model

logger = logging.getLogger("pylon")

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError("dtype must be bfloat16 or float32") from None


def weight_bytes(spec, dtype: torch.dtype, param_dtypes: Optional[Mapping[str, torch.dtype]] = None,
                 model: Optional[Model] = None) -> int:
    """Bytes of every parameter of a model of this spec, counted without allocating it.
    ``param_dtypes`` gives parameters (by path) another element type than the model builds
    them with: what a folder's stored types make of them."""
    model = model or Model(spec, dtype=dtype, device="meta")
    total = 0
    for path, owner, name in model.named_params():
        param = owner.params[name]
        size = param.element_size()
        if param_dtypes and path in param_dtypes:
            size = torch.empty((), dtype=param_dtypes[path]).element_size()
        # a matrix whose rows lie apart in memory takes what its strides span
        elements = param.shape[0] * param.stride(0) if param.dim() == 2 and param.shape[0] else param.numel()
        total += max(elements, param.numel()) * size
    return total


def check_weights_fit(needed: int, free: int, total: int, config, what) -> None:
    """Refuse a model whose weights, with their headroom, do not fit under the utilisation
    limit (/root/reference/src/pylon/kv/budget.py:49-68, model/loader.py:59-72)."""
    required = int(needed * (1 + config.weight_headroom_ratio))
    available = max(0, math.floor(total * config.max_gpu_utilization) - (total - free))
    if required > available:
        raise RuntimeError(
            f"Refusing to load {what}: weights and headroom need {required:,} bytes; "
            f"{available:,} bytes are available under the GPU utilization limit.")


def cache_budget(free: int, total: int, config, activation_bytes: Optional[int] = None) -> int:
    """Bytes for everything the cache manager keeps, once the weights are resident
    (/root/reference/src/pylon/kv/budget.py:70-113): the utilisation limit times the total,
    minus what is occupied, minus a headroom that stays free for activations and graphs:
    ``free - free / (1 + kv_cache_headroom_ratio)``, or, with the activations' measured peak,
    that peak times ``1 + kv_cache_headroom_ratio``."""
    if activation_bytes is None:
        headroom = free - int(free / (1 + config.kv_cache_headroom_ratio))
    else:
        if activation_bytes < 0:
            raise ValueError("Warmup peak memory must be non-negative.")
        headroom = math.ceil(activation_bytes * (1 + config.kv_cache_headroom_ratio))
    return math.floor(total * config.max_gpu_utilization) - (total - free) - headroom


def pool_pages(free: int, total: int, bytes_per_token: int, config, max_positions: Optional[int],
               activation_bytes: Optional[int] = None) -> int:
    """Pages of a pool whose runs all keep every token: :func:`cache_budget` over the bytes of
    a page, and no more than ``max_batch_size`` requests of the model's longest length could
    ever hold."""
    requirement = [_Bytes(bytes_per_token)]
    return plan_pool(cache_budget(free, total, config, activation_bytes), requirement, page_size=config.page_size,
                     max_requests=config.max_batch_size, max_positions=max_positions,
                     chunk=config.prefill_chunk_size)[0]


class _Bytes:
    """A stand-in for a group of runs without a window that takes so many bytes per token."""

    def __init__(self, bytes_per_token: int) -> None:
        self.bytes_per_token, self.window = bytes_per_token, None


class Runner:
    def __init__(self, model: Model, *, page_size: int, num_pages, max_requests: int) -> None:
        """``num_pages``: pages of every group of runs, or one number per group."""
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
        self.config = None
        self.pool_sizing: Optional[dict] = None  # what the pool was sized from (None: num_pages was given)
        self.startup: Dict[str, float] = {}      # seconds that the stages of start-up took
        # Per-request state of the sampler, by state slot: the token chosen last.  A step
        # may take a request's next token from here (StepEntry tokens = [PENDING]).
        self.chosen = torch.zeros(self.manager.slots.max_slots, dtype=torch.int32, device=model.device)
        self.logit_slots: Optional[torch.Tensor] = None  # state slot per row of the last step's logits

    # ---- construction ------------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder, *, dtype="bfloat16", device="cuda:0", page_size: int = 256,
                    num_pages: int, max_requests: int = 32) -> "Runner":
        """Load the model folder ``folder`` (config.json decides the model class) over a pool
        of a given size: no fit check, no sizing, no graphs."""
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
        """Start up over the model folder ``config.model_path`` as a server does."""
        if config.model_path is None:
            raise ValueError("PylonConfig.model_path (or PYLON_MODEL_PATH) names no model folder.")
        folder = Path(config.model_path)
        arch, model_config = load_model_config(folder)
        return cls._start(
            arch, model_config, config, device, what=str(folder),
            stored=lambda meta: stored_param_dtypes(meta, arch, model_config, folder),
            fill=lambda model: load_weights(model, arch, model_config, folder))

    @classmethod
    def from_random(cls, model_config: Mapping, seed: int, config, *, std: Optional[float] = None,
                    norm_jitter: float = 0.0, draw_on=None, device="cuda:0") -> "Runner":
        """The same start-up over random weights of the architecture and sizes that
        ``model_config`` (the contents of a config.json) names, drawn in place from ``seed``
        by the random-weights mode's rule: no folder is written, so a model of any size starts
        in seconds.  ``draw_on="cpu"`` draws the numbers of the folder that the mode writes
        from the same (config, seed); by default the GPU draws, other numbers by the same rule."""
        arch = resolve(model_config)
        parsed = arch.parse_config(model_config)
        return cls._start(
            arch, parsed, config, device, what="a model of random weights", stored=lambda meta: None,
            fill=lambda model: fill_random_model(model, arch, parsed, seed, std=std, norm_jitter=norm_jitter,
                                                 draw_on=draw_on))

    @classmethod
    def _start(cls, arch, model_config, config, device, *, what: str, stored: Callable, fill: Callable) -> "Runner":
        if not torch.cuda.is_available():
            raise RuntimeError("A GPU is required: the step function has no CPU path.")
        clock = time.perf_counter
        began = clock()
        dtype = resolve_dtype(config.dtype)
        spec = arch.model_spec(model_config)
        meta = Model(spec, dtype=dtype, device="meta")
        free, total = torch.cuda.mem_get_info(torch.device(device))
        check_weights_fit(weight_bytes(spec, dtype, stored(meta), model=meta), free, total, config, what)
        model = Model(spec, dtype=dtype, device=device)
        fill(model)
        torch.cuda.synchronize(model.device)
        weights_done = clock()
        num_pages, sizing = config.num_pages, None
        if num_pages is None:
            activation = measure_activation_bytes(model, config)
            torch.cuda.empty_cache()
            free, total = torch.cuda.mem_get_info(model.device)
            groups, state_bytes = cache_needs(model.cache_requirements(), model.dtype, config.max_batch_size)
            budget = cache_budget(free, total, config, activation)
            num_pages = plan_pool(budget - state_bytes, groups, page_size=config.page_size,
                                  max_requests=config.max_batch_size, max_positions=spec.max_positions,
                                  chunk=config.prefill_chunk_size)
            sizing = {"free": free, "total": total, "activation_bytes": activation, "state_bytes": state_bytes,
                      "bytes_per_token": sum(g.bytes_per_token for g in groups),
                      "num_pages": max(num_pages), "pages_per_group": list(num_pages)}
        runner = cls(model, page_size=config.page_size, num_pages=num_pages, max_requests=config.max_batch_size)
        runner.config = model_config
        runner.pool_sizing = sizing
        pool_done = clock()
        if config.cuda_graphs:
            runner.enable_graphs(config.max_batch_size)
            runner.capture_graphs(max_tokens=config.cuda_graph_max_tokens)
        done = clock()
        runner.startup = {"weights_s": weights_done - began, "pool_s": pool_done - weights_done,
                          "graphs_s": done - pool_done, "total_s": done - began}
        logger.info("runner_started what=%s weights_s=%.2f pool_s=%.2f graphs_s=%.2f pages=%s graphs=%d", what,
                    runner.startup["weights_s"], runner.startup["pool_s"], runner.startup["graphs_s"],
                    runner.manager.num_pages, 0 if runner.graphs is None else len(runner.graphs.captured))
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

    def capture_graphs(self, batch_sizes: Optional[Seq[int]] = None, bounds: Optional[Seq[int]] = None,
                       max_tokens: Optional[int] = None) -> tuple:
        """Capture decode graphs now instead of at their first use, as the reference does at
        start-up (/root/reference/src/pylon/decode/warmup.py:140-167): for these batch sizes
        (default: every size the graphs serve) and these bounds on the requests' lengths
        (default: every bound up to the one that holds ``max_tokens``, itself by default the
        longest request the graphs serve).  Bounds at which the recorded launches are the same
        share one graph (:meth:`DecodeGraphs.key`), so a model of 262,144 positions has a few
        graphs per small batch size and one per large one, not nine.  Throw-away requests of
        one token each take one decode step per graph and are closed again.  Sizes for which
        the pool has no free pages or slots are left to their first use, and so are the bounds
        beyond ``max_tokens``.  Returns the batch sizes that have a graph."""
        if self.graphs is None:
            raise RuntimeError("capture_graphs needs enable_graphs first")
        from ..cache import OutOfPages

        sizes = sorted(set(batch_sizes or range(1, self.graphs.max_batch + 1)))
        if bounds is None:
            bounds = [b for b in self.graphs.bounds() if max_tokens is None or b < 2 * max_tokens]
        bounds = sorted(set(bounds))
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
                    if self.graphs.wants(entries) and self.graphs.key(rows, bound) not in self.graphs.captured:
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
        of the entries and of their ``want``), or None if nothing is wanted.

        A step that fails leaves every request as it was before it: the pages it took go
        back, lengths stay, and fixed-size state that a mixer had already overwritten is put
        back from the copy taken before the step (models without such state copy nothing)."""
        max_positions = self.model.spec.max_positions
        if max_positions:
            for e in entries:
                if e.seq.length + len(e.tokens) > max_positions:
                    raise ValueError(
                        f"The model supports at most {max_positions:,} tokens per request."
                    )
        saved = self.manager.snapshot_state([e.seq for e in entries])
        try:
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
        except Exception:
            self.manager.restore_state(saved)
            raise


def cache_needs(requirements: Seq[object], dtype: torch.dtype, max_requests: int):
    """What a model's runs ask of the cache manager, for the budget: one entry per group of
    runs with equal key/value geometry (``bytes_per_token``, ``window``), and the bytes of all
    fixed-size per-request state for ``max_requests`` requests."""
    elem = torch.empty((), dtype=dtype).element_size()
    by_need, states = group_requirements(requirements)
    groups = []
    for need, cache_ids in by_need.items():
        entry = _Bytes(len(cache_ids) * 2 * need.n_kv_heads * need.head_dim * elem)
        entry.window = need.window
        groups.append(entry)
    state_bytes = sum(max_requests * math.prod(need.shape) * torch.empty((), dtype=need.dtype).element_size()
                      for need in states.values())
    return groups, state_bytes


def measure_activation_bytes(model: Model, config) -> int:
    """The most memory a step takes beside weights and cache: the largest step the serving
    options allow (a prompt portion of ``prefill_chunk_size`` tokens beside one token for each
    of the other ``max_batch_size - 1`` requests, all rows sampling) is run once over a
    throw-away pool of just the pages it needs, and the allocator's peak is read
    (/root/reference/src/pylon/decode/warmup.py:33-120, kv/budget.py:85-95).  To it is added
    what the decode graphs keep for good: their shared ``[max_batch_size, vocab]`` float32
    logits and as much again as the peak of a decode-only step of ``max_batch_size`` rows.
    The run also warms the library's matrix products up for the shapes of a full step."""
    device = model.device
    spec = model.spec
    page = config.page_size
    limit = spec.max_positions or config.prefill_chunk_size + 1
    chunk = max(1, min(config.prefill_chunk_size, limit))
    others = config.max_batch_size - 1
    pages = -(-chunk // page) + others + 1
    runner = Runner(model, page_size=page, num_pages=pages, max_requests=config.max_batch_size)
    seqs = [runner.open(("warm-up", i)) for i in range(config.max_batch_size)]
    try:
        torch.cuda.synchronize(device)
        base = torch.cuda.memory_allocated(device)
        torch.cuda.reset_peak_memory_stats(device)
        decode_peak = 0
        if others:
            runner.step([StepEntry(seq, [0], [0]) for seq in seqs[:others]])
            torch.cuda.synchronize(device)
            decode_peak = torch.cuda.max_memory_allocated(device) - base
            torch.cuda.reset_peak_memory_stats(device)
            entries = [StepEntry(seq, [0], [0]) for seq in seqs[:others]]
        else:
            entries = []
        entries.append(StepEntry(seqs[-1], [0] * chunk, [chunk - 1]))
        runner.step(entries)
        torch.cuda.synchronize(device)
        step_peak = torch.cuda.max_memory_allocated(device) - base
    finally:
        for seq in seqs:
            runner.close(seq)
    graphs = 0
    if config.cuda_graphs:
        graphs = config.max_batch_size * spec.vocab_size * 4 + max(decode_peak, 0)
    del runner
    return max(step_peak, decode_peak, 0) + graphs
