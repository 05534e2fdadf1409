"""The engine: the programming entry point on token ids.

``Engine.enqueue(input_ids, eos_token_id, sampling, request_id) -> Future[GenerationResult]``
has the reference's signature and meaning (/root/reference/src/pylon/engine.py:241-253);
``generate`` is the same for a list of prompts, run to completion in the calling thread.
A tick is the reference's (/root/reference/src/pylon/engine.py:255-300): drop cancelled
requests, admit, run one step that carries every decoding request's pending token beside
the prompt portions the token budget allows, sample where a row is ready, finish or
continue each request, admit again into what was freed.

Running ahead (``PylonConfig.run_ahead``, when the step executor keeps the sampler's last
token of each request on the device): a tick queues its step and its sampling and only
then reads the tokens of the tick before, so the device never waits for the host.  A
decoding request's token is fed from the device (:data:`~pylon_amd.engine.batch.PENDING`).
A request that meets a stop token has then already been given one more step; that step's
token is dropped.  The end by ``max_new_tokens`` is known beforehand and costs nothing.
"""
from __future__ import annotations

import dataclasses
import logging
import random
import threading
import time
from collections import deque
from concurrent.futures import Future
from dataclasses import dataclass, field
from typing import Callable, Deque, Iterable, List, Optional, Sequence, Tuple

from ..config.engine_config import PylonConfig
from ..sampling.params import Sampling
from .batch import PENDING, StepEntry
from .scheduler import AdmissionPolicy, PromptWork, Waiter, cut_prompts, hold_prompts

logger = logging.getLogger("pylon")


class QueueFullError(RuntimeError):
    pass


class EngineClosedError(RuntimeError):
    pass


@dataclass(frozen=True)
class GenerationResult:
    """/root/reference/src/pylon/engine.py:59-74, without the prefix-cache and
    speculation fields."""

    output_ids: List[int]
    finish_reason: str  # "eos" or "length"
    prefill_seconds: float
    inter_token_seconds: List[float]
    queue_seconds: float
    first_token_at: Optional[float] = None  # on the engine's clock
    first_token_seconds: Optional[float] = None
    token_intervals: Optional[Tuple[float, ...]] = None  # between the reads of emitted tokens
    elapsed_seconds: Optional[float] = None


@dataclass(frozen=True)
class Request:
    input_ids: List[int]
    stop_ids: frozenset
    sampling: Sampling
    request_id: str


@dataclass
class Flight:
    """A queued step whose sampled tokens have not been read yet."""

    draw: object  # .result() -> token ids of `ready`, in order
    ready: List["Active"]
    decoding: List["Active"]
    portions: List[Tuple["Active", int]]
    started: float


@dataclass
class Ticket:
    """A request waiting for admission."""

    request: Request
    future: Future
    arrived: float


@dataclass
class Active:
    """A request that holds a cache: prefilling (no pending token) or decoding."""

    ticket: Ticket
    seq: object
    reserved_pages: int
    output_ids: List[int] = field(default_factory=list)
    prompt_offset: int = 0
    pending_token_id: Optional[int] = None
    queue_seconds: float = 0.0
    prefill_seconds: float = 0.0
    inter_token_seconds: List[float] = field(default_factory=list)
    prompt_wait_started: float = 0.0
    first_token_at: Optional[float] = None
    last_token_at: Optional[float] = None
    token_intervals: List[float] = field(default_factory=list)
    # Running ahead: a sampled token waits on the device to be fed / how many sampled
    # tokens the host has not read yet / the request has ended.
    awaiting: bool = False
    unread: int = 0
    done: bool = False

    @property
    def request(self) -> Request:
        return self.ticket.request

    @property
    def decoding(self) -> bool:
        return self.pending_token_id is not None or self.awaiting

    @property
    def remaining_prompt(self) -> int:
        return len(self.request.input_ids) - self.prompt_offset


def _stop_ids(eos_token_id) -> frozenset:
    if eos_token_id is None:
        return frozenset()
    if isinstance(eos_token_id, int):
        return frozenset((eos_token_id,))
    return frozenset(eos_token_id)


class Engine:
    def __init__(self, config: PylonConfig, *, runner=None, sampler=None,
                 clock: Callable[[], float] = time.perf_counter, threaded: bool = False) -> None:
        """``runner`` executes steps (a :class:`~pylon_amd.engine.runner.Runner`; built from
        ``config.model_path`` when not given).  ``threaded`` starts the background thread
        that ticks on its own, as the reference's scheduler thread does; without it the
        caller drives the engine with :meth:`tick`, :meth:`run_until_idle` or
        :meth:`generate`."""
        self._config = config
        self._clock = clock
        if runner is None:
            runner = _load_runner(config)
        self.runner = runner
        if sampler is None:
            from ..sampling.sampler import Sampler

            sampler = Sampler(runner.model.device)
        self.sampler = sampler
        manager = runner.manager
        self.page_size = manager.page_size
        self.kv_budget_pages = manager.num_pages
        self._run_ahead = bool(config.run_ahead and hasattr(runner, "chosen")
                               and hasattr(sampler, "launch"))
        self._flight: Optional[Flight] = None
        self._landed_at = 0.0
        self._policy = AdmissionPolicy(page_budget=manager.num_pages, page_size=manager.page_size,
                                       admit_skip=config.admit_skip)
        self._max_batch_size = config.max_batch_size
        self._prefill_chunk_size = config.prefill_chunk_size
        self._waiting: Deque[Ticket] = deque()
        self._active: List[Active] = []
        self._lock = threading.RLock()
        self._wake = threading.Condition(self._lock)
        self._ticking = threading.Lock()  # one tick at a time
        self._closed = False
        self.head_skips = 0
        self._serial = 0
        self._seeds = random.Random()  # seeds of requests that bring none (from the system's entropy)
        self.steps_run = 0
        self.last_step = None  # (decode rows, prompt portions) of the most recent step
        self._thread: Optional[threading.Thread] = None
        if threaded:
            self._thread = threading.Thread(target=self._drive, name="pylon-scheduler", daemon=True)
            self._thread.start()

    # ---- construction helpers ----------------------------------------------------------
    @classmethod
    def from_folder(cls, folder, **options) -> "Engine":
        threaded = options.pop("threaded", False)
        return cls(PylonConfig(model_path=str(folder), **options), threaded=threaded)

    @classmethod
    def from_random(cls, model_config: dict, seed: int = 0, *, std: Optional[float] = None,
                    norm_jitter: float = 0.0, draw_on=None, config: Optional[PylonConfig] = None,
                    **options) -> "Engine":
        """An engine over random weights of the architecture and sizes that ``model_config``
        (the contents of a config.json) names, drawn in place on the device by the
        random-weights mode's rule (``draw_on="cpu"``: the very numbers of the folder that the
        mode writes from the same config and seed).  Serving options as ``config`` or as
        keywords.  Start-up is :meth:`Runner.from_random`: the same fit check, pool sizing and
        graph capture as for a model folder."""
        from .runner import Runner

        threaded = options.pop("threaded", False)
        if config is not None and options:
            raise TypeError("give the serving options as `config` or as keywords, not both")
        config = config if config is not None else PylonConfig(**options)
        runner = Runner.from_random(model_config, seed, config, std=std, norm_jitter=norm_jitter, draw_on=draw_on)
        return cls(config, runner=runner, threaded=threaded)

    # ---- the public surface -------------------------------------------------------------
    def enqueue(self, input_ids: Sequence[int], eos_token_id=None, sampling: Optional[Sampling] = None,
                request_id: Optional[str] = None) -> Future:
        sampling = sampling or Sampling()
        if sampling.seed is None:
            # No seed given: every request draws from a stream of its own, as requests of
            # the reference differ, which all draw from one global generator
            # (/root/reference/src/pylon/decode/runner.py:513-525).  A given seed repeats.
            sampling = dataclasses.replace(sampling, seed=self._seeds.getrandbits(63))
        request_id = request_id or "internal"
        stop_ids = _stop_ids(eos_token_id)
        input_ids = list(input_ids)
        self._validate_request(input_ids, stop_ids, sampling)
        ticket = Ticket(Request(input_ids, stop_ids, sampling, request_id), Future(), self._clock())
        with self._wake:
            if self._closed:
                raise EngineClosedError("The generation scheduler is closed.")
            self._sweep_cancelled_waiting()
            if len(self._waiting) >= self._config.max_queue_size:
                raise QueueFullError("The generation waiting queue is full.")
            self._waiting.append(ticket)
            self._wake.notify_all()
        logger.info("request_waiting request_id=%s", request_id)
        return ticket.future

    def generate(self, prompts: Iterable[Sequence[int]], sampling: Optional[Sampling] = None,
                 eos_token_id=None) -> List[GenerationResult]:
        """Run the prompts to completion and return their results in order.  More prompts
        than the queue holds are fed in as earlier ones finish."""
        prompts = [list(p) for p in prompts]
        futures: List[Optional[Future]] = [None] * len(prompts)
        nxt = 0
        while True:
            while nxt < len(prompts) and len(self._waiting) < self._config.max_queue_size:
                futures[nxt] = self.enqueue(prompts[nxt], eos_token_id, sampling, f"generate-{nxt}")
                nxt += 1
            if self._thread is not None:
                break
            busy = self.tick()
            if not busy and nxt >= len(prompts):
                break
        if self._thread is not None:
            for i in range(nxt, len(prompts)):
                while len(self._waiting) >= self._config.max_queue_size:
                    time.sleep(0.001)
                futures[i] = self.enqueue(prompts[i], eos_token_id, sampling, f"generate-{i}")
        return [f.result() for f in futures]

    def run_until_idle(self) -> None:
        while self.tick():
            pass

    def close(self) -> None:
        with self._wake:
            if self._closed:
                return
            self._closed = True
            waiting, self._waiting = list(self._waiting), deque()
            active, self._active = self._active, []
            self._flight = None
            self._wake.notify_all()
        error = EngineClosedError("The generation scheduler is closed.")
        for item in active:
            self.runner.close(item.seq)
            if not item.ticket.future.done():
                item.ticket.future.set_exception(error)
        for ticket in waiting:
            if not ticket.future.done():
                ticket.future.set_exception(error)
        if self._thread is not None and self._thread is not threading.current_thread():
            self._thread.join()

    def snapshot(self) -> dict:
        with self._lock:
            return {
                "waiting": [t.request.request_id for t in self._waiting],
                "active": [a.request.request_id for a in self._active],
                "max_batch_size": self._max_batch_size,
                "max_queue_size": self._config.max_queue_size,
                "batch_wait_ms": self._config.batch_wait_ms,
            }

    # ---- page accounting ----------------------------------------------------------------
    def request_cache_pages(self, token_count: int) -> int:
        return self._policy.pages(token_count)

    def reserved_pages(self) -> int:
        return sum(item.reserved_pages for item in self._active)

    # ---- one tick ---------------------------------------------------------------------------
    def tick(self) -> bool:
        """One round of admit, step, sample, finish.  True while work remains.

        The engine's lock guards its queue and its lists of requests, not the device: where a
        tick waits for the device (reading a step's sampled tokens, or the end of a step that
        sampled nothing), it has released the lock, so that ``enqueue``, ``snapshot`` and
        ``close`` from other threads do not wait for a step.  One exception: a decode graph
        that start-up did not capture (a request longer than ``cuda_graph_max_tokens``) is
        captured at its first use, inside the step, under the lock.  Ticks themselves run one
        at a time."""
        with self._ticking:
            with self._lock:
                if self._closed:
                    return False
                self._drop_cancelled_active()
                self._admit()
                flight = None
                try:
                    flight = self._launch_step() if self._active else None
                    if self._run_ahead:
                        # The step just queued runs behind the one before it; now read that one.
                        flight, self._flight = self._flight, flight
                except Exception as error:
                    logger.exception("model_batch_failed")
                    self._fail_active(error)
                    flight = None
            token_ids, failure = [], None
            if flight is not None and flight.draw is not None:
                try:
                    token_ids = flight.draw.result()  # waits for the device
                except Exception as error:  # noqa: BLE001 - reported under the lock below
                    failure = error
            with self._lock:
                if self._closed:
                    return False
                if failure is not None:
                    logger.error("model_batch_failed: %s", failure)
                    self._fail_active(failure)
                elif flight is not None:
                    self._land(flight, token_ids)
                self._admit()
                return bool(self._active or self._waiting or self._flight)

    # ---- admission ----------------------------------------------------------------------------
    def _sweep_cancelled_waiting(self) -> None:
        if any(t.future.cancelled() for t in self._waiting):
            self._waiting = deque(t for t in self._waiting if not t.future.cancelled())

    def _admit(self) -> None:
        while len(self._active) < self._max_batch_size:
            self._sweep_cancelled_waiting()
            if not self._waiting:
                return
            waiters = [
                Waiter(t, len(t.request.input_ids) + t.request.sampling.max_new_tokens, t.arrived)
                for t in self._waiting
            ]
            decoding = sum(1 for a in self._active if a.decoding)
            verdict = self._policy.next(waiters, reserved_pages=self.reserved_pages(),
                                        decoding=decoding, now=self._clock())
            if verdict is None:
                logger.info("continuous_admission_blocked request_id=%s reason=memory",
                            self._waiting[0].request.request_id)
                return
            ticket: Ticket = verdict.key
            self._waiting.remove(ticket)
            if not ticket.future.set_running_or_notify_cancel():
                continue
            if not verdict.admit:
                ticket.future.set_exception(RuntimeError(verdict.reason))
                continue
            if self._start(ticket, verdict.pages) and verdict.skipped_head:
                self.head_skips += 1
        if self._waiting:
            logger.info("continuous_admission_blocked request_id=%s reason=slots",
                        self._waiting[0].request.request_id)

    def _start(self, ticket: Ticket, pages: int) -> bool:
        request = ticket.request
        capacity = len(request.input_ids) + request.sampling.max_new_tokens
        try:
            self._serial += 1
            seq = self.runner.open((request.request_id, self._serial), capacity)
        except Exception as error:
            ticket.future.set_exception(error)
            return False
        self._active.append(Active(
            ticket=ticket, seq=seq, reserved_pages=pages,
            queue_seconds=self._clock() - ticket.arrived, prompt_wait_started=ticket.arrived,
        ))
        return True

    # ---- the step -----------------------------------------------------------------------------
    def _launch_step(self) -> Optional[Flight]:
        """Queue one step and the sampling of its ready rows."""
        now = self._clock()
        # A request whose unread tokens complete its max_new_tokens gets no further step.
        decoding = [a for a in self._active if a.decoding
                    and len(a.output_ids) + a.unread < a.request.sampling.max_new_tokens]
        work = [PromptWork(a, a.remaining_prompt, a.prompt_wait_started)
                for a in self._active if not a.decoding and a.remaining_prompt > 0]
        portions: List[Tuple[Active, int]] = []
        if not hold_prompts(len(decoding), self._max_batch_size, work, now):
            portions = cut_prompts(work, self._prefill_chunk_size, now)
        # Decode rows first, then prompt portions; the portions' token budget is not
        # reduced by the decode rows (/root/reference/src/pylon/engine.py:292-298).
        entries: List[StepEntry] = []
        ready: List[Active] = []
        for item in decoding:
            token = PENDING if item.awaiting else item.pending_token_id
            entries.append(StepEntry(item.seq, [token], [0]))
            ready.append(item)
        for item, count in portions:
            chunk = item.request.input_ids[item.prompt_offset: item.prompt_offset + count]
            finishes = item.prompt_offset + count >= len(item.request.input_ids)
            entries.append(StepEntry(item.seq, chunk, [count - 1] if finishes else []))
            if finishes:
                ready.append(item)
        if not entries:
            return None
        self.last_step = ([a.request.request_id for a in decoding],
                          [(a.request.request_id, c) for a, c in portions])
        started = self._clock()
        logits = self.runner.step(entries)
        self.steps_run += 1
        for item, count in portions:
            item.prompt_offset += count
            item.prompt_wait_started = self._clock()
        for item in decoding:
            item.pending_token_id = None
            item.awaiting = False
        draw = None
        if ready:
            rows = [(a.request.sampling, len(a.output_ids) + a.unread) for a in ready]
            if self._run_ahead:
                draw = self.sampler.launch(logits, rows, chosen=self.runner.chosen,
                                           place=self.runner.logit_slots)
                for item in ready:
                    item.awaiting = True
            elif hasattr(self.sampler, "launch"):
                draw = self.sampler.launch(logits, rows)  # read outside the lock, by tick
            else:
                draw = _Drawn(self.sampler.sample(logits, rows))
            for item in ready:
                item.unread += 1
        elif not self._run_ahead and hasattr(self.runner, "synchronize"):
            draw = _Finished(self.runner)  # nothing sampled: tick waits for the step, lock released
        return Flight(draw, ready, decoding, portions, started)

    def _land(self, flight: Flight, token_ids: Sequence[int]) -> None:
        """A step's tokens have been read: finish or continue its requests."""
        sampled_at = self._clock()
        elapsed = sampled_at - max(flight.started, self._landed_at)
        self._landed_at = sampled_at
        for item in flight.decoding:
            item.inter_token_seconds.append(elapsed)
        for item, _count in flight.portions:
            item.prefill_seconds += elapsed
        for item, token_id in zip(flight.ready, token_ids):
            if item.done:
                continue  # ended meanwhile (a stop token seen one step late, a cancellation)
            item.unread -= 1
            if not self._accept(item, int(token_id), sampled_at):
                item.done = True
        self._active = [a for a in self._active if not a.done]

    def _accept(self, item: Active, token_id: int, sampled_at: float) -> bool:
        """/root/reference/src/pylon/engine.py:598-618: a stop token ends the request and
        is not emitted; reaching max_new_tokens ends it with "length"."""
        if item.first_token_at is None:
            item.first_token_at = sampled_at
        if token_id in item.request.stop_ids:
            self._complete(item, "eos")
            return False
        if item.last_token_at is not None:
            item.token_intervals.append(sampled_at - item.last_token_at)
        item.last_token_at = sampled_at
        item.output_ids.append(token_id)
        if len(item.output_ids) == item.request.sampling.max_new_tokens:
            self._complete(item, "length")
            return False
        if not self._run_ahead:
            item.pending_token_id = token_id  # running ahead, the device feeds it
        return True

    def _complete(self, item: Active, reason: str) -> None:
        self.runner.close(item.seq)
        arrived = item.ticket.arrived
        result = GenerationResult(
            output_ids=item.output_ids, finish_reason=reason, prefill_seconds=item.prefill_seconds,
            inter_token_seconds=item.inter_token_seconds, queue_seconds=item.queue_seconds,
            first_token_at=item.first_token_at,
            first_token_seconds=None if item.first_token_at is None else item.first_token_at - arrived,
            token_intervals=tuple(item.token_intervals),
            elapsed_seconds=self._clock() - arrived,
        )
        if not item.ticket.future.done():
            item.ticket.future.set_result(result)

    def _drop_cancelled_active(self) -> None:
        kept = []
        for item in self._active:
            if item.ticket.future.cancelled():
                item.done = True
                self.runner.close(item.seq)
            else:
                kept.append(item)
        self._active = kept

    def _fail_active(self, error: Exception) -> None:
        """A step that raised (pages ran short, a kernel refused) fails every running
        request and frees what they hold; waiting requests stay queued."""
        for item in self._active:
            item.done = True
            self.runner.close(item.seq)
            if not item.ticket.future.done():
                item.ticket.future.set_exception(error)
        self._active = []
        self._flight = None

    # ---- validation ---------------------------------------------------------------------------
    def _validate_request(self, input_ids: List[int], stop_ids: frozenset, sampling: Sampling) -> None:
        """/root/reference/src/pylon/engine.py:731-759."""
        spec = self.runner.model.spec
        if not input_ids:
            raise ValueError("A request prompt must contain at least one token.")
        for token_id in (*stop_ids, *input_ids):
            if isinstance(token_id, bool) or not isinstance(token_id, int) or not 0 <= token_id < spec.vocab_size:
                raise ValueError(f"Token IDs must be between 0 and {spec.vocab_size - 1:,}.")
        token_count = len(input_ids) + sampling.max_new_tokens
        if spec.max_positions and token_count > spec.max_positions:
            raise ValueError(
                f"Request needs {token_count:,} cache positions, but the model supports "
                f"{spec.max_positions:,}."
            )
        max_tokens = self.kv_budget_pages * self.page_size
        if token_count > max_tokens:
            raise ValueError(
                f"Request needs {token_count:,} KV-cache tokens, but the profiled limit "
                f"is {max_tokens:,}."
            )

    # ---- the background thread ----------------------------------------------------------------
    def _drive(self) -> None:
        wait = self._config.batch_wait_ms / 1_000
        while True:
            with self._wake:
                while not self._waiting and not self._active and not self._closed:
                    self._wake.wait()
                if self._closed:
                    return
                if not self._active and self._max_batch_size > 1 and self._waiting:
                    # Nothing is running: give more arrivals a moment to join the first
                    # step (/root/reference/src/pylon/scheduler/queue.py:157-166).
                    deadline = self._waiting[0].arrived + wait
                    while (self._waiting and len(self._waiting) < self._max_batch_size
                           and not self._closed):
                        remaining = deadline - self._clock()
                        if remaining <= 0:
                            break
                        self._wake.wait(remaining)
                    if self._closed:
                        return
            try:
                self.tick()
            except Exception as error:  # noqa: BLE001 - a broken tick fails what runs
                with self._lock:
                    self._fail_active(error)


class _Finished:
    """A step that sampled nothing: waiting for it yields no token ids."""

    def __init__(self, runner) -> None:
        self._runner = runner

    def result(self) -> List[int]:
        self._runner.synchronize()
        return []


class _Drawn:
    """Token ids that are already on the host."""

    def __init__(self, ids: List[int]) -> None:
        self._ids = ids

    def result(self) -> List[int]:
        return self._ids


def _load_runner(config: PylonConfig):
    import torch

    from .runner import Runner

    if config.model_path is None:
        raise ValueError("PylonConfig.model_path (or PYLON_MODEL_PATH) names no model folder.")
    if not torch.cuda.is_available():
        raise RuntimeError("A GPU is required.")
    return Runner.from_config(config)
