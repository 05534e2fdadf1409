"""The scheduler's decisions, as pure functions of small records: who is admitted, how
prompts are cut into portions under the token budget, and when prompt work is held back.
Nothing here touches the device, a thread or a clock of its own, so every rule can be
tested by calling it.

The rules are the reference's:

* Admission (/root/reference/src/pylon/scheduler/admit.py:11-95).  A request reserves
  pages for its whole life, ``ceil((prompt + max_new) / page_size)``
  (/root/reference/src/pylon/engine.py:168-171).  It fits if all reservations stay within
  the pool and the unreserved rest still has one page per decoding request.  A request
  whose own reservation exceeds the pool is rejected; the others go on.  If the head of
  the queue does not fit and has waited under 100 ms, later arrivals are tried in order:
  the first that fits goes ahead; the scan stops at one that has waited 100 ms or after
  ``admit_skip`` that did not fit.
* Portions (/root/reference/src/pylon/scheduler/batch.py:6-54).  Up to
  ``prefill_chunk_size`` prompt tokens per step over as many requests as fit; a request
  whose prompt work has waited 100 ms first (oldest first), else the first whose rest
  fits into the budget left, else the first; each takes ``min(budget left, rest)``.
* Hold-back (/root/reference/src/pylon/engine.py:30-35).  With the decode batch full and
  the oldest prompt work younger than 100 ms, a step is decode-only.

Because reservations cover whole lives, pages cannot run out during a step; if a step
is refused for pages all the same, the engine fails the running requests and frees their
pages (/root/reference/src/pylon/engine.py:260-264,716-722).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

WAIT_LIMIT_SECONDS = 0.1  # the three 100 ms rules of the reference share this value


@dataclass(frozen=True)
class Waiter:
    """What admission needs to know about a queued request."""

    key: object
    tokens: int  # prompt + max_new_tokens
    arrived: float


@dataclass(frozen=True)
class Verdict:
    """Outcome for one waiter: start it (``pages`` reserved), or reject it for good."""

    key: object
    admit: bool
    pages: int = 0
    skipped_head: bool = False
    reason: str = ""


class AdmissionPolicy:
    def __init__(self, *, page_budget: int, page_size: int, admit_skip: int) -> None:
        self.page_budget = page_budget
        self.page_size = page_size
        self.admit_skip = admit_skip

    def pages(self, tokens: int) -> int:
        return (tokens + self.page_size - 1) // self.page_size

    def fits(self, tokens: int, reserved_pages: int, decoding: int) -> bool:
        total = reserved_pages + self.pages(tokens)
        if total > self.page_budget:
            return False
        return self.page_budget - total >= decoding  # the free-page floor

    def next(self, waiting: Sequence[Waiter], *, reserved_pages: int, decoding: int,
             now: float) -> Optional[Verdict]:
        """The next waiter to deal with, or None when admission has to wait."""
        if not waiting:
            return None
        for position, waiter in enumerate(waiting):
            if self.pages(waiter.tokens) > self.page_budget:
                return Verdict(waiter.key, admit=False,
                               reason="The FIFO request cannot fit in the KV-cache budget.")
            if self.fits(waiter.tokens, reserved_pages, decoding):
                return Verdict(waiter.key, admit=True, pages=self.pages(waiter.tokens),
                               skipped_head=position > 0)
            waited_out = now - waiter.arrived >= WAIT_LIMIT_SECONDS
            # Nobody overtakes a waiter that has aged; behind the head, `admit_skip`
            # waiters that do not fit may be passed over, and the one after them is
            # still looked at.
            passed_over = position - 1 if position else self.admit_skip - 1
            if waited_out or self.admit_skip <= 0 or passed_over >= self.admit_skip:
                return None
        return None


@dataclass(frozen=True)
class PromptWork:
    """A request with prompt tokens still to run."""

    key: object
    remaining: int
    waiting_since: float


def cut_prompts(work: Sequence[PromptWork], budget: int, now: float) -> List[Tuple[object, int]]:
    """``(key, tokens)`` portions for this step, in the order they were chosen."""
    pending = [w for w in work if w.remaining > 0]
    chosen: List[Tuple[object, int]] = []
    while pending and budget > 0:
        aged = [w for w in pending if now - w.waiting_since >= WAIT_LIMIT_SECONDS]
        if aged:
            pick = min(aged, key=lambda w: w.waiting_since)
        else:
            pick = next((w for w in pending if w.remaining <= budget), pending[0])
        pending.remove(pick)
        count = min(budget, pick.remaining)
        chosen.append((pick.key, count))
        budget -= count
    return chosen


def hold_prompts(decoding: int, max_batch_size: int, work: Sequence[PromptWork], now: float) -> bool:
    """True when this step should carry decode tokens only."""
    ages = [now - w.waiting_since for w in work if w.remaining > 0]
    if decoding != max_batch_size or not ages:
        return False
    return max(ages) < WAIT_LIMIT_SECONDS
