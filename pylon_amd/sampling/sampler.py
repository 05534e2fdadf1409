"""Choosing next tokens from a step's logits on the device.

Greedy rows take the argmax, the others draw from softmax(logits / T) restricted by
top-p (/root/reference/src/pylon/decode/runner.py:509-525).  The reference samples row
groups with separate library calls (/root/reference/src/pylon/engine.py:454-470); here
one kernel takes per-row temperature, top_p and uniform number, and one copy brings the
chosen ids back (the step's only device-to-host synchronisation, engine.py:471).

``launch`` queues the kernel and the copy and returns at once; the ids are read later
from the returned :class:`Draw`.  With ``chosen`` and ``place`` the kernel also leaves
each id in a table on the device, from which the next step can take it before the host
has seen it.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from ..kernels import ops
from .params import Sampling
from .rng import uniform


class Draw:
    """Token ids on their way to the host."""

    def __init__(self, host: torch.Tensor, rows: int, event: Optional[torch.cuda.Event]) -> None:
        self._host = host
        self._rows = rows
        self._event = event
        self._ids: Optional[List[int]] = None

    def result(self) -> List[int]:
        if self._ids is None:
            if self._event is not None:
                self._event.synchronize()
            self._ids = self._host[: self._rows].tolist()
        return self._ids


class Sampler:
    #: Draws in flight at a time before a pinned buffer is used again.
    ROTATION = 4

    def __init__(self, device, max_rows: int = 256) -> None:
        self.device = torch.device(device)
        self._max_rows = 0
        self._cursor = 0
        self._grow(max_rows)

    def _grow(self, rows: int) -> None:
        pin = self.device.type == "cuda"
        if pin and self._max_rows:
            torch.cuda.synchronize(self.device)
        self._max_rows = rows
        self._ids_host = [torch.empty(rows, dtype=torch.int32, pin_memory=pin) for _ in range(self.ROTATION)]
        self._params_host = [torch.empty((3, rows), dtype=torch.float32, pin_memory=pin)
                             for _ in range(self.ROTATION)]
        self._ids_dev = [torch.empty(rows, dtype=torch.int32, device=self.device) for _ in range(self.ROTATION)]
        self._params_dev = [torch.empty((3, rows), dtype=torch.float32, device=self.device)
                            for _ in range(self.ROTATION)]
        self._events: List[Optional[torch.cuda.Event]] = [None] * self.ROTATION

    def launch(self, logits: torch.Tensor, rows: Sequence[Tuple[Sampling, int]], *,
               chosen: Optional[torch.Tensor] = None, place: Optional[torch.Tensor] = None) -> Draw:
        """Queue the choice of one token id per row of ``logits``.  ``rows[r]`` is the row's
        sampling options and the index of the token it is about to produce (which numbers
        its random draw)."""
        n = len(rows)
        if logits.shape[0] != n:
            raise ValueError("one sampling entry per row of logits is required")
        if n > self._max_rows:
            self._grow(max(n, 2 * self._max_rows))
        k = self._cursor
        self._cursor = (k + 1) % self.ROTATION
        if self._events[k] is not None:
            self._events[k].synchronize()  # the buffers' previous use has finished
        out = self._ids_dev[k][:n]
        if all(s.temperature == 0 for s, _ in rows):
            ops.argmax(logits, out=out, chosen=chosen, place=place)
        else:
            params = self._params_host[k].numpy()
            for r, (s, index) in enumerate(rows):
                params[0, r] = s.temperature
                params[1, r] = s.top_p
                params[2, r] = uniform(s.seed or 0, index) if s.temperature > 0 else 0.0
            dev = self._params_dev[k]
            dev.copy_(self._params_host[k], non_blocking=True)
            ops.sample(logits, dev[0, :n], dev[1, :n], dev[2, :n], out=out, chosen=chosen, place=place)
        host = self._ids_host[k]
        host[:n].copy_(out, non_blocking=True)
        event = None
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
        self._events[k] = event
        return Draw(host, n, event)

    def sample(self, logits: torch.Tensor, rows: Sequence[Tuple[Sampling, int]]) -> List[int]:
        """One token id per row of ``logits``, waited for."""
        return self.launch(logits, rows).result()
