"""Choosing next tokens from a step's logits on the device.

Greedy rows take the argmax, the others draw from softmax(logits / T) restricted by
top-p (/root/reference/src/pylon/decode/runner.py:509-525).  The reference samples row
groups with separate library calls (/root/reference/src/pylon/engine.py:454-470); here
one kernel takes per-row temperature, top_p and uniform number, and one copy brings the
chosen ids back (the step's only device-to-host synchronisation, engine.py:471).
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops
from .params import Sampling
from .rng import uniform


class Sampler:
    def __init__(self, device) -> None:
        self.device = torch.device(device)

    def sample(self, logits: torch.Tensor, rows: Sequence[Tuple[Sampling, int]]) -> List[int]:
        """One token id per row of ``logits``.  ``rows[r]`` is the row's sampling options
        and the index of the token it is about to produce (which numbers its random draw)."""
        if logits.shape[0] != len(rows):
            raise ValueError("one sampling entry per row of logits is required")
        if all(s.temperature == 0 for s, _ in rows):
            return ops.argmax(logits).cpu().tolist()
        params = np.empty((3, len(rows)), dtype=np.float32)
        for r, (s, index) in enumerate(rows):
            params[0, r] = s.temperature
            params[1, r] = s.top_p
            params[2, r] = uniform(s.seed, index) if s.temperature > 0 else 0.0
        dev = torch.from_numpy(params).to(self.device)
        return ops.sample(logits, dev[0], dev[1], dev[2]).cpu().tolist()
