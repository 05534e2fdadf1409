"""Per-request sampling options, with the reference's names, defaults and ranges
(/root/reference/src/pylon/api/types.py:6-9), plus a seed: the reference draws from
torch's global generator and so cannot repeat a run.  A request with a seed draws the
same tokens whenever and beside whatever it runs; a request without one (``seed=None``,
the default) is given a fresh seed when it is enqueued, so that two equal prompts sampled
at a temperature above 0 may differ, as they do in the reference."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class Sampling:
    max_new_tokens: int = 256
    temperature: float = 0.2
    top_p: float = 0.95
    seed: Optional[int] = None

    def __post_init__(self) -> None:
        if isinstance(self.max_new_tokens, bool) or not isinstance(self.max_new_tokens, int):
            raise ValueError("max_new_tokens must be an integer.")
        if not 1 <= self.max_new_tokens <= 2048:
            raise ValueError("max_new_tokens must be between 1 and 2048.")
        if not (math.isfinite(self.temperature) and 0 <= self.temperature <= 2):
            raise ValueError("temperature must be between 0 and 2.")
        if not (math.isfinite(self.top_p) and 0 < self.top_p <= 1):
            raise ValueError("top_p must be greater than 0 and at most 1.")
        if self.seed is not None and (isinstance(self.seed, bool) or not isinstance(self.seed, int)
                                      or self.seed < 0):
            raise ValueError("seed must be a non-negative integer (or None for a fresh one per request).")
