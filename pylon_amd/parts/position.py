"""Position encodings a mixer can be given.

``rope`` follows /root/reference/src/pylon/model/layers.py:43-51 and :73-78: frequencies
``theta ** (-2i/d)`` formed in float32, the angle of a token is ``position * frequency``
(float32), and element ``i`` of a head is rotated together with element ``i + d/2``.
The reference gathers cos/sin from tables of ``max_position_embeddings`` rows; here the
fused q/k kernel forms the angle from the position, which gives the same float32 value.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..config.specs import PositionSpec
from .base import Part
from .registry import register_part


class RotaryPosition(Part):
    def __init__(self, spec: PositionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.rotary_dim < 2 or spec.rotary_dim % 2:
            raise ValueError("rotary_dim must be even and at least 2")
        self.spec = spec
        exponents = torch.arange(0, spec.rotary_dim, 2, dtype=torch.float32) / spec.rotary_dim
        inv_freq = 1.0 / (torch.tensor(spec.theta, dtype=torch.float32) ** exponents)
        self.inv_freq = inv_freq.to(device)

    def rotary(self) -> Optional[Tuple[torch.Tensor, int]]:
        return self.inv_freq, self.spec.rotary_dim


class NoPosition(Part):
    def __init__(self, spec: PositionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec

    def rotary(self):
        return None


register_part("position", "rope", RotaryPosition, replace=True)
register_part("position", "none", NoPosition, replace=True)
