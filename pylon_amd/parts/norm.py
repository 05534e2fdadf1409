"""RMSNorm over the hidden axis (/root/reference/src/pylon/model/layers.py:30-40):
``y = x / sqrt(mean(x^2) + eps) * w`` in float32, rounded once to the activation dtype.
The weight is kept in float32 whatever the model's dtype, as the reference keeps it."""
from __future__ import annotations

from typing import Optional

import torch

from ..config.specs import NormSpec
from ..kernels import ops
from .base import Part
from .registry import register_part


class RMSNorm(Part):
    def __init__(self, spec: NormSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        self.add_param("weight", (spec.dim,), torch.float32, device, role="vector")

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.params["weight"], self.spec.eps, out_dtype=self.dtype)

    def add_forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], *,
                    row_idx: Optional[torch.Tensor] = None) -> torch.Tensor:
        return ops.add_rmsnorm(resid, delta, self.params["weight"], self.spec.eps, self.dtype,
                               row_idx=row_idx)


register_part("norm", "rmsnorm", RMSNorm, replace=True)
