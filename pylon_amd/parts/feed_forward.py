"""Gated feed-forward, gate and up fused into one matrix
(/root/reference/src/pylon/model/layers.py:13-27): ``down(silu(gate(h)) * up(h))``."""
from __future__ import annotations

import torch

from ..config.specs import GatedFeedForwardSpec
from ..kernels import ops, plan
from .base import Part
from .registry import register_part


class GatedFeedForward(Part):
    def __init__(self, spec: GatedFeedForwardSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.activation != "silu":
            raise ValueError(f"activation {spec.activation!r} is not supported (only 'silu')")
        self.spec = spec
        self.dtype = dtype
        element_size = torch.empty((), dtype=dtype).element_size()
        self.add_param("gate_up", (2 * spec.intermediate_size, spec.hidden_size), dtype, device,
                       row_padding=plan.gated_row_padding(spec.hidden_size, element_size))
        self.add_param("down", (spec.hidden_size, spec.intermediate_size), dtype, device)

    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        hidden = ops.linear_glu(h, self.params["gate_up"], out_dtype=self.dtype)
        return ops.linear_for_residual(hidden, self.params["down"], out_dtype=self.dtype)


register_part("feed_forward", "gated_mlp", GatedFeedForward, replace=True)
