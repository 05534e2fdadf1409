"""The arrangement of a layer's parts.  ``pre_norm``
(/root/reference/src/pylon/model/layers.py:176-200):
``x = x + mixer(norm1(x)); x = x + feed_forward(norm2(x))``.

The residual stream is float32.  A block receives the stream together with the
previous part's output that has not been added yet, so that every residual sum is
formed inside the norm kernel that follows it; it hands back the same pair."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..config.specs import LayerSpec
from .base import Part
from .registry import build_part, register_part


class PreNormBlock(Part):
    def __init__(self, spec: LayerSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        kw = dict(dtype=dtype, device=device)
        self.mixer_norm = self.add_child("mixer_norm", build_part("norm", spec.mixer_norm, **kw))
        self.mixer = self.add_child("mixer", build_part("mixer", spec.mixer, **kw))
        self.feed_forward_norm = self.add_child(
            "feed_forward_norm", build_part("norm", spec.feed_forward_norm, **kw)
        )
        self.feed_forward = self.add_child(
            "feed_forward", build_part("feed_forward", spec.feed_forward, **kw)
        )

    def cache_requirement(self):
        return self.mixer.cache_requirement()

    def decode_signature(self, rows: int, bound: int) -> tuple:
        describe = getattr(self.mixer, "decode_signature", None)
        return ("bound", bound) if describe is None else describe(rows, bound)

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], ctx, cache,
                stores: bool) -> Tuple[torch.Tensor, torch.Tensor]:
        h = self.mixer_norm.add_forward(resid, delta)
        mixed = self.mixer.forward(h, ctx, cache, stores)
        h = self.feed_forward_norm.add_forward(resid, mixed)
        return resid, self.feed_forward.forward(h, ctx)


register_part("block", "pre_norm", PreNormBlock, replace=True)
