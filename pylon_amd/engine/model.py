"""A decoder assembled from parts, and its one forward pass: the step.

The model is architecture-blind: it builds one block per :class:`LayerSpec`, runs the
blocks in the order the schedule lists them, and applies the final norm and the
vocabulary head only at the tokens whose logits are wanted
(/root/reference/src/pylon/model/model.py:124-144).  What an architecture does outside
its layers goes into two optional lists of parts: "stream" parts between the embedding and
the first layer (``forward(resid, ctx) -> resid``, the float32 residual stream of the step's
tokens), "logits" parts after the head (``forward(logits, ctx) -> logits``, float32, one row
per wanted token; under graph replay they must write in place).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..config.specs import ModelSpec
from ..kernels import ops
from ..parts import build_part
from ..parts.base import Part
from .batch import StepContext


class Model(Part):
    def __init__(self, spec: ModelSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("the model runs in float32 or bfloat16")
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.schedule = spec.resolved_schedule()
        self.add_param("embed", (spec.vocab_size, spec.hidden_size), dtype, device)
        if not spec.tie_word_embeddings:
            self.add_param("lm_head", (spec.vocab_size, spec.hidden_size), dtype, device)
        self.blocks: List[Part] = []
        for index, layer in enumerate(spec.layers):
            block = build_part("block", layer, dtype=dtype, device=device)
            self.blocks.append(block)
            self.add_child(f"layers.{index}", block)
        self.final_norm = self.add_child(
            "final_norm", build_part("norm", spec.final_norm, dtype=dtype, device=device)
        )
        self.stream_parts = [self.add_child(f"stream.{i}", build_part("stream", part, dtype=dtype, device=device))
                             for i, part in enumerate(spec.stream_parts)]
        self.logit_parts = [self.add_child(f"logits.{i}", build_part("logits", part, dtype=dtype, device=device))
                            for i, part in enumerate(spec.logit_parts)]

    # ---- what the cache manager has to provide ------------------------------------------
    def cache_requirements(self) -> List[object]:
        """Per run of the schedule: what its mixer keeps (None for a run that borrows)."""
        needs: List[object] = []
        for layer, cache_id, stores in self.schedule:
            needs.append(self.blocks[layer].cache_requirement() if stores else None)
        for index, (layer, cache_id, stores) in enumerate(self.schedule):
            if not stores:
                own = self.blocks[layer].cache_requirement()
                if own != needs[cache_id]:
                    raise ValueError(
                        f"run {index} borrows the cache of run {cache_id}, which has another geometry"
                    )
        return needs

    def decode_signature(self, rows: int, bound: int) -> tuple:
        """What the launches of a decode-only step of ``rows`` requests take from a bound on
        the requests' lengths, over all layers: two bounds with equal signatures record the
        same graph.  A block or mixer without ``decode_signature`` is taken to depend on the
        bound itself."""
        seen = []
        for block in self.blocks:
            describe = getattr(block, "decode_signature", None)
            signature = ("bound", bound) if describe is None else describe(rows, bound)
            if signature not in seen:
                seen.append(signature)
        return tuple(seen)

    @property
    def head_weight(self) -> torch.Tensor:
        return self.params["embed"] if self.spec.tie_word_embeddings else self.params["lm_head"]

    # ---- the step --------------------------------------------------------------------------
    def step(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """Run the step's tokens through every scheduled layer, from and into the cache.
        Returns float32 logits ``[n_logits, vocab]`` (None when no logits are wanted)."""
        resid = ops.embed(ctx.token_ids, self.params["embed"], scale=self.spec.embedding_scale,
                          chosen=ctx.chosen)
        for part in self.stream_parts:
            resid = part.forward(resid, ctx)
        delta = None
        for layer, cache_id, stores in self.schedule:
            resid, delta = self.blocks[layer].forward(resid, delta, ctx, ctx.cache(cache_id), stores)
        if ctx.n_logits == 0:
            return None
        h = self.final_norm.add_forward(resid, delta, row_idx=ctx.logit_idx)
        out = None if ctx.logits_out is None else ctx.logits_out[: ctx.n_logits]
        logits = ops.linear(h, self.head_weight, out_dtype=torch.float32, out=out)
        for part in self.logit_parts:
            logits = part.forward(logits, ctx)  # in place where ``out`` was given
        return logits
