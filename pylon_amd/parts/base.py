"""What every part of a layer looks like to the model that assembles it.

A part owns named parameters (device tensors the weight loader fills by path) and a
``forward``.  It gets its sizes and constants from its spec and the batch from the
step context; it does not know which model, or which layer of it, it sits in.

Interfaces
----------
norm          ``forward(x) -> y`` and ``add_forward(resid, delta, row_idx=None) -> y``:
              ``resid`` is the float32 residual stream, ``delta`` the previous part's
              output (or None), either ``[tokens, dim]`` or a stack ``[parts, tokens, dim]``
              of float32 partial sums still to be added up (:func:`summed` makes one float32
              tensor of either); the sum is formed in float32, stored back into
              ``resid`` (unless ``row_idx`` picks rows), and its norm is returned in
              the activation dtype.
position      ``rotary() -> (inv_freq, rotary_dim) | None`` for encodings applied by
              rotating q and k: float32 frequencies of the pairs ``(i, i + rotary_dim/2)``
              of the first ``rotary_dim`` elements of a head; None encodes nothing.
mixer         ``cache_requirement() -> KVRequirement | StateRequirement | None`` and
              ``forward(h, ctx, cache, stores) -> [tokens, hidden]`` (or partial sums
              ``[parts, tokens, hidden]`` in float32, see norm): ``cache`` is the
              view of the run's cache (its own, or the one it borrows); ``stores``
              says whether this run writes it.
feed_forward  ``forward(h, ctx) -> [tokens, hidden]``.
block         ``forward(resid, delta, ctx, cache, stores) -> (resid, delta)``: takes and
              returns the residual stream and the not-yet-added output of the last part.
stream        ``forward(resid, ctx) -> resid``: the embedded tokens (float32 ``[tokens, dim]``)
              before the first layer: an embedding norm, learned positions
              (``ctx.positions``), a scale.
logits        ``forward(logits, ctx) -> logits``: float32 ``[wanted, vocab]`` after the
              vocabulary head: a soft cap, a scale, a bias (in place).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterator, Optional, Tuple

import torch


@dataclass(frozen=True)
class KVRequirement:
    """A growing cache of keys and values: one entry per token, in pages.

    Runs whose requirements are equal share a group of pages (one block table)."""

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None  # keep only the last `window` tokens' entries


@dataclass(frozen=True)
class StateRequirement:
    """Per-request state of fixed size, overwritten in place by every step."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


def summed(delta: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """A part's output that has not been added to the residual stream yet, as one float32
    ``[tokens, dim]`` tensor.  What a mixer or a feed-forward hands on is either a tensor of
    that shape in the activation dtype or a stack ``[parts, tokens, dim]`` of float32 partial
    sums (the product kernels cut the reduction over workgroups for some row counts); which
    of the two depends on the step's size, so a norm or a block that adds it up itself goes
    through this function (the built-in norm kernel takes both forms directly)."""
    if delta is None:
        return None
    return delta.sum(dim=0) if delta.dim() == 3 else delta.float()


class Part:
    """Base of all parts: a bag of named parameters and named sub-parts."""

    def __init__(self) -> None:
        self.params: Dict[str, torch.Tensor] = {}
        self.param_roles: Dict[str, str] = {}
        self.children: Dict[str, "Part"] = {}

    def add_param(self, name: str, shape, dtype: torch.dtype, device, role: str = "matrix",
                  row_padding: int = 0) -> None:
        """``row_padding``: elements left unused behind every row of a matrix in memory; the
        parameter is then the view of its rows without them, with a row stride of its own."""
        shape = tuple(shape)
        if row_padding and len(shape) == 2:
            self.params[name] = torch.empty((shape[0], shape[1] + row_padding), dtype=dtype,
                                            device=device)[:, : shape[1]]
        else:
            self.params[name] = torch.empty(shape, dtype=dtype, device=device)
        self.param_roles[name] = role

    def add_child(self, name: str, part: "Part") -> "Part":
        self.children[name] = part
        return part

    def named_params(self, prefix: str = "") -> Iterator[Tuple[str, "Part", str]]:
        """``(path, owner, name)`` of every parameter below this part."""
        for name in self.params:
            yield prefix + name, self, name
        for child_name, child in self.children.items():
            yield from child.named_params(prefix + child_name + ".")
