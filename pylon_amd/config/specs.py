"""Typed descriptions of the parts a decoder is assembled from.

A model is data: a tuple of :class:`LayerSpec` (what each layer is made of) and a
tuple of :class:`ScheduleEntry` (in which order layers run and whose cache each
run uses).  Every size and constant a part needs is a field of its spec; the
parts never look at an architecture's config.json themselves.

The specs mirror what the reference hard-codes per block
(/root/reference/src/pylon/model/layers.py:81-108 attention sizes,
:13-27 feed-forward sizes, :30-40 norm eps, :43-51 rotary constants).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis of ``dim`` elements."""

    kind: str
    dim: int
    eps: float


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.

    ``kind="rope"``: rotate the first ``rotary_dim`` elements of every head by
    ``position * theta**(-2i/rotary_dim)``, pairing element ``i`` with
    ``i + rotary_dim/2``.  ``kind="none"``: positions are not encoded.
    """

    kind: str
    theta: float = 10000.0
    rotary_dim: int = 0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache."""

    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: float
    position: PositionSpec
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    window: Optional[int] = None  # None: every earlier key; w: the last w keys
    kind: str = "attention"

    @property
    def q_size(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.n_kv_heads * self.head_dim


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """``down(act(gate(x)) * up(x))`` with gate and up fused into one matrix."""

    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which mixer, which feed-forward, which norms, how arranged.

    ``arrangement="pre_norm"``: ``x += mixer(norm1(x)); x += ff(norm2(x))``.
    """

    mixer: object
    feed_forward: object
    mixer_norm: NormSpec
    feed_forward_norm: NormSpec
    arrangement: str = "pre_norm"

    @property
    def kind(self) -> str:
        return self.arrangement


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.

    ``layer`` indexes :attr:`ModelSpec.layers`; a layer may be named by several
    entries and then runs again with the same weights.  ``cache`` names the
    cache this run works on: by default its own (the index of the entry in the
    schedule).  An entry whose ``cache`` is an *earlier* entry's index reads
    that entry's keys and values and stores none of its own.
    """

    layer: int
    cache: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    tie_word_embeddings: bool
    max_positions: int
    embedding_scale: float = 1.0
    # Parts between the embedding and the first layer (family "stream": an embedding norm,
    # learned positions, ...) and parts after the vocabulary head (family "logits": a soft
    # cap, a scale, ...), as specs with a ``kind``; the Qwen3 decoder has neither.
    stream_parts: Tuple[object, ...] = ()
    logit_parts: Tuple[object, ...] = ()
    extra: dict = field(default_factory=dict, compare=False, hash=False)

    def resolved_schedule(self) -> Tuple[Tuple[int, int, bool], ...]:
        """``(layer, cache_id, stores)`` per run, with defaults filled in and checked."""
        out = []
        for index, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(
                    f"schedule entry {index} names layer {entry.layer}, "
                    f"but the model has {len(self.layers)} layers"
                )
            cache = index if entry.cache is None else entry.cache
            if cache > index or cache < 0:
                raise ValueError(
                    f"schedule entry {index} reads cache {cache}; a run may only "
                    "read its own cache or that of an earlier run"
                )
            if cache != index and out[cache][1] != cache:
                raise ValueError(
                    f"schedule entry {index} reads cache {cache}, which itself "
                    "borrows another run's cache"
                )
            out.append((entry.layer, cache, cache == index))
        return tuple(out)
