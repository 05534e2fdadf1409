"""Qwen3 dense: config.json keys, the model as specs, and checkpoint tensor names.

Keys and their meaning follow /root/reference/src/pylon/model/config.py:35-62; the
reference additionally pins every size to one checkpoint (:9-17), which this
engine does not.  Tensor names and the row ranges of the fused matrices follow
/root/reference/src/pylon/model/weights.py:52-83.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, Mapping, Optional, Tuple

from ..config.registry import Architecture, WeightTarget, register_architecture
from ..config.specs import (
    AttentionSpec,
    GatedFeedForwardSpec,
    LayerSpec,
    ModelSpec,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
)

ARCHITECTURE = "Qwen3ForCausalLM"


def _unsupported(field: str) -> ValueError:
    # Message shape of /root/reference/src/pylon/model/config.py:65-67.
    return ValueError(f"Checkpoint config field {field} is not supported.")


@dataclass(frozen=True)
class Qwen3Config:
    """The eleven values config.json gives (no defaults: a missing key is an error)."""

    vocab_size: int
    max_position_embeddings: int
    hidden_size: int
    num_attention_heads: int
    num_hidden_layers: int
    intermediate_size: int
    head_dim: int
    num_key_value_heads: int
    rope_theta: float
    rms_norm_eps: float
    tie_word_embeddings: bool
    initializer_range: float = 0.02  # only used to draw random weights
    eos_token_id: Optional[Tuple[int, ...]] = None

    def __post_init__(self) -> None:
        for name in (
            "vocab_size",
            "max_position_embeddings",
            "hidden_size",
            "num_attention_heads",
            "num_hidden_layers",
            "intermediate_size",
            "head_dim",
            "num_key_value_heads",
        ):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        if self.num_attention_heads % self.num_key_value_heads:
            # /root/reference/src/pylon/model/layers.py:84-87
            raise ValueError(
                "The number of Q heads must be divisible by the number of KV heads."
            )
        if self.head_dim % 2:
            # /root/reference/src/pylon/model/layers.py:75-76
            raise ValueError("Qwen3 RoPE requires an even head dimension.")
        if not (self.rope_theta > 0 and math.isfinite(self.rope_theta)):
            raise ValueError("rope_theta must be positive and finite")
        if not (self.rms_norm_eps > 0 and math.isfinite(self.rms_norm_eps)):
            raise ValueError("rms_norm_eps must be positive and finite")


_REQUIRED = (
    "vocab_size",
    "max_position_embeddings",
    "hidden_size",
    "num_attention_heads",
    "num_hidden_layers",
    "intermediate_size",
    "head_dim",
    "num_key_value_heads",
    "rope_theta",
    "rms_norm_eps",
    "tie_word_embeddings",
)


def parse_config(data: Mapping) -> Qwen3Config:
    if data.get("model_type") != "qwen3":
        raise _unsupported("model_type")
    if data.get("hidden_act") != "silu":
        raise _unsupported("hidden_act")
    if data.get("attention_bias", False) is not False:
        raise _unsupported("attention_bias")
    if data.get("rope_scaling") is not None:
        raise _unsupported("rope_scaling")
    if data.get("use_sliding_window", False) is not False:
        raise _unsupported("use_sliding_window")
    if data.get("sliding_window") is not None:
        raise _unsupported("sliding_window")
    missing = [key for key in _REQUIRED if key not in data]
    if missing:
        raise ValueError("config.json lacks required keys: " + ", ".join(missing))
    if not isinstance(data["tie_word_embeddings"], bool):
        raise _unsupported("tie_word_embeddings")
    eos = data.get("eos_token_id")
    if isinstance(eos, int):
        eos = (eos,)
    elif eos is not None:
        eos = tuple(int(v) for v in eos)
    return Qwen3Config(
        vocab_size=data["vocab_size"],
        max_position_embeddings=data["max_position_embeddings"],
        hidden_size=data["hidden_size"],
        num_attention_heads=data["num_attention_heads"],
        num_hidden_layers=data["num_hidden_layers"],
        intermediate_size=data["intermediate_size"],
        head_dim=data["head_dim"],
        num_key_value_heads=data["num_key_value_heads"],
        rope_theta=float(data["rope_theta"]),
        rms_norm_eps=float(data["rms_norm_eps"]),
        tie_word_embeddings=data["tie_word_embeddings"],
        initializer_range=float(data.get("initializer_range", 0.02)),
        eos_token_id=eos,
    )


def config_to_json(cfg: Qwen3Config) -> dict:
    out = {
        "architectures": [ARCHITECTURE],
        "model_type": "qwen3",
        "hidden_act": "silu",
        "attention_bias": False,
        "rope_scaling": None,
        "use_sliding_window": False,
        "sliding_window": None,
        "vocab_size": cfg.vocab_size,
        "max_position_embeddings": cfg.max_position_embeddings,
        "hidden_size": cfg.hidden_size,
        "num_attention_heads": cfg.num_attention_heads,
        "num_hidden_layers": cfg.num_hidden_layers,
        "intermediate_size": cfg.intermediate_size,
        "head_dim": cfg.head_dim,
        "num_key_value_heads": cfg.num_key_value_heads,
        "rope_theta": cfg.rope_theta,
        "rms_norm_eps": cfg.rms_norm_eps,
        "tie_word_embeddings": cfg.tie_word_embeddings,
        "initializer_range": cfg.initializer_range,
    }
    if cfg.eos_token_id is not None:
        out["eos_token_id"] = list(cfg.eos_token_id)
    return out


def model_spec(cfg: Qwen3Config) -> ModelSpec:
    """Every layer is the same block: full-attention GQA with per-head q/k RMSNorm and
    rotary positions, then a SiLU-gated feed-forward, both pre-normed
    (/root/reference/src/pylon/model/layers.py:168-200; model.py:25-28)."""
    position = PositionSpec(
        kind="rope",
        theta=cfg.rope_theta,
        rotary_dim=cfg.head_dim,
        max_positions=cfg.max_position_embeddings,
    )
    attention = AttentionSpec(
        hidden_size=cfg.hidden_size,
        n_heads=cfg.num_attention_heads,
        n_kv_heads=cfg.num_key_value_heads,
        head_dim=cfg.head_dim,
        # No scale is passed anywhere in the reference, so the library default
        # 1/sqrt(head_dim) applies (/root/reference/src/pylon/kv/cache.py:462-475).
        scale=1.0 / math.sqrt(cfg.head_dim),
        position=position,
        qk_norm=True,
        qk_norm_eps=cfg.rms_norm_eps,
        window=None,
    )
    feed_forward = GatedFeedForwardSpec(
        hidden_size=cfg.hidden_size,
        intermediate_size=cfg.intermediate_size,
        activation="silu",
    )
    norm = NormSpec(kind="rmsnorm", dim=cfg.hidden_size, eps=cfg.rms_norm_eps)
    layer = LayerSpec(
        mixer=attention,
        feed_forward=feed_forward,
        mixer_norm=norm,
        feed_forward_norm=norm,
        arrangement="pre_norm",
    )
    count = cfg.num_hidden_layers
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        layers=tuple(layer for _ in range(count)),
        schedule=tuple(ScheduleEntry(layer=i) for i in range(count)),
        final_norm=norm,
        tie_word_embeddings=cfg.tie_word_embeddings,
        max_positions=cfg.max_position_embeddings,
    )


def weight_targets(cfg: Qwen3Config) -> Dict[str, WeightTarget]:
    hidden, inter, hd = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    q = cfg.num_attention_heads * hd
    kv = cfg.num_key_value_heads * hd
    targets: Dict[str, WeightTarget] = {
        "model.embed_tokens.weight": WeightTarget("embed", (cfg.vocab_size, hidden)),
        "model.norm.weight": WeightTarget(
            "final_norm.weight", (hidden,), role="vector", init="ones_jitter"
        ),
    }
    if cfg.tie_word_embeddings:
        # A tied checkpoint may still carry the head; it is the embedding again.
        targets["lm_head.weight"] = WeightTarget(
            "embed", (cfg.vocab_size, hidden), optional=True, init="skip"
        )
    else:
        targets["lm_head.weight"] = WeightTarget("lm_head", (cfg.vocab_size, hidden))
    for i in range(cfg.num_hidden_layers):
        src = f"model.layers.{i}"
        dst = f"layers.{i}"
        vec = dict(role="vector", init="ones_jitter")
        targets.update(
            {
                # q, k, v fill consecutive row ranges of one matrix, in that order.
                f"{src}.self_attn.q_proj.weight": WeightTarget(f"{dst}.mixer.qkv", (q, hidden), 0),
                f"{src}.self_attn.k_proj.weight": WeightTarget(f"{dst}.mixer.qkv", (kv, hidden), q),
                f"{src}.self_attn.v_proj.weight": WeightTarget(
                    f"{dst}.mixer.qkv", (kv, hidden), q + kv
                ),
                f"{src}.self_attn.o_proj.weight": WeightTarget(f"{dst}.mixer.out", (hidden, q)),
                f"{src}.self_attn.q_norm.weight": WeightTarget(f"{dst}.mixer.q_norm", (hd,), **vec),
                f"{src}.self_attn.k_norm.weight": WeightTarget(f"{dst}.mixer.k_norm", (hd,), **vec),
                f"{src}.input_layernorm.weight": WeightTarget(
                    f"{dst}.mixer_norm.weight", (hidden,), **vec
                ),
                # gate rows first, then up rows.
                f"{src}.mlp.gate_proj.weight": WeightTarget(
                    f"{dst}.feed_forward.gate_up", (inter, hidden), 0
                ),
                f"{src}.mlp.up_proj.weight": WeightTarget(
                    f"{dst}.feed_forward.gate_up", (inter, hidden), inter
                ),
                f"{src}.mlp.down_proj.weight": WeightTarget(
                    f"{dst}.feed_forward.down", (hidden, inter)
                ),
                f"{src}.post_attention_layernorm.weight": WeightTarget(
                    f"{dst}.feed_forward_norm.weight", (hidden,), **vec
                ),
            }
        )
    return targets


QWEN3 = register_architecture(
    Architecture(
        name=ARCHITECTURE,
        parse_config=parse_config,
        model_spec=model_spec,
        weight_targets=weight_targets,
        config_to_json=config_to_json,
    ),
    replace=True,
)
