from .engine_config import PylonConfig, get_config
from .registry import (
    Architecture,
    WeightTarget,
    architecture_name,
    load_model_config,
    read_config_json,
    read_stop_token_ids,
    register_architecture,
    registered_architectures,
    resolve,
    unregister_architecture,
)
from .specs import (
    AttentionSpec,
    GatedFeedForwardSpec,
    LayerSpec,
    ModelSpec,
    NormSpec,
    PositionSpec,
    ScheduleEntry,
)

__all__ = [
    "PylonConfig",
    "get_config",
    "Architecture",
    "WeightTarget",
    "architecture_name",
    "load_model_config",
    "read_config_json",
    "read_stop_token_ids",
    "register_architecture",
    "registered_architectures",
    "resolve",
    "unregister_architecture",
    "AttentionSpec",
    "GatedFeedForwardSpec",
    "LayerSpec",
    "ModelSpec",
    "NormSpec",
    "PositionSpec",
    "ScheduleEntry",
]
