"""The one registry from an architecture's name to its definition.

The reference compares ``architectures`` with a single hard-coded name
(/root/reference/src/pylon/model/config.py:40); here the name found in
config.json selects an :class:`Architecture`, and everything downstream
(loader, model builder, replay, engine) goes through :func:`resolve`.
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Dict, Mapping, Tuple

from .specs import ModelSpec


@dataclass(frozen=True)
class WeightTarget:
    """Where a checkpoint tensor lands: a model parameter, or a row range of one."""

    param: str
    shape: Tuple[int, ...]  # shape of the checkpoint tensor
    row_start: int = 0  # first row of ``param`` it fills
    role: str = "matrix"  # "matrix", "vector" (kept fp32) or "table" (integers)
    optional: bool = False
    init: str = "normal"  # random mode: "normal", "ones", "ones_jitter"


@dataclass(frozen=True)
class Architecture:
    """What the framework needs to know about one model family."""

    name: str
    parse_config: Callable[[Mapping], object]
    model_spec: Callable[[object], ModelSpec]
    weight_targets: Callable[[object], Dict[str, WeightTarget]]
    config_to_json: Callable[[object], dict]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def architecture_name(config: Mapping) -> str:
    names = config.get("architectures")
    if not isinstance(names, (list, tuple)) or len(names) != 1 or not isinstance(names[0], str):
        raise ValueError(
            "config.json must name exactly one architecture in 'architectures'; "
            f"found {names!r}"
        )
    return names[0]


def resolve(config: Mapping) -> Architecture:
    """The architecture that ``config`` (a parsed config.json) asks for."""
    # Built-in families register themselves on import.
    from .. import models  # noqa: F401

    name = architecture_name(config)
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        known = ", ".join(registered_architectures()) or "none"
        raise ValueError(
            f"Unknown architecture {name!r}; registered: {known}."
        ) from None


def read_config_json(folder) -> dict:
    path = Path(folder) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"{path} does not exist")
    return json.loads(path.read_text())


def load_model_config(folder):
    """``(architecture, typed config)`` for the model folder ``folder``."""
    raw = read_config_json(folder)
    arch = resolve(raw)
    return arch, arch.parse_config(raw)


def read_stop_token_ids(folder) -> tuple:
    """The ids that end a generation: ``eos_token_id`` (a number or a list) of the folder's
    ``generation_config.json`` if there is one, else of its ``config.json``; none if neither
    names any (/root/reference/src/pylon/model/tokenizer.py:24-38, which insists on one)."""
    folder = Path(folder)
    for name in ("generation_config.json", "config.json"):
        path = folder / name
        if not path.is_file():
            continue
        eos = json.loads(path.read_text()).get("eos_token_id")
        if eos is None:
            continue
        return (int(eos),) if isinstance(eos, int) else tuple(int(token_id) for token_id in eos)
    return ()
