"""Serving options, with the reference's names, defaults and ranges where it has them
(/root/reference/src/pylon/config.py:8-75; environment names :87-112).

Options of the reference that belong to parts this engine does not have (prefix
cache, speculation, torch.compile, hub download) are not carried.  ``cuda_graphs``
keeps its name: on this hardware it switches HIP graph replay of decode-only steps.

Every option is one row of :data:`OPTIONS`: its name, its default, how its text form is
read, and the range it must lie in.  The dataclass, its checks and the reading of the
``PYLON_*`` environment variables are all driven by that table.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass, fields
from typing import Any, Callable, NamedTuple, Optional


def _flag(text: str) -> bool:
    word = text.strip().lower()
    if word in ("1", "true"):
        return True
    if word in ("0", "false"):
        return False
    raise ValueError("expected true, false, 1 or 0")


def _optional_int(text: str) -> Optional[int]:
    return int(text) if text.strip() else None


def _optional_text(text: str) -> Optional[str]:
    return text or None


class Option(NamedTuple):
    name: str
    default: Any
    read: Callable[[str], Any]  # from the text of an environment variable
    accepts: Callable[[Any], bool]  # the range of valid values
    rule: str  # the range in words, for the error

    @property
    def variable(self) -> str:
        return "PYLON_" + self.name.upper()


def _whole(value: Any) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


def _real(value: Any) -> bool:
    return isinstance(value, (int, float)) and not isinstance(value, bool) and math.isfinite(value)


OPTIONS = (
    Option("model_path", None, _optional_text, lambda v: v is None or isinstance(v, (str, os.PathLike)),
           "a folder path"),
    Option("dtype", "bfloat16", str, lambda v: v in ("bfloat16", "float32"), "bfloat16 or float32"),
    Option("max_gpu_utilization", 0.90, float, lambda v: _real(v) and 0 < v <= 1, "above 0 and at most 1"),
    Option("weight_headroom_ratio", 0.20, float, lambda v: _real(v) and 0 <= v < 1, "from 0 to below 1"),
    Option("kv_cache_headroom_ratio", 0.20, float, lambda v: _real(v) and 0 <= v < 1, "from 0 to below 1"),
    Option("prefill_chunk_size", 2048, int, lambda v: _whole(v) and v >= 1, "a whole number of at least 1"),
    Option("max_batch_size", 32, int, lambda v: _whole(v) and v >= 1, "a whole number of at least 1"),
    Option("max_queue_size", 32, int, lambda v: _whole(v) and v >= 1, "a whole number of at least 1"),
    Option("batch_wait_ms", 2.0, float, lambda v: _real(v) and v >= 0, "a finite number of at least 0"),
    Option("cuda_graphs", False, _flag, lambda v: isinstance(v, bool), "true or false"),
    # Start-up captures the decode graphs of requests of up to this many tokens (unset: of the
    # longest request the model and the pool allow); graphs of longer ones at their first use.
    Option("cuda_graph_max_tokens", None, _optional_int, lambda v: v is None or (_whole(v) and v >= 1),
           "a whole number of at least 1, or unset"),
    Option("admit_skip", 4, int, lambda v: _whole(v) and v >= 0, "a whole number of at least 0"),
    Option("page_size", 256, int, lambda v: _whole(v) and v >= 16 and v % 16 == 0, "a positive multiple of 16"),
    # Queue the next step before the host has read the tokens of the running one (they are
    # fed back on the device); stop tokens are then noticed one step late.
    Option("run_ahead", True, _flag, lambda v: isinstance(v, bool), "true or false"),
    # Explicit pool size in pages; None sizes the pool from free device memory.
    Option("num_pages", None, _optional_int, lambda v: v is None or (_whole(v) and v >= 1),
           "a whole number of at least 1, or unset"),
)
_BY_NAME = {option.name: option for option in OPTIONS}


@dataclass(frozen=True)
class PylonConfig:
    model_path: Optional[str] = _BY_NAME["model_path"].default
    dtype: str = _BY_NAME["dtype"].default
    max_gpu_utilization: float = _BY_NAME["max_gpu_utilization"].default
    weight_headroom_ratio: float = _BY_NAME["weight_headroom_ratio"].default
    kv_cache_headroom_ratio: float = _BY_NAME["kv_cache_headroom_ratio"].default
    prefill_chunk_size: int = _BY_NAME["prefill_chunk_size"].default
    max_batch_size: int = _BY_NAME["max_batch_size"].default
    max_queue_size: int = _BY_NAME["max_queue_size"].default
    batch_wait_ms: float = _BY_NAME["batch_wait_ms"].default
    cuda_graphs: bool = _BY_NAME["cuda_graphs"].default
    cuda_graph_max_tokens: Optional[int] = _BY_NAME["cuda_graph_max_tokens"].default
    admit_skip: int = _BY_NAME["admit_skip"].default
    page_size: int = _BY_NAME["page_size"].default
    run_ahead: bool = _BY_NAME["run_ahead"].default
    num_pages: Optional[int] = _BY_NAME["num_pages"].default

    def __post_init__(self) -> None:
        for option in OPTIONS:
            value = getattr(self, option.name)
            if not option.accepts(value):
                raise ValueError(f"{option.name} = {value!r} is not allowed: it must be {option.rule}.")


assert [f.name for f in fields(PylonConfig)] == [o.name for o in OPTIONS]


def get_config(**overrides) -> PylonConfig:
    """Options from the ``PYLON_*`` environment variables (``PYLON_`` + the option's name in
    capitals); keyword arguments that are not None win over the environment."""
    values = {}
    for option in OPTIONS:
        given = overrides.get(option.name)
        if given is not None:
            values[option.name] = given
            continue
        text = os.environ.get(option.variable)
        if text is None:
            continue
        try:
            values[option.name] = option.read(text)
        except ValueError as error:
            raise ValueError(f"{option.variable} = {text!r} cannot be read: {error}") from None
    unknown = set(overrides) - set(_BY_NAME)
    if unknown:
        raise TypeError(f"unknown option(s): {', '.join(sorted(unknown))}")
    return PylonConfig(**values)
