"""Serving options, with the reference's names, defaults and checks where it has them
(/root/reference/src/pylon/config.py:8-75; environment names :87-112).

Options of the reference that belong to parts this engine does not have (prefix
cache, speculation, torch.compile, hub download) are not carried.  ``cuda_graphs``
keeps its name: on this hardware it switches HIP graph replay of decode-only steps.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass
from typing import Optional


@dataclass(frozen=True)
class PylonConfig:
    model_path: Optional[str] = None
    dtype: str = "bfloat16"
    max_gpu_utilization: float = 0.90
    weight_headroom_ratio: float = 0.20
    kv_cache_headroom_ratio: float = 0.20
    prefill_chunk_size: int = 2048
    max_batch_size: int = 32
    max_queue_size: int = 32
    batch_wait_ms: float = 2.0
    cuda_graphs: bool = False
    admit_skip: int = 4
    page_size: int = 256
    # Queue the next step before the host has read the tokens of the running one (they are
    # fed back on the device); stop tokens are then noticed one step late.
    run_ahead: bool = True
    # Explicit pool size in pages; None sizes the pool from free device memory.
    num_pages: Optional[int] = None

    def __post_init__(self) -> None:
        if self.dtype not in ("bfloat16", "float32"):
            raise ValueError("dtype must be bfloat16 or float32.")
        if not math.isfinite(self.max_gpu_utilization) or not 0 < self.max_gpu_utilization <= 1:
            raise ValueError("max_gpu_utilization must be greater than 0 and at most 1.")
        for name in ("weight_headroom_ratio", "kv_cache_headroom_ratio"):
            if not 0 <= getattr(self, name) < 1:
                raise ValueError(f"{name} must be at least 0 and less than 1.")
        for name in ("prefill_chunk_size", "page_size"):
            value = getattr(self, name)
            if not isinstance(value, int) or isinstance(value, bool) or value < 1:
                raise ValueError(f"{name} must be a positive integer.")
        if self.page_size % 16:
            raise ValueError("page_size must be a multiple of 16.")
        if self.max_batch_size < 1:
            raise ValueError("max_batch_size must be at least 1.")
        if self.max_queue_size < 1:
            raise ValueError("max_queue_size must be at least 1.")
        if not math.isfinite(self.batch_wait_ms) or self.batch_wait_ms < 0:
            raise ValueError("batch_wait_ms must be finite and non-negative.")
        if isinstance(self.admit_skip, bool) or not isinstance(self.admit_skip, int) or self.admit_skip < 0:
            raise ValueError("admit_skip must be an integer of at least 0.")
        if self.num_pages is not None and self.num_pages < 1:
            raise ValueError("num_pages must be at least 1.")


def _env_bool(name: str, default: bool) -> bool:
    value = os.getenv(name, str(default)).strip().lower()
    if value in {"1", "true"}:
        return True
    if value in {"0", "false"}:
        return False
    raise ValueError(f"{name} must be true, false, 1, or 0.")


def get_config(**overrides) -> PylonConfig:
    """Options from ``PYLON_*`` environment variables; keyword arguments win."""
    num_pages = os.getenv("PYLON_NUM_PAGES")
    values = dict(
        model_path=os.getenv("PYLON_MODEL_PATH") or None,
        dtype=os.getenv("PYLON_DTYPE", "bfloat16"),
        max_gpu_utilization=float(os.getenv("PYLON_MAX_GPU_UTILIZATION", "0.90")),
        weight_headroom_ratio=float(os.getenv("PYLON_WEIGHT_HEADROOM_RATIO", "0.20")),
        kv_cache_headroom_ratio=float(os.getenv("PYLON_KV_CACHE_HEADROOM_RATIO", "0.20")),
        prefill_chunk_size=int(os.getenv("PYLON_PREFILL_CHUNK_SIZE", "2048")),
        max_batch_size=int(os.getenv("PYLON_MAX_BATCH_SIZE", "32")),
        max_queue_size=int(os.getenv("PYLON_MAX_QUEUE_SIZE", "32")),
        batch_wait_ms=float(os.getenv("PYLON_BATCH_WAIT_MS", "2")),
        cuda_graphs=_env_bool("PYLON_CUDA_GRAPHS", False),
        admit_skip=int(os.getenv("PYLON_ADMIT_SKIP", "4")),
        run_ahead=_env_bool("PYLON_RUN_AHEAD", True),
        page_size=int(os.getenv("PYLON_PAGE_SIZE", "256")),
        num_pages=int(num_pages) if num_pages else None,
    )
    values.update({k: v for k, v in overrides.items() if v is not None})
    return PylonConfig(**values)
