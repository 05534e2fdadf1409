"""Random-weights mode: write a model folder (config.json, model.safetensors) from a
configuration and a seed.

The reference has no such mode; its tests build a model under ``torch.manual_seed``
(/root/reference/tests/test_paged_attention.py:148-149).  Every tensor is drawn from a
generator keyed by the seed and the tensor's name, so the same (config, seed) always
gives the same folder whatever order tensors are written in.
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Mapping, Optional

import torch
from safetensors.torch import save_file

from ..config.registry import resolve


def _generator(seed: int, name: str) -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return gen


def write_random_model(folder, config: Mapping, seed: int, *, dtype: str = "bfloat16",
                       std: Optional[float] = None, norm_jitter: float = 0.0) -> Path:
    """Write ``config.json`` and ``model.safetensors`` into ``folder``.

    ``config`` is the content of config.json (a dict naming its architecture).  Matrices
    are N(0, std^2) with ``std`` = the config's ``initializer_range`` unless given; norm
    weights are 1, or ``1 + norm_jitter * N(0, 1)`` so that a kernel ignoring them shows.
    ``dtype`` is the stored element type: ``bfloat16`` or ``float32``.
    """
    if dtype not in ("bfloat16", "float32"):
        raise ValueError("dtype must be bfloat16 or float32")
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    arch = resolve(config)
    cfg = arch.parse_config(config)
    sigma = float(std if std is not None else getattr(cfg, "initializer_range", 0.02))
    tensors = {}
    for name, target in arch.weight_targets(cfg).items():
        if target.init == "skip":
            continue
        gen = _generator(seed, name)
        if target.init == "normal":
            value = torch.randn(target.shape, generator=gen, dtype=torch.float32) * sigma
        elif target.init in ("ones", "ones_jitter"):
            value = torch.ones(target.shape, dtype=torch.float32)
            if target.init == "ones_jitter" and norm_jitter:
                value += norm_jitter * torch.randn(target.shape, generator=gen, dtype=torch.float32)
        else:
            raise ValueError(f"unknown init rule {target.init!r} for {name}")
        tensors[name] = value.to(store).contiguous()
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(arch.config_to_json(cfg), indent=2) + "\n")
    save_file(tensors, str(folder / "model.safetensors"))
    return folder
