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


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    gen = torch.Generator(device=device)
    gen.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return gen


_SLAB = 1 << 26  # elements drawn at a time, so that no float32 copy of a large matrix is needed


def draw_tensor(seed: int, name: str, target, sigma: float, norm_jitter: float, *, out: torch.Tensor,
                draw_on=None) -> None:
    """The one rule of the random-weights mode: fill ``out`` (of the target's shape, on any
    device, of any float type) with tensor ``name`` of seed ``seed``.  ``normal``:
    N(0, sigma^2); ``ones`` / ``ones_jitter``: 1, or 1 + norm_jitter * N(0, 1).  The numbers
    come from a generator keyed by (seed, name) on the device ``draw_on`` (default: where
    ``out`` lives): drawn on the CPU they are the numbers of the folder that
    :func:`write_random_model` writes; drawn on a GPU they follow the same rule with other
    numbers, a few hundred times faster."""
    if tuple(out.shape) != tuple(target.shape):
        raise ValueError(f"{name}: expected a tensor of shape {tuple(target.shape)}, got {tuple(out.shape)}")
    if target.init in ("ones", "ones_jitter") and not (target.init == "ones_jitter" and norm_jitter):
        out.fill_(1.0)
        return
    if target.init not in ("normal", "ones_jitter"):
        raise ValueError(f"unknown init rule {target.init!r} for {name}")
    where = torch.device(draw_on) if draw_on is not None else out.device
    gen = _generator(seed, name, where)
    scale, shift = (sigma, 0.0) if target.init == "normal" else (norm_jitter, 1.0)
    if out.is_contiguous():
        flat = out.view(-1)
        for start in range(0, flat.numel(), _SLAB):
            part = flat[start: start + _SLAB]
            part.copy_(torch.randn(part.numel(), generator=gen, dtype=torch.float32, device=where)
                       * scale + shift)
    else:
        out.copy_(torch.randn(tuple(out.shape), generator=gen, dtype=torch.float32, device=where)
                  * scale + shift)


def _sigma(cfg, std: Optional[float]) -> float:
    return float(std if std is not None else getattr(cfg, "initializer_range", 0.02))


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
    sigma = _sigma(cfg, std)
    tensors = {}
    for name, target in arch.weight_targets(cfg).items():
        if target.init == "skip":
            continue
        value = torch.empty(target.shape, dtype=torch.float32)
        draw_tensor(seed, name, target, sigma, norm_jitter, out=value)
        tensors[name] = value.to(store).contiguous()
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(arch.config_to_json(cfg), indent=2) + "\n")
    save_file(tensors, str(folder / "model.safetensors"))
    return folder


def fill_random_model(model, arch, cfg, seed: int, *, std: Optional[float] = None,
                      norm_jitter: float = 0.0, draw_on=None) -> None:
    """The same mode without the folder: fill ``model``'s parameters in place, tensor by
    tensor through the architecture's table of checkpoint names (so fused matrices get their
    parts in their row ranges, as a load would put them).  ``draw_on``: the device whose
    generator draws (default: the parameters' own; ``"cpu"`` gives the folder's numbers).
    Every parameter must be covered."""
    params = {path: (owner, name) for path, owner, name in model.named_params()}
    sigma = _sigma(cfg, std)
    covered = {path: 0 for path in params}
    for name, target in arch.weight_targets(cfg).items():
        if target.init == "skip":
            continue
        if target.param not in params:
            raise ValueError(f"{name}: the model has no parameter {target.param}")
        owner, pname = params[target.param]
        dest = owner.params[pname]
        if dest.dim() >= 1 and len(target.shape) >= 1 and tuple(dest.shape) != tuple(target.shape):
            dest = dest[target.row_start: target.row_start + target.shape[0]]
        draw_tensor(seed, name, target, sigma, norm_jitter, out=dest, draw_on=draw_on)
        covered[target.param] += dest.numel()
    short = [path for path, (owner, pname) in params.items() if covered[path] != owner.params[pname].numel()]
    if short:
        raise ValueError("the architecture's table of tensors does not cover: " + ", ".join(sorted(short)))
