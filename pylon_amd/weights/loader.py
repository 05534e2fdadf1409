"""Reading a model folder's safetensors into a model's parameters, by tensor name.

The reference maps checkpoint names to views of its fused matrices and copies shard by
shard, raising on the first wrong shape and, at the end, on missing names
(/root/reference/src/pylon/model/weights.py:17-49).  Here every problem of the folder
is collected first (missing, unexpected, wrongly shaped tensors) and reported in one
error, and nothing is copied unless the folder is sound.

Element types: a tensor stored in bfloat16 (or float16) is kept in bfloat16 when the
model runs in bfloat16; a tensor stored in 32-bit stays 32-bit; norm weights and other
vectors are always kept in float32; integer tables become int32.  In a float32 model
everything is float32.
"""
from __future__ import annotations

import json
import logging
from pathlib import Path
from typing import Dict, List, Tuple

import torch
from safetensors import safe_open

from ..config.registry import Architecture, WeightTarget

logger = logging.getLogger("pylon")

_FLOAT_STORED = {"F64", "F32", "F16", "BF16"}
_INT_STORED = {"I64", "I32", "I16", "I8", "U8"}


class WeightsError(ValueError):
    """The model folder's tensors do not match what the architecture needs."""

    def __init__(self, missing, unexpected, wrong) -> None:
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong = sorted(wrong)
        lines = ["The model folder's tensors do not match the architecture:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong:
            lines.append(f"  wrong shape or type ({len(self.wrong)}):")
            lines.extend(f"    {item}" for item in self.wrong)
        super().__init__("\n".join(lines))


def shard_files(folder: Path) -> List[Path]:
    """``model.safetensors``, or the shards its index names
    (/root/reference/src/pylon/model/weights.py:41-49)."""
    index = folder / "model.safetensors.index.json"
    if index.is_file():
        names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
        return [folder / name for name in names]
    return [folder / "model.safetensors"]


def _param_dtype(model_dtype: torch.dtype, role: str, stored: List[str]) -> torch.dtype:
    if role == "table":
        return torch.int32
    if role == "vector" or model_dtype == torch.float32:
        return torch.float32
    if any(s in ("F32", "F64") for s in stored):
        return torch.float32  # stored in 32-bit: stays so
    return torch.bfloat16


def _scan(model, arch: Architecture, config, folder: Path, strict: bool):
    """Read the shards' headers and hold them against what the architecture needs.  Returns
    (targets, {tensor name: (file, shape, stored type)}, unexpected names); raises
    :class:`WeightsError` listing every problem if a needed tensor is missing or wrong (with
    ``strict``: also if only unexpected ones are found).  No tensor data is read."""
    targets: Dict[str, WeightTarget] = arch.weight_targets(config)
    params = {path for path, _owner, _name in model.named_params()}
    files = shard_files(folder)
    for path in files:
        if not path.is_file():
            raise FileNotFoundError(f"{path} does not exist")

    found: Dict[str, Tuple[Path, Tuple[int, ...], str]] = {}
    unexpected: List[str] = []
    wrong: List[str] = []
    present = set()
    for path in files:
        with safe_open(str(path), framework="pt", device="cpu") as f:
            for name in f.keys():
                sl = f.get_slice(name)
                shape, stored = tuple(sl.get_shape()), sl.get_dtype()
                target = targets.get(name)
                if target is None:
                    unexpected.append(name)
                    continue
                present.add(name)
                if target.param not in params:
                    wrong.append(f"{name}: the model has no parameter {target.param}")
                    continue
                if shape != tuple(target.shape):
                    wrong.append(f"{name}: expected shape {tuple(target.shape)}, got {shape}")
                    continue
                ok = _INT_STORED if target.role == "table" else _FLOAT_STORED
                if stored not in ok:
                    wrong.append(f"{name}: stored as {stored}, which a {target.role} cannot be")
                    continue
                found[name] = (path, shape, stored)
    missing = [n for n, t in targets.items() if n not in present and not t.optional]
    if missing or wrong or (strict and unexpected):
        raise WeightsError(missing, unexpected, wrong)
    return targets, found, unexpected


def _decide_dtypes(model, targets, found) -> Dict[str, torch.dtype]:
    """Each parameter's element type from what is stored for it."""
    params = {path: (owner, name) for path, owner, name in model.named_params()}
    stored_by_param: Dict[str, List[str]] = {}
    for name, (_path, _shape, stored) in found.items():
        stored_by_param.setdefault(targets[name].param, []).append(stored)
    out = {}
    for param_path, stored in stored_by_param.items():
        owner, pname = params[param_path]
        out[param_path] = _param_dtype(model.dtype, owner.param_roles[pname], stored)
    return out


def stored_param_dtypes(model, arch: Architecture, config, folder) -> Dict[str, torch.dtype]:
    """``{parameter path: the element type it has once the folder is loaded}``, from the
    shards' headers alone; ``model`` may live on the meta device.  What start-up counts the
    weights' bytes with before anything is allocated: a matrix stored in 32-bit stays 32-bit
    in a bfloat16 model and takes twice the bytes."""
    targets, found, _unexpected = _scan(model, arch, config, Path(folder), strict=False)
    return _decide_dtypes(model, targets, found)


def load_weights(model, arch: Architecture, config, folder, *, strict: bool = False) -> List[str]:
    """Fill ``model``'s parameters from ``folder``; raise :class:`WeightsError` listing
    every missing, wrongly shaped and unexpected tensor if a needed tensor is missing or
    wrong (with ``strict``: also if only unexpected ones are found).  Returns the names of
    the tensors that were skipped because the architecture does not know them."""
    folder = Path(folder)
    targets, found, unexpected = _scan(model, arch, config, folder, strict)
    params = {path: (owner, name) for path, owner, name in model.named_params()}
    if unexpected:
        logger.warning("weights_skipped folder=%s count=%d names=%s", folder, len(unexpected),
                       ", ".join(sorted(unexpected)[:8]) + (" ..." if len(unexpected) > 8 else ""))

    kept_wide = []
    for param_path, want in _decide_dtypes(model, targets, found).items():
        owner, pname = params[param_path]
        if owner.params[pname].dtype != want:
            old = owner.params[pname]
            owner.params[pname] = torch.empty(old.shape, dtype=want, device=old.device)
        if want == torch.float32 and model.dtype != torch.float32 and owner.param_roles[pname] == "matrix":
            kept_wide.append(param_path)
    if kept_wide:
        logger.warning(
            "weights_kept_32bit folder=%s count=%d names=%s: matrices stored in 32-bit stay 32-bit in this "
            "%s model; they take twice the memory and their products run on the exact float32 kernel",
            folder, len(kept_wide), ", ".join(sorted(kept_wide)[:4]) + (" ..." if len(kept_wide) > 4 else ""),
            str(model.dtype).replace("torch.", ""))
    filled: Dict[str, int] = {}
    by_file: Dict[Path, List[str]] = {}
    for name, (path, _shape, _stored) in found.items():
        by_file.setdefault(path, []).append(name)
    for path, names in by_file.items():
        with safe_open(str(path), framework="pt", device="cpu") as f:
            for name in names:
                target = targets[name]
                if target.optional and target.param in filled and target.init == "skip":
                    continue  # e.g. the head of a tied model: the embedding is already there
                owner, pname = params[target.param]
                dest = owner.params[pname]
                tensor = f.get_tensor(name)
                if dest.dim() >= 1 and tensor.dim() >= 1 and dest.shape != tensor.shape:
                    dest = dest[target.row_start: target.row_start + tensor.shape[0]]
                dest.copy_(tensor.to(dest.dtype))
                filled[target.param] = filled.get(target.param, 0) + 1
    return sorted(unexpected)
