"""Shared by the tests: the tiny configurations, model folders made in temporary
folders, and reading a folder's tensors for the plain implementation."""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict

import numpy as np


def _qwen3(**sizes) -> dict:
    base = {
        "architectures": ["Qwen3ForCausalLM"],
        "model_type": "qwen3",
        "hidden_act": "silu",
        "attention_bias": False,
        "rope_scaling": None,
        "use_sliding_window": False,
        "sliding_window": None,
        "initializer_range": 0.02,
    }
    base.update(sizes)
    return base


# Two tiny configurations that differ in every size and option, plus a third with a head
# size that is no power of two and room for long sequences.
TINY_A = _qwen3(
    num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
    intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
    tie_word_embeddings=True, max_position_embeddings=128,
)
TINY_B = _qwen3(
    num_hidden_layers=3, hidden_size=96, num_attention_heads=6, num_key_value_heads=1, head_dim=32,
    intermediate_size=320, vocab_size=384, rope_theta=1000000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=False, max_position_embeddings=256,
)
TINY_C = _qwen3(
    num_hidden_layers=2, hidden_size=80, num_attention_heads=5, num_key_value_heads=5, head_dim=48,
    intermediate_size=176, vocab_size=301, rope_theta=500000.0, rms_norm_eps=3e-6,
    tie_word_embeddings=False, max_position_embeddings=2048,
)
# D has a head size that the matrix-core attention kernels take (A, B and C run on the
# general kernel), three query heads per key/value head, and room for contexts long enough
# that a request's keys are shared between workgroups.
TINY_D = _qwen3(
    num_hidden_layers=2, hidden_size=112, num_attention_heads=6, num_key_value_heads=2, head_dim=64,
    intermediate_size=208, vocab_size=331, rope_theta=250000.0, rms_norm_eps=2e-6,
    tie_word_embeddings=True, max_position_embeddings=4096,
)
# E has the head size of every published Qwen3 model, 128: with pages of 64 tokens its prompt
# portions run on the attention kernel that loads whole blocks of a page straight into LDS.
TINY_E = _qwen3(
    num_hidden_layers=2, hidden_size=72, num_attention_heads=3, num_key_value_heads=1, head_dim=128,
    intermediate_size=144, vocab_size=277, rope_theta=1000000.0, rms_norm_eps=1e-5,
    tie_word_embeddings=False, max_position_embeddings=1024,
)
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E}
# A has unit norm weights; the others draw them, so that a kernel ignoring a norm weight fails.
NORM_JITTER = {"A": 0.0, "B": 0.2, "C": 0.2, "D": 0.2, "E": 0.2}
SEEDS = {"A": 11, "B": 23, "C": 37, "D": 41, "E": 53}


def make_model_folder(tmp: Path, name: str, *, dtype: str = "float32", config=None, seed=None,
                      norm_jitter=None, std=None) -> Path:
    from pylon_amd.weights import write_random_model

    folder = Path(tmp) / f"model_{name}_{dtype}"
    write_random_model(
        folder, config or CONFIGS[name], SEEDS.get(name, 1) if seed is None else seed, dtype=dtype,
        norm_jitter=NORM_JITTER.get(name, 0.1) if norm_jitter is None else norm_jitter, std=std,
    )
    return folder


def read_folder(folder: Path):
    """(config dict, {tensor name: float64 array}) of a model folder, for the plain model."""
    import torch
    from safetensors.torch import load_file

    cfg = json.loads((Path(folder) / "config.json").read_text())
    tensors = load_file(str(Path(folder) / "model.safetensors"))
    weights: Dict[str, np.ndarray] = {
        name: t.to(torch.float64).numpy() for name, t in tensors.items()
    }
    return cfg, weights


def random_tokens(vocab: int, count: int, seed: int):
    return np.random.default_rng(seed).integers(0, vocab, count).tolist()


def rows_within(got, ref, bound: float):
    """Every row of ``got`` is within ``bound`` times that row's own largest |reference logit|
    of ``ref`` (a bad row cannot hide under another row's large logit).  Returns
    (ok, index of the worst row, its error as a fraction of its scale)."""
    got, ref = np.asarray(got), np.asarray(ref)
    if got.ndim == 1:
        got, ref = got[None], ref[None]
    assert got.shape == ref.shape, (got.shape, ref.shape)
    frac = np.abs(got - ref).max(axis=1) / np.abs(ref).max(axis=1)
    worst = int(frac.argmax())
    return bool(frac[worst] <= bound), worst, float(frac[worst])
