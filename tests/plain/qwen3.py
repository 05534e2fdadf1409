"""A plain, slow implementation of the Qwen3 dense decoder: whole sequences, no cache,
numpy float64, one function per part.  Written from the reference's formulas (each
function cites them); shares no code with ``pylon_amd``.  It is the oracle of the tests.

Weights come as a dict from checkpoint tensor name to array; the configuration is the
raw content of config.json.
"""
from __future__ import annotations

import math
from typing import Mapping, Optional, Sequence

import numpy as np

F = np.float64


def rms_norm(x: np.ndarray, weight: np.ndarray, eps: float) -> np.ndarray:
    """/root/reference/src/pylon/model/layers.py:36-40 — ``F.rms_norm(x.float(), (dim,),
    scale, eps)``: x / sqrt(mean(x^2) + eps) * scale over the last axis; no mean
    subtraction, the weight multiplies as it is (not 1 + w)."""
    x = np.asarray(x, dtype=F)
    mean_square = np.mean(x * x, axis=-1, keepdims=True)
    return x / np.sqrt(mean_square + eps) * np.asarray(weight, dtype=F)


def rope_tables(positions: Sequence[int], head_dim: int, theta: float):
    """/root/reference/src/pylon/model/layers.py:43-51 — inverse frequencies
    1 / theta**(arange(0, d, 2)/d) and angles position * frequency, both formed in
    float32 as the reference forms them; the table is the angles twice side by side."""
    exponents = np.arange(0, head_dim, 2, dtype=np.float32) / np.float32(head_dim)
    inverse = (np.float32(1.0) / np.power(np.float32(theta), exponents, dtype=np.float32)).astype(np.float32)
    pos = np.asarray(positions, dtype=np.float32)
    angles = (pos[:, None] * inverse[None, :]).astype(np.float32)
    angles = np.concatenate([angles, angles], axis=1).astype(F)
    return np.cos(angles), np.sin(angles)


def apply_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """/root/reference/src/pylon/model/layers.py:73-78 — x*cos + cat(-second, first)*sin
    where first/second are the halves of the last axis.  x: [heads, tokens, d];
    cos, sin: [tokens, d]."""
    half = x.shape[-1] // 2
    first, second = x[..., :half], x[..., half:]
    rotated = np.concatenate([-second, first], axis=-1)
    return x * cos[None, :, :] + rotated * sin[None, :, :]


def softmax(x: np.ndarray, axis: int = -1) -> np.ndarray:
    x = x - np.max(x, axis=axis, keepdims=True)
    e = np.exp(x)
    return e / np.sum(e, axis=axis, keepdims=True)


def causal_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float,
                     window: Optional[int] = None) -> np.ndarray:
    """/root/reference/src/pylon/kv/cache.py:341-365 (the reference's own CPU oracle):
    keys and values of a KV head are repeated for the query heads of its group
    (``repeat_interleave``, so query head h reads KV head h // group), the mask lets query
    i see key j iff j <= i, and scaled-dot-product attention uses the default scale
    1/sqrt(d) — passed in here as ``scale``.  ``window`` (not in the reference) further
    hides keys with j <= i - window.  q: [heads, T, d]; k, v: [kv_heads, T, d]."""
    heads, tokens, _ = q.shape
    group = heads // k.shape[0]
    k = np.repeat(k, group, axis=0)
    v = np.repeat(v, group, axis=0)
    scores = (q @ k.transpose(0, 2, 1)) * scale  # [heads, T, T]
    i = np.arange(tokens)[:, None]
    j = np.arange(tokens)[None, :]
    visible = j <= i
    if window is not None:
        visible &= j > i - window
    scores = np.where(visible[None], scores, -np.inf)
    return softmax(scores, axis=-1) @ v


def silu(x: np.ndarray) -> np.ndarray:
    return x / (1.0 + np.exp(-x))


def gated_feed_forward(x: np.ndarray, gate: np.ndarray, up: np.ndarray, down: np.ndarray) -> np.ndarray:
    """/root/reference/src/pylon/model/layers.py:25-27 — down(silu(gate(x)) * up(x));
    the reference fuses gate and up into one matrix with gate's rows first
    (/root/reference/src/pylon/model/weights.py:65-67), which is the same thing."""
    return (silu(x @ gate.T) * (x @ up.T)) @ down.T


def attention_half(h: np.ndarray, w: Mapping[str, np.ndarray], prefix: str, cfg: Mapping,
                   positions: Sequence[int], borrowed=None, window: Optional[int] = None):
    """/root/reference/src/pylon/model/layers.py:125-138 — project, split heads, RMSNorm q
    and k over the head axis (before the rotation), rotate q and k, attend, project out.
    v is neither normed nor rotated.  Returns (output, (k, v)); with ``borrowed`` = (k, v)
    of another run, only q is formed and those keys and values are attended."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    tokens = h.shape[0]
    cos, sin = rope_tables(positions, hd, cfg["rope_theta"])
    q = (h @ w[f"{prefix}.self_attn.q_proj.weight"].T).reshape(tokens, nh, hd).transpose(1, 0, 2)
    q = apply_rope(rms_norm(q, w[f"{prefix}.self_attn.q_norm.weight"], eps), cos, sin)
    if borrowed is None:
        k = (h @ w[f"{prefix}.self_attn.k_proj.weight"].T).reshape(tokens, nkv, hd).transpose(1, 0, 2)
        v = (h @ w[f"{prefix}.self_attn.v_proj.weight"].T).reshape(tokens, nkv, hd).transpose(1, 0, 2)
        k = apply_rope(rms_norm(k, w[f"{prefix}.self_attn.k_norm.weight"], eps), cos, sin)
    else:
        k, v = borrowed
    # No scale is passed in the reference: the default 1/sqrt(head_dim) applies
    # (/root/reference/src/pylon/kv/cache.py:361-363).
    ctx = causal_attention(q, k, v, 1.0 / math.sqrt(hd), window)
    ctx = ctx.transpose(1, 0, 2).reshape(tokens, nh * hd)
    return ctx @ w[f"{prefix}.self_attn.o_proj.weight"].T, (k, v)


def block(x: np.ndarray, w: Mapping[str, np.ndarray], layer: int, cfg: Mapping,
          positions: Sequence[int], borrowed=None, window: Optional[int] = None):
    """/root/reference/src/pylon/model/layers.py:191-200 —
    x = x + attention(input_norm(x)); x = x + feed_forward(post_attention_norm(x))."""
    p = f"model.layers.{layer}"
    eps = cfg["rms_norm_eps"]
    a, kv = attention_half(rms_norm(x, w[f"{p}.input_layernorm.weight"], eps), w, p, cfg,
                           positions, borrowed, window)
    x = x + a
    h = rms_norm(x, w[f"{p}.post_attention_layernorm.weight"], eps)
    x = x + gated_feed_forward(h, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                               w[f"{p}.mlp.down_proj.weight"])
    return x, kv


def forward(weights: Mapping[str, np.ndarray], cfg: Mapping, token_ids: Sequence[int], *,
            schedule: Optional[Sequence] = None, windows: Optional[Mapping[int, int]] = None,
            start_position: int = 0) -> np.ndarray:
    """/root/reference/src/pylon/model/model.py:133-139 with ``every_position``: embed,
    every block in order, final norm, vocabulary head (the embedding matrix again when
    ``tie_word_embeddings``, model.py:32).  Returns logits [tokens, vocab].

    ``schedule`` (not in the reference) lists the runs as (layer, borrowed_run or None);
    ``windows`` maps a layer to its window; ``start_position`` shifts all positions."""
    w = {name: np.asarray(value, dtype=F) for name, value in weights.items()}
    ids = np.asarray(token_ids, dtype=np.int64)
    positions = np.arange(len(ids)) + start_position
    x = w["model.embed_tokens.weight"][ids]
    if schedule is None:
        schedule = [(layer, None) for layer in range(cfg["num_hidden_layers"])]
    kept = []
    for layer, borrow in schedule:
        borrowed = kept[borrow] if borrow is not None else None
        x, kv = block(x, w, layer, cfg, positions, borrowed, (windows or {}).get(layer))
        kept.append(kv)
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return x @ head.T


# ---- sampling -------------------------------------------------------------------------------

def greedy(logits: np.ndarray) -> int:
    """/root/reference/src/pylon/decode/runner.py:511-512 — argmax (first of equals)."""
    return int(np.argmax(logits))


def sampling_distribution(logits: np.ndarray, temperature: float, top_p: float) -> np.ndarray:
    """/root/reference/src/pylon/decode/runner.py:513-523 — softmax(logits / T); with
    top_p < 1: sort descending, remove a token when the cumulative mass *before* it
    already exceeds top_p (the first is always kept), renormalise.  Returned in vocabulary
    order."""
    p = softmax(np.asarray(logits, dtype=F) / temperature)
    if top_p == 1:
        return p
    order = np.argsort(-p, kind="stable")
    sorted_p = p[order]
    remove = np.cumsum(sorted_p) > top_p
    remove[1:] = remove[:-1].copy()
    remove[0] = False
    sorted_p[remove] = 0.0
    sorted_p /= sorted_p.sum()
    out = np.zeros_like(p)
    out[order] = sorted_p
    return out


def sample_with_uniform(logits: np.ndarray, temperature: float, top_p: float, u: float) -> int:
    """The engine draws by reading the cumulative distribution, taken in vocabulary
    order, at a uniform number u in [0, 1) (the reference calls ``torch.multinomial``,
    whose stream cannot be reproduced): the first index whose cumulative mass exceeds u."""
    if temperature == 0:
        return greedy(logits)
    p = sampling_distribution(logits, temperature, top_p)
    cdf = np.cumsum(p)
    return int(min(np.searchsorted(cdf, u * cdf[-1], side="right"), len(p) - 1))
