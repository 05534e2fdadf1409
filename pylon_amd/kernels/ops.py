"""Tensor-level wrappers of the HIP entry points.

Every wrapper checks device, element type, contiguity and shapes on the host before
it launches, and launches on torch's current stream.  None has a CPU path.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import library as _lib
from . import plan
from .library import KernelError

F32 = 0
BF16 = 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"the kernels take float32 and bfloat16, not {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """The current stream's handle.  A step asks for it once per launch, a few hundred times:
    the two raw calls take a fifth of a microsecond, ``torch.cuda.current_stream()`` six."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _dev(t: Optional[torch.Tensor], name: str, dtype=None) -> int:
    """Device pointer of a checked tensor (0 for None)."""
    if t is None:
        return 0
    if not t.is_cuda:
        raise KernelError(f"{name} must live on the GPU; there is no CPU path")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
    return t.data_ptr()


def embed(ids: torch.Tensor, table: torch.Tensor, *, scale: float = 1.0,
          out: Optional[torch.Tensor] = None, chosen: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 ``out[t] = table[ids[t]] * scale``.  With ``chosen`` (int32, on the device) an
    id ``-(1 + s)`` is replaced by ``chosen[s]``: the token a sampler left there."""
    tokens = ids.numel()
    vocab, hidden = table.shape
    if out is None:
        out = torch.empty((tokens, hidden), dtype=torch.float32, device=table.device)
    elif out.shape != (tokens, hidden):
        raise KernelError(f"embed: out has shape {tuple(out.shape)}, expected {(tokens, hidden)}")
    _lib.call("pylon_embed", _dev(out, "out", torch.float32), _dev(table, "table"),
              dtype_code(table.dtype), _dev(ids, "ids", torch.int32),
              None if chosen is None else _dev(chosen, "chosen", torch.int32), tokens, hidden, vocab,
              float(scale), _stream())
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, *, out_dtype=None,
            row_idx: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``(x / sqrt(mean(x^2) + eps)) * weight`` over the last axis of a 2-D tensor."""
    if x.dim() != 2:
        raise KernelError("rmsnorm takes a 2-D input")
    dim = x.shape[1]
    if weight.shape != (dim,):
        raise KernelError(f"rmsnorm: weight has shape {tuple(weight.shape)}, expected ({dim},)")
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    out_dtype = out_dtype or x.dtype
    if out is None:
        out = torch.empty((rows, dim), dtype=out_dtype, device=x.device)
    elif out.shape != (rows, dim):
        raise KernelError("rmsnorm: out has the wrong shape")
    _lib.call("pylon_rmsnorm", _dev(out, "out"), dtype_code(out.dtype), _dev(x, "x"),
              dtype_code(x.dtype), _dev(weight, "weight", torch.float32),
              _dev(row_idx, "row_idx", torch.int32), rows, dim, float(eps), _stream())
    return out


def add_rmsnorm(resid: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out_dtype: torch.dtype, *, row_idx: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``resid += delta`` (float32, in place) and the RMSNorm of the sum.

    ``delta`` has the residual's shape, or is a stack ``[parts, tokens, dim]`` of partial
    sums that are added up first.  With ``row_idx`` only those rows are normed and
    ``resid`` is left as it is.
    """
    if resid.dim() != 2:
        raise KernelError("add_rmsnorm takes a 2-D residual")
    dim = resid.shape[1]
    n_delta, delta_stride = 1, 0
    if delta is not None:
        if delta.dim() == 3:
            n_delta, delta_stride = delta.shape[0], delta.shape[1] * delta.shape[2]
            if delta.shape[1:] != resid.shape:
                raise KernelError("add_rmsnorm: partial sums and resid differ in shape")
        elif delta.shape != resid.shape:
            raise KernelError("add_rmsnorm: delta and resid differ in shape")
    if weight.shape != (dim,):
        raise KernelError(f"add_rmsnorm: weight has shape {tuple(weight.shape)}, expected ({dim},)")
    rows = resid.shape[0] if row_idx is None else row_idx.numel()
    if out is None:
        out = torch.empty((rows, dim), dtype=out_dtype, device=resid.device)
    elif out.shape != (rows, dim) or out.dtype != out_dtype:
        raise KernelError("add_rmsnorm: out has the wrong shape or dtype")
    _lib.call("pylon_add_rmsnorm", _dev(out, "out"), dtype_code(out.dtype),
              _dev(resid, "resid", torch.float32), _dev(delta, "delta"),
              dtype_code(delta.dtype) if delta is not None else F32, n_delta, delta_stride,
              _dev(weight, "weight", torch.float32), _dev(row_idx, "row_idx", torch.int32),
              rows, dim, float(eps), _stream())
    return out


def residual_add(resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    if delta.shape != resid.shape:
        raise KernelError("residual_add: shapes differ")
    _lib.call("pylon_residual_add", _dev(resid, "resid", torch.float32), _dev(delta, "delta"),
              dtype_code(delta.dtype), resid.numel(), _stream())
    return resid


def silu_gate(gate_up: torch.Tensor, *, out_dtype: Optional[torch.dtype] = None,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate_up[:, :I]) * gate_up[:, I:]`` for a ``[tokens, 2I]`` input; the result may
    have another element type than the input (float32 sums in, bfloat16 out: one rounding)."""
    if gate_up.dim() != 2 or gate_up.shape[1] % 2:
        raise KernelError("silu_gate takes a [tokens, 2*I] input")
    tokens, two_i = gate_up.shape
    inter = two_i // 2
    out_dtype = out_dtype or (out.dtype if out is not None else gate_up.dtype)
    if out is None:
        out = torch.empty((tokens, inter), dtype=out_dtype, device=gate_up.device)
    elif out.shape != (tokens, inter) or out.dtype != out_dtype:
        raise KernelError("silu_gate: out has the wrong shape or dtype")
    _lib.call("pylon_silu_gate", _dev(out, "out"), dtype_code(out.dtype), _dev(gate_up, "gate_up"),
              dtype_code(gate_up.dtype), tokens, inter, _stream())
    return out


def qkv_prepare(qkv: torch.Tensor, q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                v_cache: Optional[torch.Tensor], *, n_heads: int, n_kv_heads: int, head_dim: int,
                q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor], eps: float,
                inv_freq: Optional[torch.Tensor], rot_dim: int, positions: Optional[torch.Tensor],
                slot_map: Optional[torch.Tensor], store_kv: bool) -> None:
    """Per-head norm and rotation of q and k; q to ``q_out``; k and v into cache slots."""
    if qkv.dim() != 2:
        raise KernelError("qkv_prepare takes a 2-D projection output")
    tokens, width = qkv.shape
    heads = n_heads + (2 * n_kv_heads if store_kv else 0)
    if width != heads * head_dim:
        raise KernelError(f"qkv_prepare: projection width {width} is not {heads} heads of {head_dim}")
    if q_out.shape != (tokens, n_heads, head_dim) or q_out.dtype != qkv.dtype:
        raise KernelError("qkv_prepare: q_out has the wrong shape or dtype")
    for name, wt in (("q_weight", q_weight), ("k_weight", k_weight)):
        if wt is not None and wt.shape != (head_dim,):
            raise KernelError(f"qkv_prepare: {name} must have shape ({head_dim},)")
    if inv_freq is not None and inv_freq.numel() != rot_dim // 2:
        raise KernelError("qkv_prepare: inv_freq must hold rot_dim/2 frequencies")
    if positions is not None and positions.numel() != tokens:
        raise KernelError("qkv_prepare: one position per token is required")
    if store_kv:
        if k_cache is None or v_cache is None or slot_map is None:
            raise KernelError("qkv_prepare: storing needs k_cache, v_cache and slot_map")
        if slot_map.numel() != tokens:
            raise KernelError("qkv_prepare: one cache slot per token is required")
        for name, c in (("k_cache", k_cache), ("v_cache", v_cache)):
            if c.dtype != qkv.dtype or c.shape[-2:] != (n_kv_heads, head_dim):
                raise KernelError(f"qkv_prepare: {name} must be [..., {n_kv_heads}, {head_dim}] of {qkv.dtype}")
    _lib.call("pylon_qkv_prepare", _dev(q_out, "q_out"), _dev(k_cache if store_kv else None, "k_cache"),
              _dev(v_cache if store_kv else None, "v_cache"), _dev(qkv, "qkv"), dtype_code(qkv.dtype),
              width, _dev(q_weight, "q_weight", torch.float32), _dev(k_weight, "k_weight", torch.float32),
              float(eps), _dev(inv_freq, "inv_freq", torch.float32), int(rot_dim),
              _dev(positions, "positions", torch.int32), _dev(slot_map if store_kv else None, "slot_map", torch.int32),
              tokens, n_heads, n_kv_heads, head_dim, 1 if store_kv else 0, _stream())


def paged_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                    block_table: torch.Tensor, tok_row: torch.Tensor, positions: torch.Tensor, *,
                    page_size: int, window: Optional[int], scale: float,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal attention of each token over its request's cached keys ``<=`` its position."""
    if q.dim() != 3:
        raise KernelError("paged_attention takes q as [tokens, heads, head_dim]")
    tokens, n_heads, head_dim = q.shape
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
        raise KernelError("paged_attention: caches must be [pages, page_size, kv_heads, head_dim]")
    pages, psize, n_kv_heads, hd = k_cache.shape
    if psize != page_size or hd != head_dim:
        raise KernelError("paged_attention: cache geometry does not match page_size/head_dim")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError("paged_attention: q and the caches differ in dtype")
    if pages * page_size >= 2 ** 31:
        raise KernelError("paged_attention: the cache holds more slots than an int32 can index")
    if block_table.dim() != 2:
        raise KernelError("paged_attention: block_table must be [rows, width]")
    if tok_row.numel() != tokens or positions.numel() != tokens:
        raise KernelError("paged_attention: one row id and one position per token are required")
    if out is None:
        out = torch.empty_like(q)
    elif out.shape != q.shape or out.dtype != q.dtype:
        raise KernelError("paged_attention: out has the wrong shape or dtype")
    _lib.call("pylon_paged_attention", _dev(out, "out"), _dev(q, "q"), _dev(k_cache, "k_cache"),
              _dev(v_cache, "v_cache"), dtype_code(q.dtype), _dev(block_table, "block_table", torch.int32),
              block_table.shape[1], _dev(tok_row, "tok_row", torch.int32),
              _dev(positions, "positions", torch.int32), tokens, n_heads, n_kv_heads, head_dim,
              page_size, int(window or 0), float(scale), _stream())
    return out


DECODE_HEAD_DIMS = (64, 128, 256)
DECODE_MAX_TOKENS = 1024  # beyond this many single-token rows the prefill kernel's tiling takes over


def decode_attention_ok(q: torch.Tensor, k_cache: torch.Tensor) -> bool:
    """Whether the key-split decode kernel takes this geometry."""
    tokens, n_heads, head_dim = q.shape
    n_kv_heads = k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and head_dim in DECODE_HEAD_DIMS and tokens <= DECODE_MAX_TOKENS
            and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16)


def decode_splits(tokens: int, n_kv_heads: int, max_len: Optional[int], units: int = plan.UNITS) -> int:
    """Wavefronts (1, 2, 4 or 8) that share the keys of one (token, key/value head):
    ranges of about 64 keys (one batch of loads per wave) while the launch stays within a
    few thousand waves.  ``max_len`` is the most keys a workgroup gets (an upper bound
    under graph capture)."""
    waves = 8
    if tokens * n_kv_heads > units:
        # more workgroups than compute units: smaller ones run side by side (64 tokens of 140
        # keys: 13.8 us with four waves, 21.6 with eight; of 1,000 keys: 47 against 52)
        waves = 4
    while waves > 1 and tokens * n_kv_heads * waves > 16 * units:
        waves //= 2
    if max_len is not None:
        while waves > 1 and (waves // 2) * 64 >= max_len:
            waves //= 2
    return waves


def _like(q: torch.Tensor, out: Optional[torch.Tensor], name: str) -> torch.Tensor:
    if out is None:
        return torch.empty_like(q)
    if out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
        raise KernelError(f"{name}: out must be contiguous and of q's shape and dtype")
    return out


def decode_cuts(tokens: int, n_kv_heads: int, max_len: Optional[int], units: int = plan.UNITS) -> int:
    """Workgroups that share the keys of one (token, key/value head) before the waves of
    each share theirs: more than one when a few requests would otherwise occupy a fraction of
    the chip.  From 768 keys of ``max_len`` on (which may be an upper bound above the true
    lengths), each cut at least 192 keys, up to one workgroup per compute unit.  Measured on 256
    units with 8 key/value heads of 128, the launch with its merge against one workgroup per
    (token, head): 1 token of 1,000 keys 14.1 us (4 cuts) against 20.6, of 2,000 keys 14.1 (8)
    against 31, of 8,000 keys 19.1 (32) against 125; 8 tokens of 700 keys 15.2 (4) against 19.7,
    of 2,000 keys 23.6 (4) against 42; 16 tokens of 2,000 keys 35 (2) against 49.  At 500 keys one
    workgroup is within a microsecond (13.2 to 14.3 us); and once the workgroups fill the units
    (32 tokens) a cut only adds the second kernel."""
    if max_len is None or max_len < 768:
        return 1
    cuts = 1
    while cuts < 64 and tokens * n_kv_heads * cuts * 2 <= units and cuts * 2 * 192 <= max_len:
        cuts *= 2
    return cuts


def decode_launch(tokens: int, n_kv_heads: int, span: int) -> tuple:
    """(cuts, splits) for decode attention of ``tokens`` single tokens that each see at most
    ``span`` keys, on the current device."""
    units = _lib.compute_units()
    cuts = decode_cuts(tokens, n_kv_heads, span, units)
    return cuts, decode_splits(tokens * cuts, n_kv_heads, -(-span // cuts), units)


def _decode_scratch(tokens: int, n_heads: int, head_dim: int, n_cuts: int, device) -> Optional[torch.Tensor]:
    if n_cuts <= 1:
        return None
    return torch.empty((tokens * n_heads * n_cuts * (head_dim + 2),), dtype=torch.float32, device=device)


def attention_decode(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_table: torch.Tensor, tok_row: Optional[torch.Tensor], positions: torch.Tensor, *,
                     page_size: int, window: Optional[int], scale: float, n_splits: int,
                     n_cuts: int = 1, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Paged attention of a few bfloat16 query tokens; ``n_splits`` wavefronts share the
    keys of each (token, key/value head) and merge their partial results, after ``n_cuts``
    workgroups have shared them first (their partial results meet in a second small
    kernel).  ``tok_row`` None means token ``t`` uses row ``t`` of the block table (a
    decode-only step), which saves the kernel one dependent trip to memory."""
    if q.dim() != 3 or not decode_attention_ok(q, k_cache):
        raise KernelError("attention_decode does not take this geometry")
    tokens, n_heads, head_dim = q.shape
    pages, psize, n_kv_heads, hd = k_cache.shape
    if psize != page_size or hd != head_dim or k_cache.shape != v_cache.shape:
        raise KernelError("attention_decode: cache geometry does not match page_size/head_dim")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError("attention_decode: q and the caches differ in dtype")
    if pages * page_size >= 2 ** 31:
        raise KernelError("attention_decode: the cache holds more slots than an int32 can index")
    if positions.numel() != tokens or block_table.dim() != 2:
        raise KernelError("attention_decode: one position per token and a 2-D table are required")
    if tok_row is None:
        if block_table.shape[0] < tokens:
            raise KernelError("attention_decode: without row ids the table needs a row per token")
    elif tok_row.numel() != tokens:
        raise KernelError("attention_decode: one row id per token is required")
    out = _like(q, out, "attention_decode")
    scratch = _decode_scratch(tokens, n_heads, head_dim, n_cuts, q.device)
    _lib.call("pylon_attention_decode", _dev(out, "out"), _dev(q, "q"), _dev(k_cache, "k_cache"),
              _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32), block_table.shape[1],
              _dev(tok_row, "tok_row", torch.int32), _dev(positions, "positions", torch.int32),
              tokens, n_heads, n_kv_heads, head_dim, page_size, int(window or 0), float(scale),
              int(n_splits), int(n_cuts), _dev(scratch, "scratch"), 0 if scratch is None else scratch.numel(),
              _stream())
    return out


def decode_fused_ok(qkv_dtype: torch.dtype, k_cache: torch.Tensor, *, tokens: int, n_heads: int, head_dim: int,
                    rot_dim: int) -> bool:
    """Whether the decode kernel can prepare q, k and v itself from a projection of
    ``qkv_dtype``: its geometry, and a rotation of the whole head or none."""
    n_kv_heads = k_cache.shape[2]
    return (qkv_dtype == torch.bfloat16 and k_cache.dtype == torch.bfloat16 and head_dim in DECODE_HEAD_DIMS
            and tokens <= DECODE_MAX_TOKENS and n_heads % n_kv_heads == 0 and n_heads // n_kv_heads <= 16
            and rot_dim in (0, head_dim))


def attention_decode_fused(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                           block_table: torch.Tensor, tok_row: Optional[torch.Tensor], positions: torch.Tensor, *,
                           n_heads: int, q_weight: Optional[torch.Tensor], k_weight: Optional[torch.Tensor],
                           eps: float, inv_freq: Optional[torch.Tensor], slot_map: Optional[torch.Tensor],
                           page_size: int, window: Optional[int], scale: float, n_splits: int,
                           n_cuts: int = 1) -> torch.Tensor:
    """:func:`qkv_prepare` and :func:`attention_decode` in one launch: from the raw projection
    ``qkv`` ``[tokens, (n_heads + 2 kv_heads) * head_dim]`` (``[tokens, n_heads * head_dim]``
    when ``slot_map`` is None and nothing is stored), bfloat16, or from float32 partial sums
    ``[parts, tokens, width]`` of it, which the kernel adds in order and rounds to bfloat16
    once.  Returns ``[tokens, n_heads, head_dim]``."""
    pages, psize, n_kv_heads, head_dim = k_cache.shape
    store = slot_map is not None
    parts = 0
    if qkv.dim() == 3:
        if qkv.dtype != torch.float32 or not qkv.is_contiguous():
            raise KernelError("attention_decode_fused: partial sums come as a contiguous float32 stack")
        parts = qkv.shape[0]
    elif qkv.dim() != 2 or qkv.dtype != torch.bfloat16:
        raise KernelError("attention_decode_fused takes a bfloat16 projection or float32 partial sums of it")
    tokens, width = qkv.shape[-2:]
    if width != (n_heads + (2 * n_kv_heads if store else 0)) * head_dim:
        raise KernelError("attention_decode_fused: the projection's width does not match the heads")
    if qkv.stride(-1) != 1 or qkv.stride(-2) % 8 or qkv.data_ptr() % 16:
        raise KernelError("attention_decode_fused: the projection's rows must be contiguous and 16-byte aligned")
    if not decode_fused_ok(torch.bfloat16, k_cache, tokens=tokens, n_heads=n_heads, head_dim=head_dim,
                           rot_dim=0 if inv_freq is None else 2 * inv_freq.numel()):
        raise KernelError("attention_decode_fused does not take this geometry")
    if psize != page_size or k_cache.shape != v_cache.shape or v_cache.dtype != k_cache.dtype:
        raise KernelError("attention_decode_fused: cache geometry does not match page_size")
    if pages * page_size >= 2 ** 31:
        raise KernelError("attention_decode_fused: the cache holds more slots than an int32 can index")
    if positions.numel() != tokens or block_table.dim() != 2 or (store and slot_map.numel() != tokens):
        raise KernelError("attention_decode_fused: one position and one slot per token and a 2-D table are required")
    for name, wt in (("q_weight", q_weight), ("k_weight", k_weight)):
        if wt is not None and wt.shape != (head_dim,):
            raise KernelError(f"attention_decode_fused: {name} must have shape ({head_dim},)")
    if tok_row is None:
        if block_table.shape[0] < tokens:
            raise KernelError("attention_decode_fused: without row ids the table needs a row per token")
    elif tok_row.numel() != tokens:
        raise KernelError("attention_decode_fused: one row id per token is required")
    out = torch.empty((tokens, n_heads, head_dim), dtype=torch.bfloat16, device=qkv.device)
    scratch = _decode_scratch(tokens, n_heads, head_dim, n_cuts, qkv.device)
    _lib.call("pylon_attention_decode_fused", _dev(out, "out"), qkv.data_ptr(), qkv.stride(-2), parts,
              qkv.stride(0) if parts else 0,
              _dev(q_weight, "q_weight", torch.float32), _dev(k_weight, "k_weight", torch.float32), float(eps),
              _dev(inv_freq, "inv_freq", torch.float32), _dev(k_cache, "k_cache"), _dev(v_cache, "v_cache"),
              _dev(slot_map, "slot_map", torch.int32), _dev(block_table, "block_table", torch.int32),
              block_table.shape[1], _dev(tok_row, "tok_row", torch.int32),
              _dev(positions, "positions", torch.int32), tokens, n_heads, n_kv_heads, head_dim, page_size,
              int(window or 0), float(scale), int(n_splits), int(n_cuts), _dev(scratch, "scratch"),
              0 if scratch is None else scratch.numel(), _stream())
    return out


PREFILL_ROWS = 128  # most (token, head) query rows one workgroup of the prefill kernel takes


def prefill_rows(tokens: int, n_heads: int, group: int) -> int:
    """Query rows per workgroup: 128 halve the traffic from LDS per matrix instruction, but a
    step with few query rows fills more of the chip with workgroups of 64 (which hold a
    group of at most 64 heads)."""
    return 128 if tokens * n_heads >= 128 * 512 or group > 64 else 64


def prefill_fold(n_kv_heads: int) -> int:
    """Tiles whose workgroups (one per tile and key/value head) fill the chip once: the unit in
    which the order of a step's tiles is folded (2,048 tokens at the Qwen3-4B geometry: 59 -> 56
    us; 4,096: 164 -> 158)."""
    return max(1, _lib.compute_units() // n_kv_heads)


PREFILL_MAX_PAGES = 4096  # block-table columns the prefill kernel keeps in LDS


def prefill_attention_ok(q: torch.Tensor, k_cache: torch.Tensor, block_table: Optional[torch.Tensor] = None) -> bool:
    tokens, n_heads, head_dim = q.shape
    n_kv_heads = k_cache.shape[2]
    return (q.dtype == torch.bfloat16 and head_dim in DECODE_HEAD_DIMS and n_heads % n_kv_heads == 0
            and n_heads // n_kv_heads <= PREFILL_ROWS
            and (block_table is None or block_table.shape[1] <= PREFILL_MAX_PAGES))


def attention_prefill(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_table: torch.Tensor, tiles: torch.Tensor, *, page_size: int,
                      window: Optional[int], scale: float, rows: Optional[int] = None,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Paged causal attention of bfloat16 prompt portions on the matrix cores.  ``tiles`` is
    int32 ``[n, 4]``: first token index, token count, block-table row and first position of
    runs of at most ``rows // group`` consecutive tokens of one request; ``rows`` (64 or 128,
    default :data:`PREFILL_ROWS`) is the number of query rows a workgroup takes."""
    rows = rows or PREFILL_ROWS
    if q.dim() != 3 or not prefill_attention_ok(q, k_cache, block_table):
        raise KernelError("attention_prefill does not take this geometry")
    tokens, n_heads, head_dim = q.shape
    pages, psize, n_kv_heads, hd = k_cache.shape
    if psize != page_size or hd != head_dim or k_cache.shape != v_cache.shape:
        raise KernelError("attention_prefill: cache geometry does not match page_size/head_dim")
    if k_cache.dtype != q.dtype or v_cache.dtype != q.dtype:
        raise KernelError("attention_prefill: q and the caches differ in dtype")
    if pages * page_size >= 2 ** 31:
        raise KernelError("attention_prefill: the cache holds more slots than an int32 can index")
    if tiles.dim() != 2 or tiles.shape[1] != 4 or block_table.dim() != 2:
        raise KernelError("attention_prefill: tiles must be [n, 4] and the block table 2-D")
    out = _like(q, out, "attention_prefill")  # rows that no tile covers are left as they are
    _lib.call("pylon_attention_prefill", _dev(out, "out"), _dev(q, "q"), _dev(k_cache, "k_cache"),
              _dev(v_cache, "v_cache"), _dev(block_table, "block_table", torch.int32), block_table.shape[1],
              _dev(tiles, "tiles", torch.int32), tiles.shape[0], n_heads, n_kv_heads, head_dim, page_size,
              int(window or 0), float(scale), int(rows), _stream())
    return out


def gemm_tiled(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: Optional[torch.dtype] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` with float accumulation on the vector units (no matrix cores)."""
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm: cannot multiply {tuple(x.shape)} by the transpose of {tuple(weight.shape)}")
    m, k = x.shape
    n = weight.shape[0]
    out_dtype = out_dtype or x.dtype
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    elif out.shape != (m, n):
        raise KernelError("gemm: out has the wrong shape")
    if x.stride(1) != 1 or weight.stride(1) != 1 or out.stride(1) != 1:
        raise KernelError("gemm: rows must be contiguous")
    for name, t in (("x", x), ("weight", weight), ("out", out)):
        if not t.is_cuda:
            raise KernelError(f"gemm: {name} must live on the GPU; there is no CPU path")
    _lib.call("pylon_gemm_tiled", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), dtype_code(x.dtype),
              weight.data_ptr(), dtype_code(weight.dtype), m, n, k, x.stride(0), weight.stride(0),
              out.stride(0), _stream())
    return out


SKINNY_ROWS = plan.FEW_ROWS    # one tile of rows of x
STREAM_ROWS = plan.STREAM_ROWS  # most rows of x a workgroup of a weight-streaming kernel takes
SPLIT_ROWS = plan.SPLIT_ROWS    # most rows the rows kernel takes, as two halves


def _streaming_ok(x: torch.Tensor, weight: torch.Tensor, rows: int) -> bool:
    """Operands a weight-streaming kernel takes: bfloat16, at most ``rows`` rows of x, rows of
    multiples of 8 elements at 16-byte aligned addresses."""
    return (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and 0 < x.shape[0] <= rows
            and weight.shape[1] % 8 == 0 and weight.stride(0) % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


def gemm_skinny(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype = torch.bfloat16,
                parts: int = 1, glu: bool = False,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` for at most 64 rows of bfloat16 ``x``, streaming ``weight`` once.

    ``parts > 1`` cuts K into that many ranges and returns float32 partial results
    ``[parts, M, N]`` for the consumer to add.  ``glu``: ``weight`` is a fused
    ``[2N, K]`` gate/up matrix and the result is ``silu(x @ gate.T) * (x @ up.T)``.
    """
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm_skinny: cannot multiply {tuple(x.shape)} by the transpose of {tuple(weight.shape)}")
    m, k = x.shape
    n = weight.shape[0]
    if glu:
        if n % 2:
            raise KernelError("gemm_skinny: a fused gate/up matrix has an even number of rows")
        n //= 2
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise KernelError("gemm_skinny takes bfloat16 operands")
    if not (x.is_cuda and weight.is_cuda) or x.stride(1) != 1 or weight.stride(1) != 1:
        raise KernelError("gemm_skinny: operands must be on the GPU with contiguous rows")
    shape = (parts, m, n) if parts > 1 else (m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32 if parts > 1 else out_dtype, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != (torch.float32 if parts > 1 else out_dtype) \
            or not out.is_cuda or not out.is_contiguous():
        raise KernelError(f"gemm_skinny: out must be contiguous, on the GPU and of shape {shape}")
    _lib.call("pylon_gemm_skinny", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), weight.data_ptr(),
              m, n, k, x.stride(0), weight.stride(0), n, parts, m * n, 1 if glu else 0, _stream())
    return out


def gemm_rows(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype = torch.bfloat16,
              parts: int = 1, col_tiles: int = 1, glu: bool = False, waves: int = 0, cols: int = 0,
              out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` for at most 128 rows of bfloat16 ``x``: the rows of ``x`` pass through
    LDS once per workgroup of up to 64 (``col_tiles=1``) or 128 (``col_tiles=2``) columns and
    ``weight`` is streamed once (beyond 64 rows each half of the rows has workgroups of its
    own, and two that take the same columns run side by side).  ``parts > 1`` cuts K into that many ranges and returns
    float32 partial results ``[parts, M, N]`` for the consumer to add.  ``glu``: ``weight`` is
    a fused ``[2N, K]`` gate/up matrix and the result is ``silu(x @ gate.T) * (x @ up.T)``,
    rounded once.  ``waves``: wavefronts per workgroup, 4 or 2 (0: the kernel's choice);
    ``cols``: columns per workgroup (0: the kernel's choice, an equal share for every
    workgroup of whole rounds over the compute units where that pays).  The sums depend on
    neither."""
    if x.dim() != 2 or weight.dim() != 2 or x.shape[1] != weight.shape[1]:
        raise KernelError(f"gemm_rows: cannot multiply {tuple(x.shape)} by the transpose of {tuple(weight.shape)}")
    m, k = x.shape
    n = weight.shape[0]
    if glu:
        if n % 2:
            raise KernelError("gemm_rows: a fused gate/up matrix has an even number of rows")
        n //= 2
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise KernelError("gemm_rows takes bfloat16 operands")
    if not (x.is_cuda and weight.is_cuda) or x.stride(1) != 1 or weight.stride(1) != 1:
        raise KernelError("gemm_rows: operands must be on the GPU with contiguous rows")
    shape = (parts, m, n) if parts > 1 else (m, n)
    if out is None:
        out = torch.empty(shape, dtype=torch.float32 if parts > 1 else out_dtype, device=x.device)
    elif tuple(out.shape) != shape or out.dtype != (torch.float32 if parts > 1 else out_dtype) \
            or not out.is_cuda or not out.is_contiguous():
        raise KernelError(f"gemm_rows: out must be contiguous, on the GPU and of shape {shape}")
    _lib.call("pylon_gemm_rows", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), weight.data_ptr(),
              m, n, k, x.stride(0), weight.stride(0), n, parts, m * n, int(col_tiles), 1 if glu else 0, int(waves),
              int(cols), _stream())
    return out


def _library_float(x: torch.Tensor, weight: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` of bfloat16 operands as float32: the library's product with a float32
    result, that is its float32 sums before any rounding."""
    if out is None:
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    return torch.mm(x, weight.t(), out_dtype=torch.float32, out=out)


def linear(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x @ weight.T`` (into ``out`` if given: contiguous, of the result's shape and type).

    bfloat16 by bfloat16: up to 64 rows go to a weight-streaming kernel where one is faster
    (:func:`plan.plan_projection`), more rows to the library matrix product (as the
    reference's ``nn.Linear`` does).  With a bfloat16 result the float32 sums are rounded once
    either way; with a float32 result (the logits) they come back unrounded either way (the
    library then writes its float32 sums): what a request's logits are rounded to does not
    depend on how many rows share its step.  Every pairing that involves float32 operands runs
    on the exact tiled kernel, which never uses a reduced-precision matrix mode.
    """
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16:
        if not x.is_cuda:
            raise KernelError("linear: operands must live on the GPU; there is no CPU path")
        if _streaming_ok(x, weight, STREAM_ROWS):
            choice = plan.plan_projection(x.shape[0], *weight.shape)  # no rule of it counts compute units
            if choice.kernel == "rows":
                return gemm_rows(x, weight, out_dtype=out_dtype, col_tiles=choice.col_tiles, out=out)
            if choice.kernel == "skinny":
                return gemm_skinny(x, weight, out_dtype=out_dtype, out=out)
        if out_dtype == torch.float32:
            return _library_float(x, weight, out)
        y = torch.nn.functional.linear(x, weight)
        y = y if out_dtype == torch.bfloat16 else y.to(out_dtype)
        return y if out is None else out.copy_(y)
    return gemm_tiled(x, weight, out_dtype=out_dtype, out=out)


def linear_summed_later(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype) -> torch.Tensor:
    """``x @ weight.T`` for a consumer that takes either the product in ``out_dtype`` or float32
    partial sums ``[parts, M, N]`` of it, to be added in order and rounded to ``out_dtype`` once
    (:func:`attention_decode_fused` does): up to 128 bfloat16 rows the weight-streaming
    kernel with K cut over workgroups (:func:`plan.plan_summed_later`), else :func:`linear`."""
    if out_dtype == torch.bfloat16 and _streaming_ok(x, weight, SPLIT_ROWS):
        choice = plan.plan_summed_later(x.shape[0], *weight.shape, units=_lib.compute_units())
        if choice.kernel == "rows" and choice.parts > 1:
            return gemm_rows(x, weight, out_dtype=torch.float32, parts=choice.parts, col_tiles=choice.col_tiles)
    return linear(x, weight, out_dtype=out_dtype)


def linear_for_residual(x: torch.Tensor, weight: torch.Tensor, *, out_dtype: torch.dtype) -> torch.Tensor:
    """A product whose result is about to be added to the float32 residual stream.  For up
    to 128 bfloat16 rows it comes back as unrounded float32 sums, which the fused residual norm
    adds: partial sums ``[parts, M, N]`` of a streaming kernel (K cut over workgroups), or,
    from 17 rows on for a matrix at which the library is faster, the library's float32
    result (:func:`plan.plan_residual`).  For more rows (prompt portions) it is the library's
    product rounded once to bfloat16."""
    if _streaming_ok(x, weight, SPLIT_ROWS):
        choice = plan.plan_residual(x.shape[0], *weight.shape, units=_lib.compute_units())
        if choice.kernel == "rows":
            return gemm_rows(x, weight, out_dtype=torch.float32, parts=choice.parts, col_tiles=choice.col_tiles)
        if choice.kernel == "skinny":
            return gemm_skinny(x, weight, out_dtype=torch.float32, parts=choice.parts)
        return _library_float(x, weight)
    return linear(x, weight, out_dtype=out_dtype)


def linear_glu(x: torch.Tensor, gate_up: torch.Tensor, *, out_dtype: torch.dtype) -> torch.Tensor:
    """``silu(x @ gate.T) * (x @ up.T)`` for a fused ``[2I, K]`` gate/up matrix.  Up to 128
    bfloat16 rows: the activation works on the float32 sums and its result is rounded once
    (in a streaming kernel's epilogue; or, where the library is faster and beyond 64 rows,
    from its float32 result: :func:`plan.plan_gated`).  More rows (prompt portions): the
    library's product rounded to bfloat16 first."""
    if _streaming_ok(x, gate_up, SPLIT_ROWS) and x.is_cuda and gate_up.shape[0] % 2 == 0:
        choice = plan.plan_gated(x.shape[0], gate_up.shape[0] // 2, gate_up.shape[1], gate_up.stride(0))
        if choice.kernel == "rows":
            return gemm_rows(x, gate_up, out_dtype=out_dtype, glu=True)
        if choice.kernel == "skinny":
            return gemm_skinny(x, gate_up, out_dtype=out_dtype, glu=True)
        return silu_gate(_library_float(x, gate_up), out_dtype=out_dtype)
    return silu_gate(linear(x, gate_up, out_dtype=out_dtype))


def _chosen_args(rows: int, chosen: Optional[torch.Tensor], place: Optional[torch.Tensor]):
    """The optional table that also receives the chosen ids: ``chosen[place[r]] = id``."""
    if chosen is None and place is None:
        return None, None
    if chosen is None or place is None:
        raise KernelError("chosen and place go together")
    if place.numel() != rows:
        raise KernelError("place must have one index per row")
    return _dev(chosen, "chosen", torch.int32), _dev(place, "place", torch.int32)


def _ids_out(rows: int, device, out: Optional[torch.Tensor]) -> torch.Tensor:
    if out is None:
        return torch.empty((rows,), dtype=torch.int32, device=device)
    if out.shape != (rows,) or out.dtype != torch.int32 or not out.is_cuda:
        raise KernelError("out must be int32 [rows] on the GPU")
    return out


_argmax_scratch: dict = {}


def _argmax_partials(rows: int, device: torch.device) -> torch.Tensor:
    """The first launch leaves up to 64 partial results of 8 bytes per row for the second: one
    buffer per device, kept and grown, so that a serving loop allocates nothing per step.
    Calls on one stream follow each other; callers on other streams bring their own order."""
    need = max(rows, 1) * 64 * 8
    have = _argmax_scratch.get(device)
    if have is None or have.numel() < need:
        have = torch.empty((max(need, 256 * 64 * 8),), dtype=torch.uint8, device=device)
        _argmax_scratch[device] = have
    return have


def argmax(logits: torch.Tensor, *, out: Optional[torch.Tensor] = None,
           chosen: Optional[torch.Tensor] = None, place: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The index of each row's largest logit (the lowest among equals); with ``chosen`` and
    ``place`` the ids are also written to ``chosen[place[r]]``."""
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("argmax takes [rows, vocab] logits with contiguous rows")
    rows, vocab = logits.shape
    if not logits.is_cuda or logits.dtype != torch.float32:
        raise KernelError("argmax takes float32 logits on the GPU")
    out = _ids_out(rows, logits.device, out)
    chosen_ptr, place_ptr = _chosen_args(rows, chosen, place)
    scratch = _argmax_partials(rows, logits.device)
    _lib.call("pylon_argmax", out.data_ptr(), logits.data_ptr(), rows, vocab, logits.stride(0),
              chosen_ptr, place_ptr, scratch.data_ptr(), scratch.numel(), _stream())
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, *, out: Optional[torch.Tensor] = None,
           chosen: Optional[torch.Tensor] = None, place: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row; rows with temperature 0 take the argmax.  ``chosen`` and ``place``
    as for :func:`argmax`."""
    if logits.dim() != 2 or logits.stride(1) != 1:
        raise KernelError("sample takes [rows, vocab] logits with contiguous rows")
    rows, vocab = logits.shape
    if not logits.is_cuda or logits.dtype != torch.float32:
        raise KernelError("sample takes float32 logits on the GPU")
    for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
        if t.numel() != rows:
            raise KernelError(f"sample: {name} must have one value per row")
    out = _ids_out(rows, logits.device, out)
    chosen_ptr, place_ptr = _chosen_args(rows, chosen, place)
    _lib.call("pylon_sample", out.data_ptr(), logits.data_ptr(), rows, vocab, logits.stride(0),
              _dev(temperature, "temperature", torch.float32), _dev(top_p, "top_p", torch.float32),
              _dev(uniform, "uniform", torch.float32), chosen_ptr, place_ptr, _stream())
    return out


def probe_read(data: torch.Tensor, sink: torch.Tensor) -> None:
    """Read every byte of ``data`` once (a measurement aid: the device's read bandwidth)."""
    if not data.is_contiguous() or not data.is_cuda:
        raise KernelError("probe_read takes a contiguous tensor on the GPU")
    _lib.call("pylon_probe_read", data.data_ptr(), data.numel() * data.element_size(),
              _dev(sink, "sink", torch.int32), _stream())
