"""Grouped-query attention over the paged cache
(/root/reference/src/pylon/model/layers.py:81-138; cache side
/root/reference/src/pylon/kv/cache.py:457-476).

``[q; k; v] = Wqkv h`` in one product, per-head RMSNorm of q and k (if the spec asks),
position encoding of q and k, k and v stored at the tokens' cache slots, causal softmax
attention of every token over its request's keys, output projection.  A run that borrows
another run's cache projects q only and stores nothing.
"""
from __future__ import annotations

import torch

from ..config.specs import AttentionSpec
from ..kernels import ops
from .base import KVRequirement, Part
from .registry import build_part, register_part


class Attention(Part):
    def __init__(self, spec: AttentionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("The number of Q heads must be divisible by the number of KV heads.")
        if spec.head_dim % 16 or not 16 <= spec.head_dim <= 512:
            raise ValueError(
                f"head_dim {spec.head_dim} is not supported: the attention kernels take "
                "multiples of 16 from 16 to 512"
            )
        if spec.window is not None and spec.window < 1:
            raise ValueError("window must be positive (or None for full attention)")
        self.spec = spec
        self.dtype = dtype
        q, kv = spec.q_size, spec.kv_size
        self.add_param("qkv", (q + 2 * kv, spec.hidden_size), dtype, device)
        self.add_param("out", (spec.hidden_size, q), dtype, device)
        if spec.qk_norm:
            self.add_param("q_norm", (spec.head_dim,), torch.float32, device, role="vector")
            self.add_param("k_norm", (spec.head_dim,), torch.float32, device, role="vector")
        self.position = self.add_child("position", build_part("position", spec.position, dtype=dtype, device=device))

    def cache_requirement(self) -> KVRequirement:
        return KVRequirement(self.spec.n_kv_heads, self.spec.head_dim, self.spec.window)

    def _span(self, ctx) -> int:
        """The most keys a token of this step attends to."""
        return ctx.max_len if self.spec.window is None else min(ctx.max_len, self.spec.window)

    def decode_signature(self, rows: int, bound: int) -> tuple:
        """Of a bound on the lengths, a decode-only step's launches take only how the keys of
        a request are shared between workgroups and waves."""
        span = bound if self.spec.window is None else min(bound, self.spec.window)
        return ("attention",) + tuple(ops.decode_launch(rows, self.spec.n_kv_heads, span))

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        spec = self.spec
        tokens = h.shape[0]
        weight = self.params["qkv"]
        if not stores:
            weight = weight[: spec.q_size]
        rotary = self.position.rotary()
        if ctx.decode_only and cache.k is not None and ops.decode_fused_ok(
                self.dtype, cache.k, tokens=tokens, n_heads=spec.n_heads, head_dim=spec.head_dim,
                rot_dim=rotary[1] if rotary else 0):
            # one launch adds the projection's partial sums if it comes as such, norms and
            # rotates q and k, stores k and v, and attends
            qkv = ops.linear_summed_later(h, weight, out_dtype=self.dtype)
            cuts, splits = ops.decode_launch(tokens, spec.n_kv_heads, self._span(ctx))
            context = ops.attention_decode_fused(
                qkv, cache.k, cache.v, cache.block_table, None, ctx.positions,
                n_heads=spec.n_heads, q_weight=self.params.get("q_norm"), k_weight=self.params.get("k_norm"),
                eps=spec.qk_norm_eps, inv_freq=rotary[0] if rotary else None,
                slot_map=cache.slot_map if stores else None,
                page_size=cache.page_size, window=spec.window, scale=spec.scale, n_splits=splits, n_cuts=cuts,
            )
            return ops.linear_for_residual(context.view(tokens, spec.q_size), self.params["out"],
                                           out_dtype=self.dtype)
        qkv = ops.linear(h, weight, out_dtype=self.dtype)
        q = torch.empty((tokens, spec.n_heads, spec.head_dim), dtype=self.dtype, device=h.device)
        ops.qkv_prepare(
            qkv, q, cache.k, cache.v,
            n_heads=spec.n_heads, n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim,
            q_weight=self.params.get("q_norm"), k_weight=self.params.get("k_norm"),
            eps=spec.qk_norm_eps,
            inv_freq=rotary[0] if rotary else None, rot_dim=rotary[1] if rotary else 0,
            positions=ctx.positions, slot_map=cache.slot_map, store_kv=stores,
        )
        if ctx.decode_only and ops.decode_attention_ok(q, cache.k):
            cuts, splits = ops.decode_launch(tokens, spec.n_kv_heads, self._span(ctx))
            # in a decode-only step token t is row t
            context = ops.attention_decode(
                q, cache.k, cache.v, cache.block_table, None, ctx.positions,
                page_size=cache.page_size, window=spec.window, scale=spec.scale, n_splits=splits, n_cuts=cuts,
            )
        elif ops.prefill_attention_ok(q, cache.k, cache.block_table):
            group = spec.n_heads // spec.n_kv_heads
            rows = ops.prefill_rows(tokens, spec.n_heads, group)
            context = torch.empty_like(q)
            # Decoding requests at the head of a mixed step go to the decode kernel (a
            # single query row would walk a long context alone in a prefill workgroup).
            singles = ctx.leading_singles
            if not (0 < singles <= ops.DECODE_MAX_TOKENS and ops.decode_attention_ok(q[:singles], cache.k)):
                singles = 0
            if singles:
                span = int(ctx.starts[:singles].max()) + 1
                if spec.window is not None:
                    span = min(span, spec.window)
                cuts, splits = ops.decode_launch(singles, spec.n_kv_heads, span)
                ops.attention_decode(
                    q[:singles], cache.k, cache.v, cache.block_table, None, ctx.positions[:singles],
                    page_size=cache.page_size, window=spec.window, scale=spec.scale, n_splits=splits,
                    n_cuts=cuts, out=context[:singles],
                )
            if singles < ctx.rows:
                tiles = ctx.token_tiles(rows // group, skip_rows=singles, fold=ops.prefill_fold(spec.n_kv_heads))
                ops.attention_prefill(
                    q, cache.k, cache.v, cache.block_table, tiles,
                    page_size=cache.page_size, window=spec.window, scale=spec.scale, rows=rows, out=context,
                )
        else:
            context = ops.paged_attention(
                q, cache.k, cache.v, cache.block_table, ctx.tok_row, ctx.positions,
                page_size=cache.page_size, window=spec.window, scale=spec.scale,
            )
        return ops.linear_for_residual(context.view(tokens, spec.q_size), self.params["out"],
                                       out_dtype=self.dtype)


register_part("mixer", "attention", Attention, replace=True)
