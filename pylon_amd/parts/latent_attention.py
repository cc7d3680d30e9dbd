"""Latent attention: softmax attention whose keys and values are linear maps of one small latent
per token, which is all that the cache keeps.

``[c_q'; c'; g] = W_down h`` in one product (float32 sums); ``c_q = norm(c_q')``, ``c = norm(c')``
(root mean square over the latent, times a weight) and ``sigmoid(g)`` in one kernel, which also
puts ``c`` into the token's cache slot; ``q = W_uq c_q``.  Per head ``k_j = W_uk c_j`` and
``v_j = W_uv c_j``, so ``q . k_j = (W_uk^T q) . c_j`` and ``sum_j p_j v_j = W_uv (sum_j p_j c_j)``:
the queries are carried into the latent's space head by head, attention runs over the cached
latents themselves (one key/value head that all query heads share, keys and values the same
tensor), and the result is carried to the value space head by head, multiplied by the head's gate.
No positions are encoded; the mask is a sliding window, chunks, or plain causal.

The cache is ``[pages, page_size, 1, kv_rank]`` per run (``KVRequirement(values=False)``).
bfloat16 steps over latents of 64, 128 or 256 numbers run on the matrix-core attention kernels
(for a step of single tokens the heads are handed to the decode kernel in groups of at most 16,
each group as a query token of its own); everything else on the general kernel.
"""
from __future__ import annotations

import torch

from ..config.specs import LatentAttentionSpec
from ..kernels import ops
from .base import KVRequirement, Part
from .registry import register_part


def head_group(n_heads: int, most: int = 16) -> int:
    """The largest divisor of ``n_heads`` that is at most ``most``."""
    return max(g for g in range(1, min(n_heads, most) + 1) if n_heads % g == 0)


class LatentAttention(Part):
    def __init__(self, spec: LatentAttentionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        for name in ("n_heads", "head_dim", "v_head_dim", "q_rank", "kv_rank"):
            if getattr(spec, name) < 1:
                raise ValueError(f"latent attention: {name} must be positive")
        if spec.kv_rank > 512:
            raise ValueError(f"a latent of {spec.kv_rank} numbers is not supported: the attention kernels take up to 512")
        if spec.window is not None and spec.window < 1:
            raise ValueError("window must be positive (or None)")
        if spec.chunk is not None and (spec.chunk < 1 or spec.window is not None):
            raise ValueError("chunk must be positive, and a layer has a window or chunks, not both")
        self.spec = spec
        self.dtype = dtype
        self.n_gate = spec.n_heads if spec.gate else 0
        self.add_param("down", (spec.q_rank + spec.kv_rank + self.n_gate, spec.hidden_size), dtype, device)
        self.add_param("q_norm", (spec.q_rank,), torch.float32, device, role="vector")
        self.add_param("c_norm", (spec.kv_rank,), torch.float32, device, role="vector")
        self.add_param("uq", (spec.n_heads * spec.head_dim, spec.q_rank), dtype, device)
        self.add_param("uk", (spec.n_heads * spec.head_dim, spec.kv_rank), dtype, device)
        self.add_param("uv", (spec.n_heads * spec.v_head_dim, spec.kv_rank), dtype, device)
        self.add_param("out", (spec.hidden_size, spec.n_heads * spec.v_head_dim), dtype, device)
        self._uv_by_latent = None  # (version of uv, uv as [heads, kv_rank, v_head_dim])

    def cache_requirement(self) -> KVRequirement:
        spec = self.spec
        return KVRequirement(1, spec.kv_rank, spec.window, chunk=spec.chunk, values=False)

    def value_maps(self) -> torch.Tensor:
        """``uv`` with the latent's axis first inside every head, ``[heads, kv_rank, v_head_dim]``:
        how the per-head product reads it; made anew when the parameter has been written."""
        uv = self.params["uv"]
        key = (uv.data_ptr(), uv._version, uv.dtype)
        if self._uv_by_latent is None or self._uv_by_latent[0] != key:
            spec = self.spec
            self._uv_by_latent = (key, uv.view(spec.n_heads, spec.v_head_dim, spec.kv_rank).transpose(1, 2).contiguous())
        return self._uv_by_latent[1]

    def _span(self, bound: int) -> int:
        limit = self.spec.window if self.spec.window is not None else self.spec.chunk
        return bound if limit is None else min(bound, limit)

    def _decode_launch(self, queries: int, span: int) -> tuple:
        """(cuts, waves) of the decode kernel for ``queries`` query tokens (a group of heads each) over
        one shared key/value head: with so few workgroups a request's latents are cut over workgroups
        down to 128 a cut, until the workgroups fill the chip."""
        units = ops.compute_units()
        cuts = 1
        while cuts < 64 and queries * cuts * 2 <= units and cuts * 2 * 128 <= span:
            cuts *= 2
        return cuts, ops.decode_splits(queries * cuts, 1, -(-span // cuts), units)

    def _group(self) -> int:
        """Query heads that go to the decode kernel as one query token.  It takes up to 16, but over
        latents of 256 numbers it is faster with 8 (8 requests, 32 heads, a window of 1,024: 38.7 us
        in groups of 16 over 8 cuts, 17.4 in groups of 8)."""
        return head_group(self.spec.n_heads, 8 if self.spec.kv_rank >= 256 else 16)

    def _matrix_cores(self) -> bool:
        return self.dtype == torch.bfloat16 and self.spec.kv_rank in ops.DECODE_HEAD_DIMS

    def decode_signature(self, rows: int, bound: int) -> tuple:
        if not self._matrix_cores():
            return ("latent_attention",)
        group = self._group()
        return ("latent_attention",) + tuple(self._decode_launch(rows * (self.spec.n_heads // group), self._span(bound)))

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        spec = self.spec
        tokens = h.shape[0]
        heads, rank = spec.n_heads, spec.kv_rank
        down = ops.linear(h, self.params["down"], out_dtype=torch.float32)
        q_latent, gate = ops.latent_prepare(
            down, cache.k if stores else None, cache.slot_map if stores else None, q_rank=spec.q_rank,
            kv_rank=rank, n_gate=self.n_gate, q_weight=self.params["q_norm"], c_weight=self.params["c_norm"],
            eps=spec.norm_eps, out_dtype=self.dtype)
        q = ops.linear(q_latent, self.params["uq"], out_dtype=self.dtype)
        # the queries in the latent's space: q'_h = W_uk[h]^T q_h
        q = ops.head_project(q.view(tokens, heads, spec.head_dim), self.params["uk"].view(heads, spec.head_dim, rank))
        mask = dict(window=spec.window, chunk=spec.chunk)
        latents = cache.k  # [pages, page_size, 1, kv_rank]: keys and values at once
        group = self._group()
        repeat = heads // group
        if self._matrix_cores() and q.dtype == latents.dtype and ctx.decode_only \
                and tokens * repeat <= ops.DECODE_MAX_TOKENS:
            positions, rows = ctx.positions, None
            if repeat > 1:  # every group of heads a query token of its own, on its request's row of the table
                key = ("latent_attention.groups", repeat)
                if key not in ctx.memo:  # once a step, not once a layer
                    ctx.memo[key] = (ctx.positions.repeat_interleave(repeat), ctx.tok_row.repeat_interleave(repeat))
                positions, rows = ctx.memo[key]
            cuts, splits = self._decode_launch(tokens * repeat, self._span(ctx.max_len))
            mixed = ops.attention_decode(
                q.view(tokens * repeat, group, rank), latents, latents, cache.block_table, rows, positions,
                page_size=cache.page_size, scale=spec.scale, n_splits=splits, n_cuts=cuts, **mask,
            ).view(tokens, heads, rank)
        elif self._matrix_cores() and q.dtype == latents.dtype and ops.prefill_attention_ok(q, latents, cache.block_table):
            rows = ops.prefill_rows(tokens, heads, heads)
            mixed = torch.empty_like(q)
            tiles = ctx.token_tiles(rows // heads, fold=ops.prefill_fold(1))
            ops.attention_prefill(q, latents, latents, cache.block_table, tiles, page_size=cache.page_size,
                                  scale=spec.scale, rows=rows, out=mixed, **mask)
        else:
            mixed = ops.paged_attention(q, latents, latents, cache.block_table, ctx.tok_row, ctx.positions,
                                        page_size=cache.page_size, scale=spec.scale, **mask)
        # to the value space head by head, times the head's gate
        context = ops.head_project(mixed, self.value_maps(), gate=gate)
        return ops.linear_for_residual(context.view(tokens, heads * spec.v_head_dim), self.params["out"],
                                       out_dtype=self.dtype)


register_part("mixer", "latent_attention", LatentAttention, replace=True)
