"""Retention: linear attention with a fixed decay per head, no softmax and no denominator.

``[q; k; v; g] = W h`` in one product; q and k are rotated by the token's position and k is
multiplied by ``head_dim ** -0.5``; per request and head a float32 state ``S`` of
``head_dim x v_head_dim`` numbers goes from token to token, ``S_t = decay S_{t-1} + k_t v_t^T``,
``o_t = S_t^T q_t``; every head's ``o`` is divided by its root mean square, the heads are
multiplied by ``silu(g)`` and projected.  The state lives in the request's state slot and
starts at zero; rotation, state, norm and gate are computed in float32 whatever the model's
element type."""
from __future__ import annotations

import torch

from ..config.specs import RetentionSpec
from ..kernels import ops
from .base import Part, StateRequirement
from .registry import build_part, register_part


CHUNKED_FROM = 4  # a step whose longest row brings at least this many tokens takes the chunked form


class Retention(Part):
    def __init__(self, spec: RetentionSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if len(spec.decay) != spec.n_heads:
            raise ValueError(f"retention needs one decay per head: {len(spec.decay)} for {spec.n_heads} heads")
        if not 1 <= spec.v_head_dim <= 256 or not 1 <= spec.head_dim <= 1024:
            raise ValueError("retention takes heads of up to 1024 key and 256 value elements")
        self.spec = spec
        self.dtype = dtype
        qk, vg = spec.n_heads * spec.head_dim, spec.n_heads * spec.v_head_dim
        self.add_param("qkvg", (2 * qk + 2 * vg, spec.hidden_size), dtype, device)
        self.add_param("out", (spec.hidden_size, vg), dtype, device)
        self.decay = torch.tensor(list(spec.decay), dtype=torch.float32).to(device)
        self.position = self.add_child("position", build_part("position", spec.position, dtype=dtype, device=device))

    def cache_requirement(self) -> StateRequirement:
        spec = self.spec
        return StateRequirement((spec.n_heads, spec.head_dim, spec.v_head_dim), torch.float32)

    def decode_signature(self, rows: int, bound: int) -> tuple:
        return ("retention",)  # nothing of its launches depends on the requests' lengths

    def forward(self, h: torch.Tensor, ctx, cache, stores: bool) -> torch.Tensor:
        spec = self.spec
        if not stores:
            raise ValueError("a retention layer cannot borrow another run's state")
        rotary = self.position.rotary()
        proj = ops.linear(h, self.params["qkvg"], out_dtype=self.dtype)
        rot_dims = rotary[1] if rotary else 0
        # prompt portions of a bfloat16 model run 32 tokens at a time on the matrix cores; steps of
        # single tokens, float32 models and odd head sizes token by token
        chunked = (not ctx.decode_only and ctx.max_count >= CHUNKED_FROM and ops.retention_chunked_ok(
            self.dtype, dim=spec.head_dim, vdim=spec.v_head_dim, rot_dims=rot_dims))
        mixed = ops.retention_recurrent(
            proj, cache.state, self.decay, rotary[0] if rotary else None, ctx.positions, ctx.row_start,
            ctx.row_slots, rows=ctx.rows, heads=spec.n_heads, dim=spec.head_dim, vdim=spec.v_head_dim,
            rot_dims=rot_dims, eps=spec.norm_eps, k_scale=spec.head_dim ** -0.5, chunked=chunked,
            max_count=ctx.max_count)
        return ops.linear_for_residual(mixed, self.params["out"], out_dtype=self.dtype)


register_part("mixer", "retention", Retention, replace=True)
