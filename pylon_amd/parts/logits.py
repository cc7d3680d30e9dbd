"""Parts that work on the float32 logits after the vocabulary head."""
from __future__ import annotations

import torch

from ..config.specs import LogitScaleSpec
from ..kernels import ops
from .base import Part
from .registry import register_part


class LogitScale(Part):
    """``logits *= factor``, in place (so that a replayed graph leaves them where it did)."""

    def __init__(self, spec: LogitScaleSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec

    def forward(self, logits: torch.Tensor, ctx) -> torch.Tensor:
        if self.spec.factor != 1.0:
            ops.scale_(logits, self.spec.factor)
        return logits


register_part("logits", "scale", LogitScale, replace=True)
