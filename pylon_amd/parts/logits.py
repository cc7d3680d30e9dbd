"""Parts that work on the float32 logits after the vocabulary head."""
from __future__ import annotations

import torch

from ..config.specs import LogitScaleSpec, LogitSoftcapSpec
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


class LogitSoftcap(Part):
    """``logits <- cap * tanh(logits / cap)``, in place."""

    def __init__(self, spec: LogitSoftcapSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if not spec.cap > 0:
            raise ValueError(f"a soft cap must be positive, got {spec.cap!r}")
        self.spec = spec

    def forward(self, logits: torch.Tensor, ctx) -> torch.Tensor:
        ops.softcap_(logits, self.spec.cap)
        return logits


register_part("logits", "scale", LogitScale, replace=True)
register_part("logits", "softcap", LogitSoftcap, replace=True)
