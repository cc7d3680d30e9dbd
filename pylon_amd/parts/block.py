"""The arrangement of a layer's parts.  ``pre_norm``
(/root/reference/src/pylon/model/layers.py:176-200):
``x = x + mixer(norm1(x)); x = x + feed_forward(norm2(x))``.

The residual stream is float32.  A block receives the stream together with the
previous part's output that has not been added yet, so that every residual sum is
formed inside the norm kernel that follows it; it hands back the same pair."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from ..config.specs import LayerSpec
from .base import Part, requirement_list
from .registry import build_part, register_part


class PreNormBlock(Part):
    def __init__(self, spec: LayerSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        self.spec = spec
        kw = dict(dtype=dtype, device=device)
        self.mixer_norm = self.add_child("mixer_norm", build_part("norm", spec.mixer_norm, **kw))
        self.mixer = self.add_child("mixer", build_part("mixer", spec.mixer, **kw))
        if (spec.feed_forward is None) != (spec.feed_forward_norm is None):
            raise ValueError("a feed-forward and its norm come together or not at all")
        self.feed_forward = None  # a layer may consist of its mixer alone
        if spec.feed_forward is not None:
            self.feed_forward_norm = self.add_child(
                "feed_forward_norm", build_part("norm", spec.feed_forward_norm, **kw)
            )
            self.feed_forward = self.add_child(
                "feed_forward", build_part("feed_forward", spec.feed_forward, **kw)
            )

    def cache_requirement(self):
        return self.mixer.cache_requirement()

    def decode_signature(self, rows: int, bound: int) -> tuple:
        describe = getattr(self.mixer, "decode_signature", None)
        return ("bound", bound) if describe is None else describe(rows, bound)

    def forward(self, resid: torch.Tensor, delta: Optional[torch.Tensor], ctx, cache,
                stores: bool) -> Tuple[torch.Tensor, torch.Tensor]:
        h = self.mixer_norm.add_forward(resid, delta)
        mixed = self.mixer.forward(h, ctx, cache, stores)
        if self.feed_forward is None:
            return resid, mixed
        h = self.feed_forward_norm.add_forward(resid, mixed)
        return resid, self.feed_forward.forward(h, ctx)


class SandwichNormBlock(Part):
    """Every sublayer normed on both sides: ``x += post1(mixer(conv(norm1(x))))``, then, if the
    layer has a feed-forward, ``x += post2(ff(norm2(x)))``; ``conv`` is an optional short
    convolution in front of the mixer, whose input is then kept in float32.  The norm after a
    sublayer is not a launch of its own: its output travels as :class:`~.base.Normed` to the
    next norm, which norms it, adds it and norms the sum in one kernel."""

    def __init__(self, spec: LayerSpec, *, dtype: torch.dtype, device) -> None:
        super().__init__()
        if spec.mixer_post_norm is None:
            raise ValueError("a sandwich_norm layer needs the norm after its mixer")
        if (spec.feed_forward is None) != (spec.feed_forward_norm is None) or \
                (spec.feed_forward is None) != (spec.feed_forward_post_norm is None):
            raise ValueError("a feed-forward and its two norms come together or not at all")
        self.spec = spec
        kw = dict(dtype=dtype, device=device)
        self.input_conv = None
        if spec.input_conv is not None:
            self.input_conv = self.add_child("input_conv", build_part("conv", spec.input_conv, **kw))
        self.mixer_norm = self.add_child("mixer_norm", build_part(
            "norm", spec.mixer_norm, dtype=torch.float32 if self.input_conv is not None else dtype, device=device))
        self.mixer = self.add_child("mixer", build_part("mixer", spec.mixer, **kw))
        self.mixer_post_norm = self.add_child("mixer_post_norm", build_part("norm", spec.mixer_post_norm, **kw))
        self.feed_forward = None
        if spec.feed_forward is not None:
            self.feed_forward_norm = self.add_child("feed_forward_norm", build_part("norm", spec.feed_forward_norm, **kw))
            self.feed_forward = self.add_child("feed_forward", build_part("feed_forward", spec.feed_forward, **kw))
            self.feed_forward_post_norm = self.add_child(
                "feed_forward_post_norm", build_part("norm", spec.feed_forward_post_norm, **kw))

    def cache_requirement(self):
        needs = requirement_list(self.mixer.cache_requirement())
        if self.input_conv is not None:
            needs += requirement_list(self.input_conv.cache_requirement())
        return needs if len(needs) != 1 else needs[0]

    def decode_signature(self, rows: int, bound: int) -> tuple:
        describe = getattr(self.mixer, "decode_signature", None)
        return ("bound", bound) if describe is None else describe(rows, bound)

    def forward(self, resid: torch.Tensor, delta, ctx, cache, stores: bool):
        h = self.mixer_norm.add_forward(resid, delta)
        if self.input_conv is not None:
            h = self.input_conv.forward(h, ctx, cache)
        pending = self.mixer_post_norm.pending(self.mixer.forward(h, ctx, cache, stores))
        if self.feed_forward is None:
            return resid, pending
        h = self.feed_forward_norm.add_forward(resid, pending)
        return resid, self.feed_forward_post_norm.pending(self.feed_forward.forward(h, ctx))


register_part("block", "pre_norm", PreNormBlock, replace=True)
register_part("block", "sandwich_norm", SandwichNormBlock, replace=True)
