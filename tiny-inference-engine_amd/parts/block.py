"""Arrangements of a layer's parts.

``pre_norm`` is the reference's block (``src/model/qwen3.cpp:216-239``):
``x += mixer(norm(x)); x += feed_forward(norm(x))`` with the norms named
``pre_mixer`` and ``pre_feed_forward`` in the layer's spec and nothing applied
to the sub-layer outputs. A layer that has only one of the two parts runs that
half alone (and needs that half's norm only).
"""

from __future__ import annotations

import torch

from ..errors import InvalidArgument
from .base import Block, StepContext, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    NORMS = ("pre_mixer", "pre_feed_forward")

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        if layer.mixer is not None:
            h = self.normed(ctx, layer.norms["pre_mixer"], x, consumer=layer.mixer)
            layer.mixer.forward(ctx, h, cache, x)
        if layer.feed_forward is not None:
            h = self.normed(ctx, layer.norms["pre_feed_forward"], x, consumer=layer.feed_forward)
            layer.feed_forward.forward(ctx, h, x)

    @classmethod
    def check_layer(cls, layer) -> None:
        needed = [n for n, part in zip(cls.NORMS, (layer.mixer, layer.feed_forward)) if part is not None]
        if not needed:
            raise InvalidArgument("a pre_norm block needs a mixer, a feed-forward or both")
        missing = [n for n in needed if n not in layer.norms]
        if missing:
            raise InvalidArgument(f"a pre_norm block needs the norms {', '.join(needed)}; missing {', '.join(missing)}")
