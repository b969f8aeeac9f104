"""The end of the model: final norm and vocabulary projection on the wanted rows only.

``last = x[rows]``; ``last = norm(last)``; ``logits = last @ W^T`` in float32;
no scaling, no soft-cap, no bias (``src/model/qwen3.cpp:248-262``). With
``tied_to`` set the projection uses that tensor (the embedding matrix) and a
``lm_head`` tensor in the file is accepted, shape-checked and ignored
(``qwen3.cpp:94-100``). Parameters: ``vocab``, ``hidden``, ``norm`` (a PartSpec),
``weight`` (tensor name), ``tied_to`` (tensor name or None).
"""

from __future__ import annotations

from typing import List

import torch

from .. import kernels
from .base import Head, Part, StepContext, TensorSpec, build_part, register_part


@register_part("head", "lm_head")
class LmHead(Head):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph

    def __init__(self, params):
        super().__init__(params)
        self.vocab = int(params["vocab"])
        self.hidden = int(params["hidden"])
        self.norm = build_part("norm", params["norm"])
        self.weight_name = params["weight"]
        self.tied_to = params.get("tied_to")
        self.weight: torch.Tensor = None

    def children(self) -> List[Part]:
        return [self.norm]

    def tensors(self) -> List[TensorSpec]:
        shape = (self.vocab, self.hidden)
        if self.tied_to:
            return [TensorSpec(self.tied_to, shape, "matrix", ("normal", 0.02)),
                    TensorSpec(self.weight_name, shape, "matrix", ("normal", 0.02), optional=True)]
        return [TensorSpec(self.weight_name, shape, "matrix", ("normal", 0.02))]

    def load(self, fetch, mode, device) -> None:
        w = fetch(self.tied_to or self.weight_name, "matrix")
        # The blocked copy is the head's own: a tied embedding table keeps its rows for the gather.
        self.weight = kernels.pack_weight(w) if kernels.packable(w) else w

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        last = self.norm.forward(ctx, x, rows=rows, out_name="head.norm")
        logits = ctx.scratch("head.logits", (rows.numel(), self.vocab), torch.float32)
        kernels.linear(last, self.weight, logits)
        return logits
