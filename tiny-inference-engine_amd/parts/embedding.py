"""Token embedding: ``x[t, :] = float32(E[tokens[t], :])``, no scaling.

Reference: ``src/model/qwen3.cpp:75,213`` and ``src/backend/cpu/cpu_backend.cpp:51-76``.
Token ids are checked against the vocabulary when a batch is built, before
anything runs. Parameters: ``vocab``, ``hidden``, ``weight`` (tensor name).
"""

from __future__ import annotations

from typing import List

import torch

from .. import kernels
from .base import Embedding, StepContext, TensorSpec, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Embedding):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph

    def __init__(self, params):
        super().__init__(params)
        self.vocab = int(params["vocab"])
        self.hidden = int(params["hidden"])
        self.weight_name = params["weight"]
        self.weight: torch.Tensor = None

    def tensors(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.vocab, self.hidden), "matrix", ("normal", 0.02))]

    def load(self, fetch, mode, device) -> None:
        self.weight = fetch(self.weight_name, "matrix")

    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        x = ctx.scratch("residual", (token_ids.numel(), self.hidden), torch.float32)
        kernels.embed(self.weight, token_ids, x)
        return x
