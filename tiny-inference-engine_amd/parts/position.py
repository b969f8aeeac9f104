"""Rotary position encoding, rotate-half pairing.

``inv_freq[i] = 1 / theta^(2i / head_dim)`` for i < head_dim / 2, computed in
float32 exactly as ``src/backend/rope.h:9-13`` does; the angle of pair
(i, i + head_dim/2) at position p is ``float(p) * inv_freq[i]``
(``src/backend/cpu/cpu_backend.cpp:180-188``). The whole head is rotated; queries
and keys are, values are not. Parameters: ``head_dim``, ``theta``.
"""

from __future__ import annotations

import numpy as np
import torch

from .. import kernels
from ..errors import InvalidArgument
from .base import Position, register_part


@register_part("position", "rope_neox")
class RopeNeox(Position):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True

    def __init__(self, params):
        super().__init__(params)
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        if self.head_dim % 2:
            raise InvalidArgument(f"head_dim {self.head_dim} must be even for rotary embeddings")
        if not self.theta > 0:
            raise InvalidArgument(f"rope theta must be positive, got {self.theta}")
        self.inv_freq: torch.Tensor = None

    def host_inv_freq(self) -> np.ndarray:
        i = np.arange(self.head_dim // 2, dtype=np.float32)
        exponent = (np.float32(2.0) * i) / np.float32(self.head_dim)
        return (np.float32(1.0) / np.power(np.float32(self.theta), exponent, dtype=np.float32)).astype(np.float32)

    def load(self, fetch, mode, device) -> None:
        self.inv_freq = torch.from_numpy(self.host_inv_freq()).to(device)

    def rotary_table(self):
        return self.inv_freq, self.head_dim, "rotate_half"

    def angles(self, ctx) -> torch.Tensor:
        """cos | sin of this step's positions, ``[T, head_dim]`` float32: computed once a step, shared by all layers."""
        key = ("rope_angles", self.head_dim, self.theta)
        table = ctx.notes.get(key)
        if table is None:
            table = ctx.scratch(f"rope.angles:{self.head_dim}:{self.theta}", (ctx.num_tokens, self.head_dim),
                                torch.float32)
            kernels.rope_angles(ctx.batch.positions, self.inv_freq, table)
            ctx.notes[key] = table
        return table


@register_part("position", "none")
class NoPosition(Position):
    """No position encoding: queries and keys are left as they are."""

    capturable = True
    replayable = True

    def rotary_table(self):
        return None, 0, "none"
