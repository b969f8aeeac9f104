"""The dense SwiGLU feed-forward.

``g = h @ Wg^T``, ``u = h @ Wu^T``, ``a = g / (1 + exp(-g)) * u`` evaluated left
to right, ``out = a @ Wd^T``, added to the residual; no bias, no experts
(``src/model/qwen3.cpp:235-239``, ``src/backend/cpu/cpu_backend.cpp:195-207``).
Gate and up run as one product over the two matrices side by side; with bfloat16 weights
their rows are interleaved in blocks of 8 and the product's epilogue applies the activation.
Parameters: ``hidden``, ``intermediate``, ``names`` (``gate``, ``up``, ``down``).
"""

from __future__ import annotations

from typing import List

import torch

from .. import kernels
from .base import FeedForward, StepContext, TensorSpec, register_part
from .linear import Linear


@register_part("feed_forward", "swiglu")
class SwiGLU(FeedForward):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    takes_row_scale = True   # h goes into the gate/up product only

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.intermediate = int(params["intermediate"])
        names = params["names"]
        self.gate_up = Linear([names["gate"], names["up"]], [self.intermediate, self.intermediate], self.hidden)
        self.down = Linear([names["down"]], [self.hidden], self.intermediate)

    def tensors(self) -> List[TensorSpec]:
        return self.gate_up.tensors() + self.down.tensors()

    def load(self, fetch, mode, device) -> None:
        self.down.load(fetch)
        gate, up = fetch(self.gate_up.names[0], "matrix"), fetch(self.gate_up.names[1], "matrix")
        # bfloat16 weights and widths in steps of 8: gate and up rows are interleaved so that one
        # product computes both and its epilogue applies silu(gate) * up before anything is stored.
        self.fused = gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16 and \
            self.intermediate % 8 == 0 and self.hidden % 8 == 0
        if self.fused:
            self.gate_up.set_weight(kernels.interleave_gate_up(gate, up))
        else:
            self.gate_up.load(fetch)

    def forward(self, ctx: StepContext, h: torch.Tensor, residual: torch.Tensor) -> None:
        T = h.shape[0]
        act = ctx.scratch("swiglu.act", (T, self.intermediate))
        if self.fused and h.dtype == torch.bfloat16:
            kernels.linear_swiglu(h, self.gate_up.weight, act, row_scale=Linear.row_scale_for(ctx, h, self.gate_up.weight))
        else:
            gate_up = ctx.scratch("swiglu.gate_up", (T, 2 * self.intermediate))
            self.gate_up(h, gate_up, ctx=ctx)
            kernels.swiglu(gate_up, act)
        self.down(act, residual, accumulate=True, ctx=ctx)
