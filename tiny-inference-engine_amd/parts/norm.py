"""RMSNorm: ``out = (x * inv) * w`` with ``inv = 1 / sqrt(mean(x^2) + eps)``.

The weight multiplies after normalisation and is the plain ``w`` (not ``1 + w``);
no bias, no mean subtraction; statistics in float32
(``src/backend/cpu/cpu_backend.cpp:141-159``). Parameters: ``dim``, ``eps``,
``weight`` (tensor name).
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from .base import Norm, StepContext, TensorSpec, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    adds_owed = True
    leaves_row_scale = True

    def __init__(self, params):
        super().__init__(params)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])
        self.weight_name = params["weight"]
        self.weight: torch.Tensor = None

    def tensors(self) -> List[TensorSpec]:
        return [TensorSpec(self.weight_name, (self.dim,), "vector", ("one_plus_uniform", 0.1))]

    def load(self, fetch, mode, device) -> None:
        self.weight = fetch(self.weight_name, "vector")

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                out_name: str = "norm.out", out_dtype: torch.dtype = None, lazy: bool = False) -> torch.Tensor:
        """``lazy``: the caller's consumer applies a row scale (``Block.normed``). If the product that ends the
        sub-layer before is still pending, it is launched here with an epilogue that adds it to ``x`` and leaves
        ``x * weight`` and the rows' sums of squares: the result lacks its ``1 / rms``, which the consumer's
        products apply (``ctx.row_scale_of``), and no norm kernel runs."""
        count = x.shape[0] if rows is None else rows.numel()
        out = ctx.scratch(out_name, (count, self.dim), out_dtype or ctx.act_dtype)
        if lazy and rows is None and out.dtype == torch.bfloat16 and self.dim % 16 == 0:
            pending = ctx.take_pending_product(x)
            if pending is not None:
                linear, rows_in = pending
                squares = ctx.scratch(out_name + ".squares", (count, self.dim // 16), torch.float32)
                linear.add_to_and_prepare_norm(rows_in, x, self.weight, out, squares)
                ctx.set_row_scale(out, kernels.RowScale(squares, self.dim, self.eps))
                return out
        ctx.set_row_scale(out, None)
        owed = ctx.take_owed(x)
        if owed is not None and rows is None:
            kernels.add_partials(x, owed, self.weight, self.eps, out)   # x += owed sums; out = norm(x), one pass
            return out
        if owed is not None:
            kernels.add_partials(x, owed)
        kernels.rms_norm(x, self.weight, self.eps, out, rows)
        return out
