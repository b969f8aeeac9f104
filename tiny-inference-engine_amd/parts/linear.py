"""A projection ``out = x @ W^T`` whose weight may be several stored matrices side by side.

Weights keep their stored ``[out, in]`` layout (``src/model/qwen3.cpp:81-90``).
Listing several names concatenates them along the output dimension at load
time (q, k, v or gate, up in one product): the arithmetic of each output
column is unchanged, the activation is read once instead of several times.
The reference's projections have no bias; ``bias`` names one vector per weight for architectures that have
(added by a kernel of its own after the product, which then is neither cut into planes nor left pending).
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from .. import kernels
from ..errors import InvalidArgument
from ..weights.binder import TensorSpec


class Linear:
    def __init__(self, names: Sequence[str], out_features: Sequence[int], in_features: int, init_std: float = 0.02,
                 bias: Optional[Sequence[str]] = None):
        if len(names) != len(out_features) or not names:
            raise InvalidArgument("a projection needs one output size per weight name")
        if bias is not None and len(bias) != len(names):
            raise InvalidArgument("a projection with a bias needs one bias name per weight name")
        self.names = list(names)
        self.bias_names = list(bias) if bias is not None else None
        self.bias: Optional[torch.Tensor] = None          # float32 [total_out], the stored vectors side by side
        self.out_features = list(out_features)
        self.in_features = in_features
        self.init_std = init_std
        self.weight: torch.Tensor = None
        self._splits = None
        self._tiled_splits = {}

    @property
    def total_out(self) -> int:
        return sum(self.out_features)

    def tensors(self) -> List[TensorSpec]:
        specs = [TensorSpec(n, (o, self.in_features), "matrix", ("normal", self.init_std))
                 for n, o in zip(self.names, self.out_features)]
        if self.bias_names is not None:
            specs += [TensorSpec(b, (o,), "vector", ("normal", self.init_std))
                      for b, o in zip(self.bias_names, self.out_features)]
        return specs

    def load(self, fetch) -> None:
        if self.bias_names is not None:
            self.bias = torch.cat([fetch(b, "vector").to(torch.float32) for b in self.bias_names]).contiguous()
        parts = [fetch(n, "matrix") for n in self.names]
        if len(parts) == 1:
            self.set_weight(parts[0])
            return
        dtypes = {p.dtype for p in parts}
        if len(dtypes) > 1:  # stored in different widths: the wider one decides
            parts = [p.to(torch.float32) for p in parts]
        self.set_weight(torch.cat(parts, dim=0).contiguous())

    def set_weight(self, w: torch.Tensor) -> None:
        """Keeps ``w`` (``[out, in]``), in the matrix cores' blocked layout where the bfloat16 products can read that."""
        self.weight = kernels.pack_weight(w) if kernels.packable(w) else w

    def __call__(self, x: torch.Tensor, out: torch.Tensor, accumulate: bool = False, ctx=None) -> torch.Tensor:
        """out (+)= x @ W^T. With ``ctx`` an accumulating product may leave its addition owed to ``out``.

        In a step of a few rows the whole product is left pending: the norm that reads ``out`` next launches it
        with the norm's work in its epilogue (``add_to_and_prepare_norm``), or ``ctx.settle()`` launches it the
        ordinary way. Otherwise a decode-size product over a weight of few rows is cut along K into planes of
        partial sums; the step context remembers that their sum is still to be added, and the next norm over
        ``out`` (or ``ctx.settle()``) adds it. Callers that pass no context always get the sum at once. With
        ``ctx``, rows ``x`` that lack their norm's 1 / rms (``ctx.row_scale_of``) have it applied to the sums.
        """
        if self.bias is not None:
            if ctx is not None:
                ctx.settle()                      # what is still owed to ``out`` lands before this adds to it
            kernels.linear(x, self.weight, out, accumulate, row_scale=self.row_scale_for(ctx, x, self.weight))
            kernels.add_bias(out, self.bias)
            return out
        if ctx is not None and accumulate and out.dtype == torch.float32:
            if self.prepares_norms(x):
                ctx.defer_product(out, self, x)
                return out
            return self.add_to(ctx, x, out)
        kernels.linear(x, self.weight, out, accumulate, row_scale=self.row_scale_for(ctx, x, self.weight))
        return out

    def prepares_norms(self, x: torch.Tensor) -> bool:
        """Whether the decode product takes this product with the next norm's work in its epilogue."""
        w = self.weight
        return kernels.NORMS_IN_PRODUCTS and x.dtype == torch.bfloat16 and isinstance(w, kernels.PackedWeight) and \
            x.is_cuda and x.shape[0] <= kernels.norm_epilogue_rows(w.shape[0], w.shape[1])

    def add_to(self, ctx, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out += x @ W^T now, or as planes of partial sums owed to ``out``."""
        # An earlier product's planes may still be owed and live in the buffer the new planes take:
        # add them before they are overwritten (after a norm that took the debt this does nothing).
        ctx.settle()
        planes = self.partial_planes(ctx, x, "linear.partials")
        if planes is not None:
            ctx.defer_add(out, planes)
            return out
        kernels.linear(x, self.weight, out, True, row_scale=self.row_scale_for(ctx, x, self.weight))
        return out

    def add_to_and_prepare_norm(self, x: torch.Tensor, out: torch.Tensor, norm_weight: torch.Tensor,
                                next_rows: torch.Tensor, squares: torch.Tensor) -> None:
        """out += x @ W^T in one plane, and in the same epilogue ``next_rows = bfloat16(out * norm_weight)`` and the
        sums of ``out ** 2`` per 16-column tile (``prepares_norms`` says whether this product can)."""
        kernels.skinny_gemm_bf16(x, self.weight, out, accumulate=True, next_norm=(norm_weight, next_rows, squares))

    @staticmethod
    def row_scale_for(ctx, x: torch.Tensor, weight):
        """The factor that rows ``x`` still lack, if the product about to run can apply it; otherwise it is applied
        to the rows themselves first."""
        scale = ctx.row_scale_of(x) if ctx is not None else None
        if scale is not None and not kernels.applies_row_scale(x, weight):
            kernels.scale_rows(x, scale)
            ctx.set_row_scale(x, None)
            return None
        return scale

    def partial_planes(self, ctx, x: torch.Tensor, name: str):
        """Runs the product as ``[S, M, N]`` float32 planes of partial sums if that is the faster way; else None.

        The decode product decides by the weight's shape alone up to 16 rows and by its plan for the number of rows
        above (up to 32 rows, or 64 where the tiled product is not the faster); the tiled product is cut along K
        when its tiles alone would leave most of the GPU idle.
        """
        M, K = x.shape
        w = self.weight
        if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or K % 8 or self.bias is not None:
            return None
        decode_product = kernels.decode_product_rows(M, w)
        if decode_product:
            if M <= 16 or not isinstance(w, kernels.PackedWeight):
                if self._splits is None:
                    self._splits = kernels.skinny_splits(w.shape[0], K)
                splits = self._splits
            else:
                splits = kernels.few_rows_plan(M, w.shape[0], K)[2]
        else:
            splits = self._tiled_splits.get(M)
            if splits is None:
                splits = self._tiled_splits[M] = kernels.gemm_splits(M, w.shape[0], K, isinstance(w, kernels.PackedWeight))
        if splits <= 1:
            return None
        planes = ctx.scratch(name, (splits, M, w.shape[0]), torch.float32)
        scale = self.row_scale_for(ctx, x, w)
        if decode_product:
            kernels.skinny_gemm_bf16(x, w, planes, splits=splits, row_scale=scale)
        else:
            kernels.gemm_bf16(x, w, planes, splits=splits)      # above the rows a scale travels with: none here
        return planes
