"""Grouped-query attention over the paged cache.

In the reference's order (``src/model/qwen3.cpp:219-231``): q, k, v projections
without bias; per-head RMSNorm of q and k (one weight vector of length
head_dim shared by all heads, the layer's eps) BEFORE the rotation; rotate-half
rotary on q and k; k (normalised, rotated) and raw v written to the cache at
the step's slots; causal attention of every new row over its sequence's cached
keys with ``score = scale * q.k``, query head h reading KV head
``h // (num_heads // num_kv_heads)``; output projection, added to the residual.

Parameters (all from the spec, none assumed): ``hidden``, ``num_heads``,
``num_kv_heads``, ``head_dim``, ``scale``, ``window`` (None = all keys),
``qk_norm`` (None or ``{"eps", "q_weight", "k_weight"}``), ``position`` (a
PartSpec of the position family), ``names`` (``q``, ``k``, ``v``, ``o``) and, for
architectures whose projections have one, ``bias`` (names of bias vectors under ``q``,
``k``, ``v`` - all three or none - and/or ``o``; the reference has none).
"""

from __future__ import annotations

from typing import List, Optional

import torch

from .. import kernels
from ..cache.spec import PagedKV
from ..errors import InvalidArgument
from .base import Mixer, Part, PartSpec, StepContext, TensorSpec, build_part, register_part
from .linear import Linear


@register_part("mixer", "paged_attention")
class PagedAttention(Mixer):
    capturable = True      # reads the step on the device only: may be recorded into a HIP graph
    replayable = True
    takes_row_scale = True   # h goes into the QKV projection only, through Linear with the step context

    def __init__(self, params):
        super().__init__(params)
        self.hidden = int(params["hidden"])
        self.num_heads = int(params["num_heads"])
        self.num_kv_heads = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        self.scale = float(params["scale"])
        self.window: Optional[int] = params.get("window")
        kernels.check_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim)
        names = params["names"]
        q_dim, kv_dim = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        self.q_dim, self.kv_dim = q_dim, kv_dim
        bias = params.get("bias") or {}
        if any(k in bias for k in "qkv") and not all(k in bias for k in "qkv"):
            raise InvalidArgument("the q, k and v projections run as one product: a bias for all three or for none")
        self.qkv = Linear([names["q"], names["k"], names["v"]], [q_dim, kv_dim, kv_dim], self.hidden,
                          bias=[bias["q"], bias["k"], bias["v"]] if "q" in bias else None)
        self.out = Linear([names["o"]], [self.hidden], q_dim, bias=[bias["o"]] if "o" in bias else None)
        self.qk_norm = params.get("qk_norm")
        self.q_norm_weight: torch.Tensor = None
        self.k_norm_weight: torch.Tensor = None
        position: PartSpec = params.get("position") or PartSpec("none")
        self.position = build_part("position", position)

    def children(self) -> List[Part]:
        return [self.position]

    def cache_need(self):
        return PagedKV(self.num_kv_heads, self.head_dim, self.window)

    def tensors(self) -> List[TensorSpec]:
        specs = self.qkv.tensors() + self.out.tensors()
        if self.qk_norm:
            init = ("one_plus_uniform", 0.1)
            specs.append(TensorSpec(self.qk_norm["q_weight"], (self.head_dim,), "vector", init))
            specs.append(TensorSpec(self.qk_norm["k_weight"], (self.head_dim,), "vector", init))
        return specs

    def load(self, fetch, mode, device) -> None:
        self.qkv.load(fetch)
        self.out.load(fetch)
        if self.qk_norm:
            self.q_norm_weight = fetch(self.qk_norm["q_weight"], "vector")
            self.k_norm_weight = fetch(self.qk_norm["k_weight"], "vector")

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: torch.Tensor) -> None:
        T = h.shape[0]
        H, KVH, Dh = self.num_heads, self.num_kv_heads, self.head_dim
        step = cache.step
        eps = float(self.qk_norm["eps"]) if self.qk_norm else 0.0

        width = self.q_dim + 2 * self.kv_dim
        q = ctx.scratch("attention.q", (T, self.q_dim))
        table = self.position.rotary_table()
        # Decode-size steps: the projection comes as planes of partial sums, added by the kernel that reads them.
        planes = self.qkv.partial_planes(ctx, h, "attention.qkv") if table is not None else None
        if planes is not None:
            qkv = planes[0]
        else:
            qkv = ctx.scratch("attention.qkv", (T, width), torch.float32)
            self.qkv(h, qkv, ctx=ctx)
        if table is not None:
            inv_freq, rotary_dim, pairing = table
            if (inv_freq is not None and rotary_dim == Dh and pairing == "rotate_half"
                    and kernels.decode_attention_prepares(ctx.batch, q.dtype, cache.k_cache, H)):
                # A step of single decoded tokens: the attention kernel sums the planes, norms and rotates its own
                # queries and writes the newest keys and values itself: one kernel less.
                attn = ctx.scratch("attention.out", (T, self.q_dim))
                kernels.paged_attention_prepared(
                    planes if planes is not None else qkv.unsqueeze(0),
                    self.q_norm_weight if self.qk_norm else None, self.k_norm_weight if self.qk_norm else None, eps, self.position.angles(ctx), cache.writes, cache.k_cache, cache.v_cache, attn, step, ctx.batch,
                    H, self.scale, self.window, ctx.scratch)
                self.out(attn, residual, accumulate=True, ctx=ctx)
                return
            if inv_freq is None:                      # an encoding that leaves queries and keys as they are
                rotary_dim, pairing = None, "rotate_half"
            kernels.qk_norm_rope_kv_write(
                qkv, q, self.q_norm_weight, self.k_norm_weight, eps, inv_freq, ctx.batch.positions,
                step.slot_mapping, cache.k_cache, cache.v_cache, H, KVH, Dh, cache.block_size,
                write_kv=cache.writes, planes=1 if planes is None else planes.shape[0], plane_stride=T * width,
                angles=self.position.angles(ctx) if inv_freq is not None else None,
                rotary_dim=rotary_dim, pairing=pairing)
        else:
            # A position encoding that is no rotation table: normalise in place, let the part
            # change q and k (float32 views into the projection rows), then convert and store.
            q_view = qkv[:, :self.q_dim]
            k_view = qkv[:, self.q_dim:self.q_dim + self.kv_dim]
            if self.qk_norm:
                kernels.qk_norm_rope_kv_write(
                    qkv, q_view, self.q_norm_weight, self.k_norm_weight, eps, None, ctx.batch.positions,
                    None, None, None, H, KVH, Dh, cache.block_size, write_kv=False, k_dense=k_view)
            self.position.apply(ctx, q_view.unflatten(1, (H, Dh)), k_view.unflatten(1, (KVH, Dh)),
                                ctx.batch.positions)
            kernels.qk_norm_rope_kv_write(
                qkv, q, None, None, 0.0, None, ctx.batch.positions, step.slot_mapping, cache.k_cache,
                cache.v_cache, H, KVH, Dh, cache.block_size, write_kv=cache.writes)

        attn = ctx.scratch("attention.out", (T, self.q_dim))
        kernels.paged_attention(q, cache.k_cache, cache.v_cache, attn, step, ctx.batch, H, self.scale, self.window,
                                scratch=ctx.scratch)
        self.out(attn, residual, accumulate=True, ctx=ctx)
