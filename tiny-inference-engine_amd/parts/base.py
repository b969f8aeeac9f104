"""Interfaces of the parts a model is put together from, and their registries.

Five kinds of part exist, each with a registry from a kind name to a class:

* norm          ``forward(ctx, x, rows=None) -> h``
* position      describes or applies a position encoding to queries and keys
* mixer         ``forward(ctx, h, cache, residual)``; declares a cache need
* feed_forward  ``forward(ctx, h, residual)``
* block         ``forward(ctx, x, layer, cache)``: the arrangement of the above

plus the two ends of a model, ``embedding`` and ``head``. A part is built from
the parameters of its PartSpec (sizes, constants, tensor names) and never looks
at the model around it. It declares the tensors it expects (``tensors()``),
takes them at load time (``load``) and runs on a StepContext.

The residual stream is float32 in both compute modes; ``h`` (a norm's output,
a matrix product's input) has the activation dtype of the mode. Mixers and
feed-forwards ADD their result to the ``residual`` tensor they are given, which
lets the last matrix product of a part fold the addition into its epilogue, or
leave it owed to the stream (``StepContext.defer_add``) for the next norm to add
in the pass in which it reads the stream anyway - or, in steps of a few rows,
leave the whole product owed (``StepContext.defer_product``): the norm that
follows then has the product's own epilogue add to the stream and prepare the
norm's output (``Norm.forward(..., lazy=True)``), and no norm kernel runs.
"""

from __future__ import annotations

from typing import Any, Callable, Dict, List, Mapping, Optional

import torch

import dataclasses

from ..errors import InvalidArgument
from ..weights.binder import BFLOAT16, FLOAT32, TensorSpec

@dataclasses.dataclass(frozen=True)
class PartSpec:
    """A registered part kind plus the parameters (sizes, constants, tensor names) it is built with."""

    kind: str
    params: Mapping[str, Any] = dataclasses.field(default_factory=dict)


_KINDS = ("norm", "position", "mixer", "feed_forward", "block", "embedding", "head")
_REGISTRIES: Dict[str, Dict[str, type]] = {k: {} for k in _KINDS}


def register_part(family: str, kind: str, cls: type = None):
    """Registers ``cls`` as the part ``kind`` of ``family``; usable as a decorator."""
    if family not in _REGISTRIES:
        raise InvalidArgument(f"unknown part family '{family}' (families: {', '.join(_KINDS)})")

    def apply(c):
        _REGISTRIES[family][kind] = c
        return c

    return apply(cls) if cls is not None else apply


def unregister_part(family: str, kind: str) -> None:
    _REGISTRIES.get(family, {}).pop(kind, None)


def registered_parts(family: str):
    return tuple(sorted(_REGISTRIES[family]))


def build_part(family: str, spec: PartSpec, **extra):
    """Instantiates the part ``spec`` names from the registry of ``family``."""
    try:
        cls = _REGISTRIES[family][spec.kind]
    except KeyError:
        raise InvalidArgument(
            f"no {family} part is registered as '{spec.kind}' (registered: {', '.join(registered_parts(family)) or 'none'})"
        ) from None
    return cls(dict(spec.params), **extra)


class Part:
    """Base of every part: declared tensors, loading, and nothing else.

    ``capturable`` says whether the part's ``forward`` may be recorded into a HIP graph and replayed
    for later steps: true only if everything that differs between steps is read ON THE DEVICE from
    the step's arrays (``ctx.batch.tokens``, ``positions``, ``state_slots``, a group's block tables:
    they live at fixed addresses) and the launches themselves depend only on the step's shape. A
    part that reads host-side values of the step (``ctx.batch.host_*``), loops over them, or calls
    anything that waits for the GPU (``nonzero``, ``.item()``, ``.cpu()``) must leave it False; a model
    with one such part runs every step eagerly. False is the default, so a part written elsewhere that
    says nothing is never baked into a recording; the parts of this package say True.
    """

    capturable = False
    # True: in a step, what the part launches is the same for every layer of the same shape except for the
    # addresses of the layer's own tensors and cache (no host-side work per layer beyond kernel launches, no
    # torch operations, nothing that depends on which layer it is). The model then runs such layers from the
    # launch list of one of them (``Model._run_alike``). Parts defined elsewhere keep the default.
    replayable = False

    def __init__(self, params: Mapping[str, Any]):
        self.params = dict(params)

    def tensors(self) -> List[TensorSpec]:
        return []

    def load(self, fetch: Callable[[str, str], torch.Tensor], mode: str, device) -> None:
        """Takes the part's tensors: ``fetch(name, role)`` returns the placed device tensor."""

    def children(self) -> List["Part"]:
        return []

    def all_tensors(self) -> List[TensorSpec]:
        out = list(self.tensors())
        for child in self.children():
            out.extend(child.all_tensors())
        return out

    def load_all(self, fetch, mode: str, device) -> None:
        self.load(fetch, mode, device)
        for child in self.children():
            child.load_all(fetch, mode, device)

    def all_capturable(self) -> bool:
        return bool(self.capturable) and all(child.all_capturable() for child in self.children())


class Workspace:
    """Named scratch tensors that live across steps and only ever grow.

    A part asks for ``get(name, shape, dtype)`` each step and receives a view of
    the buffer kept under that name; steady-state steps allocate nothing, and
    the addresses stay put, which replaying a recorded step relies on.
    """

    MAX_VIEWS = 4096      # views kept for reuse; steps of ever new sizes start the memo afresh

    def __init__(self, device):
        self.device = device
        self._buffers: Dict[Any, torch.Tensor] = {}
        self._views: Dict[Any, torch.Tensor] = {}     # (name, dtype, shape) -> view: a layer asks again every step
        self.generation = 0   # grows whenever a buffer is replaced: recorded steps are then stale

    def get(self, name: str, shape, dtype: torch.dtype) -> torch.Tensor:
        shape = tuple(shape)
        view = self._views.get((name, dtype, shape))
        if view is not None:
            return view
        numel = 1
        for d in shape:
            numel *= int(d)
        key = (name, dtype)
        buf = self._buffers.get(key)
        if buf is None or buf.numel() < numel:
            buf = torch.empty(max(numel, 1), dtype=dtype, device=self.device)
            self._buffers[key] = buf
            self.generation += 1
            self._views = {k: v for k, v in self._views.items() if k[:2] != key}     # they showed the old buffer
        if len(self._views) >= self.MAX_VIEWS:
            self._views.clear()
        view = self._views[(name, dtype, shape)] = buf[:numel].view(*shape)
        return view

    def nbytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._buffers.values())


class StepContext:
    """What a part sees of one step: the batch, the mode, scratch memory and the caches."""

    def __init__(self, batch, mode: str, device, workspace: Workspace, cache_manager, cache_plan):
        self.batch = batch
        self.mode = mode
        self.device = device
        self.workspace = workspace
        self.cache_manager = cache_manager
        self.cache_plan = cache_plan
        self.act_dtype = torch.float32 if mode == FLOAT32 else torch.bfloat16
        self.notes: Dict[Any, Any] = {}   # per-step memo shared by parts (e.g. one plan for all layers)
        self._owed = None                  # (target, planes): target += planes[0] + planes[1] + ... is still to be done
        self._pending = None               # (target, linear, x): target += x @ linear.weight^T is still to be launched
        self._row_scales: Dict[int, Any] = {}   # address of rows that lack their norm's 1 / rms -> kernels.RowScale

    @property
    def num_tokens(self) -> int:
        return self.batch.num_tokens

    def scratch(self, name: str, shape, dtype: torch.dtype = None) -> torch.Tensor:
        return self.workspace.get(name, shape, dtype or self.act_dtype)

    # A product cut along K hands its planes of partial sums to the step instead of adding them; the
    # next reader of the target adds them in its own pass (a norm does) or has them added by settle().
    def defer_add(self, target: torch.Tensor, planes: torch.Tensor) -> None:
        self.settle()
        self._owed = (target, planes)

    # A product that ends a sub-layer in a step of a few rows is not even launched by its part: the norm that
    # reads the stream next launches it with an epilogue that adds to the stream and prepares that norm's rows
    # (take_pending_product), or settle() launches it the ordinary way.
    def defer_product(self, target: torch.Tensor, linear, x: torch.Tensor) -> None:
        self.settle()
        self._pending = (target, linear, x)

    def take_pending_product(self, target: torch.Tensor):
        """``(linear, x)`` of the product still to be added to ``target`` (the caller launches it now), or None."""
        if self._pending is None:
            return None
        owed_to, linear, x = self._pending
        if owed_to.data_ptr() == target.data_ptr() and owed_to.shape == target.shape:
            self._pending = None
            return linear, x
        return None

    def launch_pending(self) -> None:
        """Launches a product left pending the ordinary way (it may leave planes of partial sums owed in turn)."""
        if self._pending is not None:
            target, linear, x = self._pending
            self._pending = None
            linear.add_to(self, x, target)

    # Rows that a norm left without their 1 / rms (kernels.RowScale): the products formed from them apply it.
    def set_row_scale(self, rows: torch.Tensor, scale) -> None:
        if scale is None:
            self._row_scales.pop(rows.data_ptr(), None)
        else:
            self._row_scales[rows.data_ptr()] = scale

    def row_scale_of(self, rows: torch.Tensor):
        return self._row_scales.get(rows.data_ptr()) if self._row_scales else None

    def take_owed(self, target: torch.Tensor) -> Optional[torch.Tensor]:
        """The planes still owed to ``target`` (the caller now adds them itself), or None; other debts are settled."""
        self.launch_pending()
        if self._owed is None:
            return None
        owed_to, planes = self._owed
        if owed_to.data_ptr() == target.data_ptr() and owed_to.shape == target.shape:
            self._owed = None
            return planes
        self.settle()
        return None

    def settle(self) -> None:
        self.launch_pending()
        if self._owed is not None:
            from .. import kernels
            target, planes = self._owed
            self._owed = None
            kernels.add_partials(target, planes)

    def cache_of(self, call_index: int):
        """The cache binding of run-order entry ``call_index`` (None if its mixer has no cache)."""
        from ..cache.spec import PagedKV

        entry = self.cache_plan.calls[call_index]
        if entry is None:
            return None
        need = self.cache_plan.groups[entry.group].need
        if isinstance(need, PagedKV):
            k, v = self.cache_manager.kv_planes(entry.group, entry.plane)
            return PagedBinding(need, entry.writes, k, v, self.batch.groups[entry.group],
                                self.cache_manager.block_size)
        return StateBinding(need, entry.writes, self.cache_manager.state_plane(entry.group, entry.plane),
                            self.batch.state_slots)


class PagedBinding:
    """Keys and values of one plane plus this step's slots and block tables of its group."""

    def __init__(self, need, writes, k_cache, v_cache, step, block_size):
        self.need = need
        self.writes = writes
        self.k_cache = k_cache      # [num_blocks, kv_heads, block_size, head_dim]
        self.v_cache = v_cache
        self.step = step            # GroupStep: slot_mapping [T], block_tables [S, MB], ...
        self.block_size = block_size


class StateBinding:
    """The fixed-size states of one plane plus the slot of each sequence of this step."""

    def __init__(self, need, writes, state, state_slots):
        self.need = need
        self.writes = writes
        self.state = state          # [max_state_slots, *shape]
        self.state_slots = state_slots  # int32 [S] on the device


class Norm(Part):
    adds_owed = False   # True: forward() adds partial sums owed to x (ctx.take_owed) in its own pass
    # True: forward() takes ``lazy=True`` and may then return rows without their 1 / rms, registered with
    # ``ctx.set_row_scale``: only for a consumer that applies it (``takes_row_scale``; see ``Block.normed``).
    leaves_row_scale = False

    def forward(self, ctx: StepContext, x: torch.Tensor, rows: Optional[torch.Tensor] = None,
                out_name: str = "norm.out", out_dtype: torch.dtype = None) -> torch.Tensor:
        raise NotImplementedError


class Position(Part):
    """A position encoding applied to queries and keys inside an attention mixer.

    ``rotary_table()`` returns ``(inv_freq float32 [rotary_dim/2], rotary_dim,
    pairing)`` when the encoding is a rotation of pairs by position * inv_freq,
    which the fused kernel applies itself: the first ``rotary_dim`` (even, at
    most head_dim) dimensions of every head are rotated, paired as
    ``(i, i + rotary_dim/2)`` for pairing ``"rotate_half"`` or ``(2i, 2i + 1)``
    for ``"interleaved"``; the other dimensions pass unchanged. ``inv_freq`` None
    means no rotation at all. Any other encoding returns None here and the
    mixer calls ``apply(ctx, q, k, positions)`` on float32 tensors
    ``[T, heads, head_dim]`` instead.
    """

    def rotary_table(self):
        return None

    def angles(self, ctx: "StepContext") -> Optional[torch.Tensor]:
        """Optional: ``[T, rotary_dim]`` float32, cos of the ``rotary_dim/2`` angles then their sines, of this
        step's positions, for the fused kernel (which otherwise computes them per head)."""
        return None

    def apply(self, ctx: StepContext, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor) -> None:
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        """What this mixer needs from the cache: a PagedKV, a FixedState, or None."""
        return None

    def forward(self, ctx: StepContext, h: torch.Tensor, cache, residual: torch.Tensor) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx: StepContext, h: torch.Tensor, residual: torch.Tensor) -> None:
        raise NotImplementedError


class Block(Part):
    """The arrangement of one layer's parts. ``layer`` carries .mixer, .feed_forward and .norms.

    An arrangement settles what is owed to the residual stream before it hands the stream to a part
    that does not add the debt itself (``normed`` does so for norms). ``consumer``: the part the normed rows
    go to and to nothing else; if it says ``takes_row_scale`` (every product it forms from the rows goes through
    ``parts.Linear`` with the step context, or asks ``ctx.row_scale_of`` itself), a norm that can may hand it the
    rows without their 1 / rms.
    """

    @staticmethod
    def normed(ctx: StepContext, norm, x: torch.Tensor, consumer=None) -> torch.Tensor:
        if not norm.adds_owed:
            ctx.settle()
        if getattr(norm, "leaves_row_scale", False) and getattr(consumer, "takes_row_scale", False):
            return norm.forward(ctx, x, lazy=True)
        return norm.forward(ctx, x)

    def forward(self, ctx: StepContext, x: torch.Tensor, layer, cache) -> None:
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ctx: StepContext, token_ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class Head(Part):
    def forward(self, ctx: StepContext, x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


__all__ = [
    "BFLOAT16", "FLOAT32", "Block", "Embedding", "FeedForward", "Head", "Mixer", "Norm", "PagedBinding",
    "Part", "PartSpec", "Position", "StateBinding", "StepContext", "TensorSpec", "Workspace", "build_part",
    "register_part", "registered_parts", "unregister_part",
]
