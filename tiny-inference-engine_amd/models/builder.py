"""From a ModelSpec to a model that can be loaded and stepped.

``Model`` instantiates the parts the spec names, plans the cache from the
mixers' needs and the run order, collects the tensors all parts expect, loads
them through the binder (one error for everything that does not fit) and runs
a step: embedding, the run order, the head on the wanted rows.
"""

from __future__ import annotations

import dataclasses
import sys
from typing import Callable, Dict, List, Optional

import torch

from ..cache.spec import CachePlan, plan_cache
from ..config.registry import resolve_architecture
from ..errors import InvalidArgument
from .. import kernels
from ..parts import base as parts_base
from ..parts.base import Part, StepContext, TensorSpec, build_part
from ..weights.binder import BFLOAT16, check_tensors, normalize_mode, place_tensor
from ..weights.loader import ModelFiles, load_model_folder
from ..weights.safetensors_io import StoredTensor
from .spec import ModelSpec


def _walk_parts(obj, tensors, classes, seen, scalars=None, path="") -> None:
    """The device tensors ``(address, bytes, shape, dtype)``, the part classes and (``scalars``) the plain values
    ``(path, value)`` - numbers, strings, None - of an object tree, in a fixed order."""
    if isinstance(obj, torch.Tensor):
        if obj.is_cuda:
            tensors.append((obj.data_ptr(), obj.numel() * obj.element_size(), tuple(obj.shape), obj.dtype))
        elif scalars is not None:        # a host tensor (a table of frequencies) is a value like any other
            small = obj.numel() <= 65536
            scalars.append((path, (tuple(obj.shape), str(obj.dtype),
                                   tuple(obj.flatten().tolist()) if small else id(obj))))
    elif isinstance(obj, kernels.PackedWeight):
        blocks = obj.blocks
        tensors.append((blocks.data_ptr(), blocks.numel() * blocks.element_size(), tuple(obj.shape), "packed"))
    elif isinstance(obj, Part):
        if id(obj) in seen:
            return
        seen.add(id(obj))
        classes.append(type(obj))
        for name in sorted(vars(obj)):
            _walk_parts(getattr(obj, name), tensors, classes, seen, scalars, f"{path}.{name}")
    elif isinstance(obj, (list, tuple)):
        for i, value in enumerate(obj):
            _walk_parts(value, tensors, classes, seen, scalars, f"{path}[{i}]")
    elif isinstance(obj, dict):
        for name in sorted(obj, key=str):
            _walk_parts(obj[name], tensors, classes, seen, scalars, f"{path}[{name!r}]")
    elif obj is None or isinstance(obj, (bool, int, float, str)):
        if scalars is not None:
            scalars.append((path, obj))
    elif isinstance(obj, (torch.dtype, torch.device)):
        if scalars is not None:
            scalars.append((path, str(obj)))
    elif dataclasses.is_dataclass(obj) and not isinstance(obj, type):
        if scalars is not None:
            scalars.append((path, type(obj).__name__))
        for field in dataclasses.fields(obj):
            _walk_parts(getattr(obj, field.name), tensors, classes, seen, scalars, f"{path}.{field.name}")
    elif type(obj).__module__.startswith(__name__.split(".")[0] + ".") and hasattr(obj, "__dict__"):
        if id(obj) in seen:          # a helper object of this package that a part holds (a Linear with its weight)
            return
        seen.add(id(obj))
        for name in sorted(vars(obj)):
            _walk_parts(getattr(obj, name), tensors, classes, seen, scalars, f"{path}.{name}")
    elif scalars is not None:
        scalars.append((path, ("object", type(obj).__qualname__, id(obj))))     # unknown: alike only if the very same


def _constants(scalars, tensor_names) -> tuple:
    """What of a layer's plain values must agree for two layers to launch the same kernels with the same numbers:
    everything but the strings that name its tensors (whole names, their parts and prefixes), which differ from
    layer to layer by design."""
    def names_a_tensor(value) -> bool:
        return isinstance(value, str) and value != "" and any(value in name for name in tensor_names)

    return tuple((path, value) for path, value in scalars if not names_a_tensor(value))


class _Launch:
    """One noted kernel launch of a layer and where another layer's pointers go into its arguments."""

    __slots__ = ("fn", "what", "args", "patches")

    def __init__(self, fn, what, args, patches):
        self.fn, self.what, self.args, self.patches = fn, what, args, patches    # patches: (argument, tensor, offset)


class LayerParts:
    def __init__(self, spec):
        self.block = build_part("block", spec.block)
        self.mixer = build_part("mixer", spec.mixer) if spec.mixer is not None else None
        self.feed_forward = build_part("feed_forward", spec.feed_forward) if spec.feed_forward is not None else None
        self.norms = {name: build_part("norm", s) for name, s in spec.norms.items()}
        check = getattr(self.block, "check_layer", None)
        if check is not None:
            check(self)
        else:
            check = getattr(self.block, "check", None)
            if check is not None:
                check(self.norms)

    def parts(self):
        return [p for p in (self.block, self.mixer, self.feed_forward, *self.norms.values()) if p is not None]


class Model:
    def __init__(self, spec: ModelSpec, config=None):
        spec.validate()
        self.spec = spec
        self.config = config
        self.embedding = build_part("embedding", spec.embedding)
        self.layers: List[LayerParts] = [LayerParts(s) for s in spec.layers]
        self.head = build_part("head", spec.head)
        self.cache_plan: CachePlan = plan_cache(
            [self.layers[c.layer].mixer.cache_need() if self.layers[c.layer].mixer is not None else None
             for c in spec.order],
            [c.reads_cache_of for c in spec.order])
        self.mode: Optional[str] = None
        self.device = None
        self.layer_hook: Optional[Callable[[int, torch.Tensor], None]] = None
        # Entries of the run order whose layers have the same shape launch the same kernels with the same numbers
        # and differ only in the addresses of their weights and caches: see _run_alike.
        self.replay_layers = True
        self.layers_replayed = 0                      # entries of the run order run from another's launch list
        self._alike: Dict[int, int] = {}              # first entry of a run of layers alike -> one past its last
        self._layer_tensors: Dict[int, list] = {}     # entry -> (address, bytes) of its layer's device tensors

    # --------------------------------------------------------------- tensors
    def _all_parts(self):
        out = [self.embedding]
        for layer in self.layers:
            out.extend(layer.parts())
        out.append(self.head)
        return out

    def expected_tensors(self) -> List[TensorSpec]:
        specs: List[TensorSpec] = []
        for part in self._all_parts():
            specs.extend(part.all_tensors())
        # A name declared both as required and as optional is required.
        required = {s.name for s in specs if not s.optional}
        return [s for s in specs if not (s.optional and s.name in required)]

    def load(self, tensors: Dict[str, StoredTensor], mode: str, device) -> "Model":
        mode = normalize_mode(mode)
        check_tensors(self.expected_tensors(), tensors, what=f"{self.spec.architecture}")
        placed: Dict[tuple, torch.Tensor] = {}

        def fetch(name: str, role: str) -> torch.Tensor:
            key = (name, role)
            if key not in placed:
                placed[key] = place_tensor(tensors[name], role, mode, device)
            return placed[key]

        for part in self._all_parts():
            part.load_all(fetch, mode, device)
        self.mode = mode
        self.device = device
        self._find_layers_alike()
        wide = sorted(name for (name, role), t in placed.items() if role == "matrix" and t.dtype == torch.float32)
        if mode == BFLOAT16 and wide:
            # Stored in 32 bits (or F16, widened): kept so, and every product over them runs on the float32
            # kernel instead of the matrix cores. Correct, but far slower; say it once, loudly.
            print(f"[tie_amd] WARNING: {len(wide)} weight matrices are not stored as BF16 (first: {wide[0]}); they "
                  f"stay 32-bit and their products run on the float32 kernels, roughly ten times slower than the "
                  f"bfloat16 ones. Convert the checkpoint to BF16 for serving speed.", file=sys.stderr, flush=True)
        return self

    def capturable(self) -> bool:
        """Whether every part allows its launches to be recorded and replayed (see ``Part.capturable``)."""
        return all(part.all_capturable() for part in self._all_parts())

    # ---------------------------------------------------------- layers alike
    MIN_ALIKE = 4     # the first runs as it is, two are noted and compared, the rest replayed: fewer gain nothing

    def _find_layers_alike(self) -> None:
        """Finds runs of consecutive entries of the run order whose layers are of one shape.

        Alike: the same part classes, every one of them ``replayable``, the same parameters and other plain values
        (an eps, a scale, a window: all but the names of tensors), device tensors of the same shapes and dtypes in
        the same places, the same kind of cache binding; each entry a layer of its own, and each with a cache plane
        of its own or all reading one.
        """
        self._alike, self._layer_tensors = {}, {}
        signatures = []
        for index, call in enumerate(self.spec.order):
            tensors, classes, scalars = [], [], []
            layer_parts = self.layers[call.layer].parts()
            _walk_parts(layer_parts, tensors, classes, set(), scalars)
            self._layer_tensors[index] = [(address, size) for address, size, _, _ in tensors]
            entry = self.cache_plan.calls[index]
            binding = None if entry is None else (entry.group, entry.writes)
            ok = all(getattr(c, "replayable", False) for c in classes)
            names = {spec.name for part in layer_parts for spec in part.all_tensors()}
            signatures.append((tuple(classes), tuple(t[2:] for t in tensors), binding, _constants(scalars, names))
                              if ok else None)
        start = 0
        while start < len(signatures):
            end = start + 1
            if signatures[start] is not None:
                layers = {self.spec.order[start].layer}
                while (end < len(signatures) and signatures[end] == signatures[start]
                       and self.spec.order[end].layer not in layers):
                    layers.add(self.spec.order[end].layer)
                    end += 1
            # A tensor is every layer's own or shared by all of them (a table built once): two of the layers
            # sharing one would pass for "the same argument" when their launches are compared.
            for slot in range(len(self._layer_tensors[start])):
                addresses = {self._layer_tensors[i][slot][0] for i in range(start, end)}
                if len(addresses) not in (1, end - start):
                    end = start + 1
                    break
            # The same for the cache: entries that read an earlier entry's plane pass for "the same argument" too.
            planes = {None if self.cache_plan.calls[i] is None else self.cache_plan.calls[i].plane
                      for i in range(start, end)}
            if len(planes) not in (1, end - start):
                end = start + 1
            if end - start >= self.MIN_ALIKE:
                self._alike[start] = end
            start = end

    def _entry_tensors(self, ctx: StepContext, index: int, cache) -> list:
        """(address, bytes) of everything entry ``index`` owns on the device: its layer's tensors and its cache."""
        tensors = list(self._layer_tensors[index])
        for name in ("k_cache", "v_cache", "state"):
            t = getattr(cache, name, None)
            if isinstance(t, torch.Tensor):
                tensors.append((t.data_ptr(), t.numel() * t.element_size()))
        return tensors

    @staticmethod
    def _launch_list(noted_a, noted_b, tensors_a, tensors_b) -> Optional[List[_Launch]]:
        """The launches of one layer as a list another layer of the same shape can run, or None.

        Two layers' noted launches must be the same functions with the same arguments, except where an
        argument is an address inside the same tensor of either layer (a weight, a cache plane) at the same
        offset; anything else that differs means the layers are not alike after all.
        """
        if len(noted_a) != len(noted_b) or not noted_a:
            return None
        launches = []
        for (fn_a, args_a, what), (fn_b, args_b, _) in zip(noted_a, noted_b):
            if fn_a is not fn_b or len(args_a) != len(args_b):
                return None
            patches = []
            for position, (a, b) in enumerate(zip(args_a, args_b)):
                if a == b and type(a) is type(b):
                    continue
                if type(a) is not int or type(b) is not int:
                    return None
                for slot, ((base_a, size_a), (base_b, size_b)) in enumerate(zip(tensors_a, tensors_b)):
                    if 0 <= a - base_a < size_a and a - base_a == b - base_b and size_a == size_b:
                        patches.append((position, slot, a - base_a))
                        break
                else:
                    return None
            launches.append(_Launch(fn_a, what, args_a, tuple(patches)))
        return launches

    def _run_alike(self, ctx: StepContext, x: torch.Tensor, start: int, end: int) -> None:
        """Runs entries ``start`` to ``end`` of the run order, layers of one shape.

        What a layer launches depends on the step (rows, splits, work lists) but not on which of these layers it
        is: only the addresses of its weights and cache differ. So the parts' own code runs for the first three
        (the first may differ: it settles what the entry before it left), the launches of the second and third
        are noted and compared, and the others run from that list with their own addresses, which takes a
        fraction of the host time; small models' steps of many short kernels wait for the host otherwise.
        """
        def run(index):
            cache = ctx.cache_of(index)
            layer = self.layers[self.spec.order[index].layer]
            layer.block.forward(ctx, x, layer, cache)
            return cache

        run(start)
        noted, tensors = [], []
        for index in (start + 1, start + 2):
            record = kernels.start_recording()
            try:
                cache = run(index)
            finally:
                kernels.stop_recording()
            noted.append(record)
            tensors.append(self._entry_tensors(ctx, index, cache))
        launches = self._launch_list(noted[0], noted[1], tensors[0], tensors[1])
        for index in range(start + 3, end):
            if launches is None:
                run(index)
                continue
            own = self._entry_tensors(ctx, index, ctx.cache_of(index))
            for launch in launches:
                if launch.patches:
                    args = list(launch.args)
                    for position, slot, offset in launch.patches:
                        args[position] = own[slot][0] + offset
                    kernels.replay_call(launch.fn, launch.what, args)
                else:
                    kernels.replay_call(launch.fn, launch.what, launch.args)
            self.layers_replayed += 1

    # ------------------------------------------------------------------ step
    def forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """Runs the tokens of ``ctx.batch``; returns float32 logits ``[R, vocab]`` or None if none are wanted."""
        batch = ctx.batch
        x = self.embedding.forward(ctx, batch.tokens)
        index, entries = 0, len(self.spec.order)
        # Layers run from another's launch list only where a layer's launches are its own: in steps of a few rows a
        # sub-layer's last product may stay pending in the step context for the next layer's norm to launch, and a
        # replayed launch list would not carry that over.
        replay = self.replay_layers and self.layer_hook is None and not (
            kernels.NORMS_IN_PRODUCTS and batch.num_tokens <= kernels.NORM_EPILOGUE_ROWS)
        while index < entries:
            alike_to = self._alike.get(index) if replay else None
            if alike_to is not None:
                self._run_alike(ctx, x, index, alike_to)
                index = alike_to
                continue
            layer = self.layers[self.spec.order[index].layer]
            layer.block.forward(ctx, x, layer, ctx.cache_of(index))
            if self.layer_hook is not None:
                ctx.settle()
                self.layer_hook(index, x)
            index += 1
        ctx.settle()     # the last layer's product may still be owed to the stream
        if batch.num_logit_rows == 0:
            return None
        return self.head.forward(ctx, x, batch.logit_rows)


def model_from_config(config_values: dict) -> Model:
    arch = resolve_architecture(config_values)
    config = arch.read_config(config_values)
    return Model(arch.build_spec(config), config)


def expected_tensors_for_config(config_values: dict) -> List[TensorSpec]:
    return model_from_config(config_values).expected_tensors()


def load_model(path, dtype: str = "bfloat16", device="cuda:0") -> Model:
    """Reads a model folder, picks the model class its config.json names, and loads its weights."""
    files: ModelFiles = load_model_folder(path)
    model = model_from_config(files.config_values)
    return model.load(files.tensors, dtype, device)


def load_model_from_tensors(config_values: dict, tensors: Dict[str, torch.Tensor], dtype: str, device) -> Model:
    """Builds a model from tensors already in memory (random weights generated on the device)."""
    stored = {name: StoredTensor.from_tensor(name, t) for name, t in tensors.items()}
    return model_from_config(config_values).load(stored, dtype, device)
