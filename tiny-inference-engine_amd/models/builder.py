"""From a ModelSpec to a model that can be loaded and stepped.

``Model`` instantiates the parts the spec names, plans the cache from the
mixers' needs and the run order, collects the tensors all parts expect, loads
them through the binder (one error for everything that does not fit) and runs
a step: embedding, the run order, the head on the wanted rows.
"""

from __future__ import annotations

import sys
from typing import Callable, Dict, List, Optional

import torch

from ..cache.spec import CachePlan, plan_cache
from ..config.registry import resolve_architecture
from ..errors import InvalidArgument
from ..parts import base as parts_base
from ..parts.base import StepContext, TensorSpec, build_part
from ..weights.binder import BFLOAT16, check_tensors, normalize_mode, place_tensor
from ..weights.loader import ModelFiles, load_model_folder
from ..weights.safetensors_io import StoredTensor
from .spec import ModelSpec


class LayerParts:
    def __init__(self, spec):
        self.block = build_part("block", spec.block)
        self.mixer = build_part("mixer", spec.mixer)
        self.feed_forward = build_part("feed_forward", spec.feed_forward)
        self.norms = {name: build_part("norm", s) for name, s in spec.norms.items()}
        check = getattr(self.block, "check", None)
        if check is not None:
            check(self.norms)

    def parts(self):
        return [self.block, self.mixer, self.feed_forward, *self.norms.values()]


class Model:
    def __init__(self, spec: ModelSpec, config=None):
        spec.validate()
        self.spec = spec
        self.config = config
        self.embedding = build_part("embedding", spec.embedding)
        self.layers: List[LayerParts] = [LayerParts(s) for s in spec.layers]
        self.head = build_part("head", spec.head)
        self.cache_plan: CachePlan = plan_cache(
            [self.layers[c.layer].mixer.cache_need() for c in spec.order],
            [c.reads_cache_of for c in spec.order])
        self.mode: Optional[str] = None
        self.device = None
        self.layer_hook: Optional[Callable[[int, torch.Tensor], None]] = None

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

    # ------------------------------------------------------------------ step
    def forward(self, ctx: StepContext) -> Optional[torch.Tensor]:
        """Runs the tokens of ``ctx.batch``; returns float32 logits ``[R, vocab]`` or None if none are wanted."""
        batch = ctx.batch
        x = self.embedding.forward(ctx, batch.tokens)
        for index, call in enumerate(self.spec.order):
            layer = self.layers[call.layer]
            layer.block.forward(ctx, x, layer, ctx.cache_of(index))
            if self.layer_hook is not None:
                ctx.settle()
                self.layer_hook(index, x)
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
