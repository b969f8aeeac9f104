"""Random-weights mode: a model folder from a configuration and a seed.

The tensors are exactly those the architecture's parts expect (names, shapes
and roles come from their TensorSpecs), so a folder written here loads through
the ordinary loader. Matrices and embedding tables are drawn from N(0, std),
norm weights from 1 + U(-w, w); the defaults (0.02 and 0.1) are the ones the
benchmark configurations name. Each tensor has its own stream, keyed by the
seed and the tensor's name, so its values do not depend on the order or the
number of the other tensors. The reference has random weights only in its
tests (``tests/support/tiny_model.h:66-93``).
"""

from __future__ import annotations

import hashlib
import json
import pathlib
from typing import Iterator, List, Tuple

import torch

from ..errors import InvalidArgument
from .binder import TensorSpec
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16,
          "bf16": torch.bfloat16, "fp32": torch.float32, "f32": torch.float32}


def _stream_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & (2 ** 63 - 1)


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    """One tensor of the random model, drawn in float32 and rounded once to ``dtype``."""
    gen = torch.Generator(device=device)
    gen.manual_seed(_stream_seed(seed, spec.name))
    kind = spec.init[0]
    if spec.role == "int_table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if kind == "normal":
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, float(spec.init[1]), generator=gen)
    elif kind == "one_plus_uniform":
        w = float(spec.init[1])
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).uniform_(-w, w, generator=gen).add_(1.0)
    elif kind == "zeros":
        t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
    else:
        raise InvalidArgument(f"tensor '{spec.name}' has unknown init '{kind}'")
    return t.to(dtype)


def random_tensors(specs: List[TensorSpec], seed: int, dtype: torch.dtype, device="cpu",
                   vector_dtype: torch.dtype = None) -> Iterator[Tuple[str, torch.Tensor]]:
    seen = set()
    for spec in specs:
        if spec.optional or spec.name in seen:
            continue
        seen.add(spec.name)
        store = dtype if spec.role == "matrix" else (vector_dtype or dtype)
        yield spec.name, random_tensor(spec, seed, store, device)


def write_random_model(folder, config_values: dict, seed: int, dtype: str = "bfloat16", device="cpu") -> str:
    """Writes ``config.json`` and ``model.safetensors`` for the architecture config_values names."""
    from ..models.builder import expected_tensors_for_config

    if dtype not in _STORE:
        raise InvalidArgument(f"weights can be written as bfloat16, float16 or float32, got '{dtype}'")
    store = _STORE[dtype]
    specs = [s for s in expected_tensors_for_config(config_values) if not s.optional]
    folder = pathlib.Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(dict(config_values), indent=2) + "\n")
    declared, seen = [], set()
    for s in specs:
        if s.name in seen:
            continue
        seen.add(s.name)
        declared.append((s.name, tuple(s.shape), torch.int32 if s.role == "int_table" else store))
    write_safetensors(folder / "model.safetensors", random_tensors(specs, seed, store, device),
                      shapes_and_dtypes=declared, metadata={"format": "pt", "seed": seed})
    return str(folder)
