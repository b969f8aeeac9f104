"""Matching the tensors a model expects with the tensors a file holds.

Parts declare what they expect as TensorSpecs. ``check_tensors`` compares all of
them with the stored table at once and raises ONE LoadError that lists every
missing tensor, every tensor no part uses, every wrong shape and every dtype
that cannot be used - the reference stops at the first
(``src/model/qwen3.cpp:47-71,102-106``); the rules are the same: exact shapes,
float matrices and vectors only, nothing left over.

``place_tensor`` is the dtype policy on the way to the device:
  * matrices stored as BF16 stay BF16; matrices stored in 32-bit stay 32-bit
    (F16 is widened to F32, which is exact); in float32 mode everything is
    widened to F32;
  * vectors (norm weights) always become F32, as in ``qwen3.cpp:60-71``;
  * integer tables become int32.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, Iterable, List, Tuple

import torch

from ..errors import InvalidArgument, LoadError
from .safetensors_io import StoredTensor

_FLOAT = ("F32", "F16", "BF16")
_INT = ("I32", "I64")

FLOAT32 = "float32"
BFLOAT16 = "bfloat16"


def normalize_mode(mode: str) -> str:
    """Accepts the spellings of the two compute modes; anything else is an InvalidArgument."""
    names = {"float32": FLOAT32, "fp32": FLOAT32, "f32": FLOAT32,
             "bfloat16": BFLOAT16, "bf16": BFLOAT16}
    if mode not in names:
        raise InvalidArgument(f"dtype must be bfloat16 or float32, got '{mode}'")
    return names[mode]


@dataclasses.dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: Tuple[int, ...]
    role: str = "matrix"                     # "matrix", "vector" or "int_table"
    init: Tuple = ("normal", 0.02)           # how random-weights mode fills it
    optional: bool = False                   # may be absent; if present it is shape-checked


def check_tensors(expected: Iterable[TensorSpec], stored: Dict[str, StoredTensor], what: str = "the model") -> None:
    expected = list(expected)
    missing: List[str] = []
    wrong_shape: List[str] = []
    wrong_dtype: List[str] = []
    known = set()
    for spec in expected:
        if spec.name in known:
            continue
        known.add(spec.name)
        tensor = stored.get(spec.name)
        if tensor is None:
            if not spec.optional:
                missing.append(spec.name)
            continue
        if tuple(tensor.shape) != tuple(spec.shape):
            wrong_shape.append(f"{spec.name}: has {list(tensor.shape)}, expected {list(spec.shape)}")
        allowed = _INT if spec.role == "int_table" else _FLOAT
        if tensor.dtype not in allowed:
            wrong_dtype.append(f"{spec.name}: has {tensor.dtype}, expected one of {', '.join(allowed)}")
    unexpected = sorted(name for name in stored if name not in known)
    if not (missing or wrong_shape or wrong_dtype or unexpected):
        return
    lines = [f"the tensors of the model file do not fit {what}:"]
    if missing:
        lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
    if unexpected:
        lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
    if wrong_shape:
        lines.append(f"  wrong shape ({len(wrong_shape)}): " + "; ".join(wrong_shape))
    if wrong_dtype:
        lines.append(f"  wrong dtype ({len(wrong_dtype)}): " + "; ".join(wrong_dtype))
    raise LoadError("\n".join(lines))


def place_tensor(tensor: StoredTensor, role: str, mode: str, device) -> torch.Tensor:
    """Uploads a stored tensor to ``device`` in the dtype the policy above gives it."""
    data = tensor.torch()
    if role == "int_table":
        if data.dtype == torch.int64:
            if data.numel() and (int(data.max()) > 2 ** 31 - 1 or int(data.min()) < -2 ** 31):
                raise LoadError(f"integer table '{tensor.name}' has values outside int32")
        return data.to(device=device, dtype=torch.int32).contiguous()
    if role == "vector" or mode == FLOAT32:
        return data.to(device=device).to(torch.float32).contiguous()
    if role != "matrix":
        raise InvalidArgument(f"unknown tensor role '{role}'")
    if data.dtype == torch.bfloat16:
        return data.to(device=device).contiguous()
    return data.to(device=device).to(torch.float32).contiguous()
