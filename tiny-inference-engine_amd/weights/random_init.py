"""Random-weights mode: a model folder from a configuration and a seed.

The tensors are exactly those the architecture's parts expect (names, shapes
and roles come from their TensorSpecs), so a folder written here loads through
the ordinary loader. Matrices and embedding tables are drawn from N(0, std),
norm weights from 1 + U(-w, w); the defaults (0.02 and 0.1) are the ones the
benchmark configurations name. Each tensor has its own stream, keyed by the
seed and the tensor's name, and an element is a function of (that key, its
index) alone: its values depend neither on the other tensors nor on where
they are drawn. The host draws them with numpy and the GPU with a kernel
(``kernels.random_fill``) through the same sequence of IEEE double
operations, so a folder written on the host, a model built on the GPU and a
test's copy of one tensor are the same bits for one seed. The reference has
random weights only in its tests (``tests/support/tiny_model.h:66-93``).

The recipe: ``z = mix64(key + (i + 1) * 0x9E3779B97F4A7C15)`` (SplitMix64),
``u = ((z >> 12) + 0.5) * 2**-52`` in (0, 1), and for a normal value the
inverse normal distribution function of ``u`` by Wichura's algorithm AS 241
(PPND16), whose logarithm is a fixed series here so that no library routine
with its own rounding takes part.
"""

from __future__ import annotations

import hashlib
import json
import pathlib
from typing import Iterator, List, Tuple

import numpy as np
import torch

from ..errors import InvalidArgument
from .binder import TensorSpec
from .safetensors_io import write_safetensors

_STORE = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16,
          "bf16": torch.bfloat16, "fp32": torch.float32, "f32": torch.float32}


def _stream_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & (2 ** 63 - 1)


_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_CHUNK = 1 << 22          # elements drawn at a time on the host


def _uniform(key: int, first: int, count: int) -> np.ndarray:
    """u of elements ``first`` .. ``first + count - 1`` of the stream ``key``, float64 in (0, 1)."""
    with np.errstate(over="ignore"):
        z = np.uint64(key) + (np.arange(first + 1, first + count + 1, dtype=np.uint64)) * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return ((z >> np.uint64(12)).astype(np.float64) + 0.5) * 2.0 ** -52


def _log(x: np.ndarray) -> np.ndarray:
    """log(x) for x in (0, 1) by 2 atanh((m - 1) / (m + 1)) + e ln 2: additions, products and quotients only."""
    m, e = np.frexp(x)
    low = m < 0.70710678118654752440
    m = np.where(low, m * 2.0, m)
    e = np.where(low, e - 1, e)
    s = (m - 1.0) / (m + 1.0)
    s2 = s * s
    series = np.full_like(s, 1.0 / 27.0)
    for odd in range(25, 0, -2):
        series = series * s2 + 1.0 / odd
    return 2.0 * s * series + e.astype(np.float64) * 0.69314718055994530942


def _poly(c, r: np.ndarray) -> np.ndarray:
    v = np.full_like(r, c[7])
    for k in range(6, -1, -1):
        v = v * r + c[k]
    return v


_A = (3.3871328727963666080, 1.3314166789178437745e2, 1.9715909503065514427e3, 1.3731693765509461125e4,
      4.5921953931549871457e4, 6.7265770927008700853e4, 3.3430575583588128105e4, 2.5090809287301226727e3)
_B = (1.0, 4.2313330701600911252e1, 6.8718700749205790830e2, 5.3941960214247511077e3, 2.1213794301586595867e4,
      3.9307895800092710610e4, 2.8729085735721942674e4, 5.2264952788528545610e3)
_C = (1.42343711074968357734, 4.63033784615654529590, 5.76949722146069140550, 3.64784832476320460504,
      1.27045825245236838258, 2.41780725177450611770e-1, 2.27238449892691845833e-2, 7.74545014278341407640e-4)
_D = (1.0, 2.05319162663775882187, 1.67638483018380384940, 6.89767334985100004550e-1, 1.48103976427480074590e-1,
      1.51986665636164571966e-2, 5.47593808499534494600e-4, 1.05075007164441684324e-9)
_E = (6.65790464350110377720, 5.46378491116411436990, 1.78482653991729133580, 2.96560571828504891230e-1,
      2.65321895265761230930e-2, 1.24266094738807843860e-3, 2.71155556874348757815e-5, 2.01033439929228813265e-7)
_F = (1.0, 5.99832206555887937690e-1, 1.36929880922735805310e-1, 1.48753612908506148525e-2,
      7.86869131145613259100e-4, 1.84631831751005468180e-5, 1.42151175831644588870e-7, 2.04426310338993978564e-15)


def _normal_of(p: np.ndarray) -> np.ndarray:
    """The inverse normal distribution function (Wichura 1988, algorithm AS 241, PPND16), step for step what
    ``random_normal_of`` of csrc/elementwise.hip computes."""
    q = p - 0.5
    out = np.empty_like(p)
    central = np.abs(q) <= 0.425
    qc = q[central]
    r = 0.180625 - qc * qc
    out[central] = qc * _poly(_A, r) / _poly(_B, r)
    tail = ~central
    if tail.any():
        pt, qt = p[tail], q[tail]
        r = np.sqrt(-_log(np.where(qt < 0.0, pt, 1.0 - pt)))
        near = r <= 5.0
        rn, rf = r - 1.6, r - 5.0
        with np.errstate(all="ignore"):           # each branch is evaluated for all, kept where it applies
            v = np.where(near, _poly(_C, rn) / _poly(_D, rn), _poly(_E, rf) / _poly(_F, rf))
        out[tail] = np.where(qt < 0.0, -v, v)
    return out


def _draw_on_host(key: int, count: int, kind: str, scale: float) -> torch.Tensor:
    out = np.empty(count, dtype=np.float32)
    for first in range(0, count, _CHUNK):
        n = min(_CHUNK, count - first)
        u = _uniform(key, first, n)
        v = scale * _normal_of(u) if kind == "normal" else 1.0 + scale * (2.0 * u - 1.0)
        out[first:first + n] = v.astype(np.float32)
    return torch.from_numpy(out)


def random_tensor(spec: TensorSpec, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    """One tensor of the random model, drawn in float64, rounded to float32 and then once to ``dtype``; the same
    bits on the host and on a GPU."""
    kind = spec.init[0]
    if spec.role == "int_table":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if kind == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    if kind not in ("normal", "one_plus_uniform"):
        raise InvalidArgument(f"tensor '{spec.name}' has unknown init '{kind}'")
    key, scale = _stream_seed(seed, spec.name), float(spec.init[1])
    count = 1
    for d in spec.shape:
        count *= int(d)
    if torch.device(device).type == "cpu":
        return _draw_on_host(key, count, kind, scale).view(*spec.shape).to(dtype)
    from .. import kernels

    t = torch.empty(spec.shape, dtype=torch.float32, device=device)
    kernels.random_fill(t, key, kind, scale)
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
