"""Reading and writing the safetensors container.

Layout: an 8-byte little-endian header length, a JSON header
``{name: {dtype, shape, data_offsets: [begin, end]}, "__metadata__": ...}``, then
the raw tensor bytes; offsets count from the end of the header. The checks on
the header follow ``src/model/safetensors.cpp:22-85`` of the reference: every
failure is a LoadError that names the file and the tensor. Tensor bytes are
memory-mapped and never copied here.
"""

from __future__ import annotations

import dataclasses
import json
import mmap
import pathlib
import struct
from typing import Dict, Iterable, Iterator, Tuple

import torch

from ..errors import LoadError, UnsupportedError

# safetensors dtype name -> (torch dtype, bytes per element)
_DTYPES = {
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
_NAMES = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
          torch.int32: "I32", torch.int64: "I64"}
_INT64_MAX = 2 ** 63 - 1


@dataclasses.dataclass(frozen=True)
class StoredTensor:
    """One tensor of a model file: its stored dtype and shape and where its bytes lie."""

    name: str
    dtype: str                   # "F32", "F16", "BF16", "I32", "I64"
    shape: Tuple[int, ...]
    source: str                  # file the bytes come from, for error messages
    _buffer: object = dataclasses.field(repr=False, default=None)
    _offset: int = 0
    _tensor: object = dataclasses.field(repr=False, default=None)

    @property
    def numel(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    def torch(self) -> torch.Tensor:
        """A CPU tensor in the stored dtype; a view of the mapped file, not a copy."""
        if self._tensor is not None:
            return self._tensor
        dtype, _ = _DTYPES[self.dtype]
        if self.numel == 0:
            return torch.empty(self.shape, dtype=dtype)
        flat = torch.frombuffer(self._buffer, dtype=dtype, count=self.numel, offset=self._offset)
        return flat.view(self.shape)

    @classmethod
    def from_tensor(cls, name: str, tensor: torch.Tensor, source: str = "<memory>") -> "StoredTensor":
        """Wraps a tensor that is already in memory (on any device) as a stored tensor."""
        if tensor.dtype not in _NAMES:
            raise UnsupportedError(f"tensor '{name}' has dtype {tensor.dtype} (supported: {', '.join(_DTYPES)})")
        return cls(name, _NAMES[tensor.dtype], tuple(tensor.shape), source, None, 0, tensor)


class SafetensorsFile:
    """The parsed header of one .safetensors file over a private read-only mapping."""

    def __init__(self, path):
        self.path = pathlib.Path(path)
        where = str(self.path)
        try:
            with open(self.path, "rb") as f:
                size = f.seek(0, 2)
                if size < 8:
                    raise LoadError(f"{where}: truncated: no header length")
                # Copy-on-write mapping: nothing is copied or written, but the
                # pages count as writable, which torch.frombuffer asks for.
                self._map = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
        except OSError as e:
            raise LoadError(f"cannot read {where}: {e.strerror or e}") from None
        (header_len,) = struct.unpack_from("<Q", self._map, 0)
        if header_len > size - 8:
            raise LoadError(f"{where}: header length {header_len} runs past the end of the {size}-byte file")
        data_start = 8 + header_len
        data_size = size - data_start
        try:
            header = json.loads(bytes(self._map[8:data_start]).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise LoadError(f"{where}: header is not valid JSON: {e}") from None
        if not isinstance(header, dict):
            raise LoadError(f"{where}: header is not a JSON object")

        self.metadata = header.get("__metadata__") or {}
        self.tensors: Dict[str, StoredTensor] = {}
        for name, entry in header.items():
            if name == "__metadata__":
                continue
            if not isinstance(entry, dict):
                raise LoadError(f"{where}: malformed header entry for '{name}'")
            dtype = entry.get("dtype")
            if not isinstance(dtype, str):
                raise LoadError(f"{where}: malformed header entry for '{name}': no dtype")
            if dtype not in _DTYPES:
                raise UnsupportedError(
                    f"{where}: tensor '{name}' has dtype {dtype} (supported: {', '.join(_DTYPES)})")
            dims = entry.get("shape")
            if not isinstance(dims, list) or not all(isinstance(d, int) and not isinstance(d, bool) for d in dims):
                raise LoadError(f"{where}: malformed header entry for '{name}': bad shape")
            if not dims:
                dims = [1]  # scalars are stored with shape []
            numel = 1
            for d in dims:
                if d < 0:
                    raise LoadError(f"{where}: tensor '{name}' has an invalid or overflowing shape")
                numel *= d
                if numel > _INT64_MAX:
                    raise LoadError(f"{where}: tensor '{name}' has an invalid or overflowing shape")
            if len(dims) > 4:
                raise LoadError(f"{where}: tensor '{name}' has an unsupported shape: {len(dims)} dimensions")
            offsets = entry.get("data_offsets")
            if (not isinstance(offsets, list) or len(offsets) != 2
                    or not all(isinstance(o, int) and not isinstance(o, bool) and o >= 0 for o in offsets)
                    or offsets[1] < offsets[0]):
                raise LoadError(f"{where}: tensor '{name}' has bad data_offsets")
            if offsets[1] > data_size:
                raise LoadError(f"{where}: tensor '{name}' extends past the end of the file")
            nbytes = offsets[1] - offsets[0]
            need = numel * _DTYPES[dtype][1]
            if need != nbytes:
                raise LoadError(
                    f"{where}: tensor '{name}' {dtype} {dims} needs {need} bytes but its data_offsets span {nbytes}")
            self.tensors[name] = StoredTensor(name, dtype, tuple(dims), where, self._map, data_start + offsets[0])


def read_safetensors(path) -> Dict[str, StoredTensor]:
    return SafetensorsFile(path).tensors


def write_safetensors(path, tensors: Iterable[Tuple[str, torch.Tensor]], shapes_and_dtypes=None,
                      metadata=None) -> None:
    """Writes tensors to ``path`` in the order given.

    ``tensors`` is consumed twice unless ``shapes_and_dtypes`` (a list of
    ``(name, shape, torch dtype)`` in the same order) is given, in which case it
    may be a one-shot generator: the header is written first from the
    declarations and the data is streamed after it, one tensor in memory at a time.
    """
    if shapes_and_dtypes is None:
        tensors = list(tensors)
        shapes_and_dtypes = [(n, tuple(t.shape), t.dtype) for n, t in tensors]
    header = {}
    offset = 0
    for name, shape, dtype in shapes_and_dtypes:
        if dtype not in _NAMES:
            raise UnsupportedError(f"cannot store tensor '{name}' of dtype {dtype}")
        if name in header:
            raise LoadError(f"duplicate tensor '{name}'")
        numel = 1
        for d in shape:
            numel *= d
        nbytes = numel * _DTYPES[_NAMES[dtype]][1]
        header[name] = {"dtype": _NAMES[dtype], "shape": list(shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * (-len(blob) % 8)  # keep the data section 8-byte aligned
    declared = iter(shapes_and_dtypes)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, tensor in tensors:
            want_name, want_shape, want_dtype = next(declared)
            if name != want_name or tuple(tensor.shape) != tuple(want_shape) or tensor.dtype != want_dtype:
                raise LoadError(f"tensor '{name}' does not match its declaration ({want_name}, {want_shape}, {want_dtype})")
            data = tensor.detach().contiguous().cpu()
            if data.numel():
                f.write(memoryview(data.reshape(-1).view(torch.uint8).numpy()))
