"""From a model folder to its config.json values and a table of stored tensors.

A folder holds ``config.json`` and either ``model.safetensors`` or the files
that ``model.safetensors.index.json`` lists. As in the reference
(``src/model/loader.cpp:224-249``), only the *set of file names* of the index is
used: each tensor comes from the header of the file that holds it, and a name
that appears in two files is an error.
"""

from __future__ import annotations

import dataclasses
import pathlib
from typing import Dict

from ..config.base import read_config_json
from ..errors import LoadError
from .safetensors_io import SafetensorsFile, StoredTensor


@dataclasses.dataclass
class ModelFiles:
    path: str
    config_values: dict
    tensors: Dict[str, StoredTensor]


def load_model_folder(path) -> ModelFiles:
    folder = pathlib.Path(path)
    if not folder.exists():
        raise LoadError(f"{folder}: no such file or directory")
    if not folder.is_dir():
        raise LoadError(f"{folder}: expected a directory containing config.json and model.safetensors")
    config_path = folder / "config.json"
    if not config_path.exists():
        raise LoadError(f"{folder}: no config.json in the model folder")
    config_values = read_config_json(config_path)

    index_path = folder / "model.safetensors.index.json"
    if index_path.exists():
        index = read_config_json(index_path)
        weight_map = index.get("weight_map")
        if not isinstance(weight_map, dict) or not all(isinstance(v, str) for v in weight_map.values()):
            raise LoadError(f"{index_path}: 'weight_map' must map tensor names to file names")
        files = sorted(set(weight_map.values()))
        if not files:
            raise LoadError(f"{index_path}: 'weight_map' lists no files")
    else:
        files = ["model.safetensors"]
        if not (folder / files[0]).exists():
            raise LoadError(f"{folder}: no model.safetensors (and no model.safetensors.index.json) in the model folder")

    tensors: Dict[str, StoredTensor] = {}
    for name in files:
        for tensor_name, tensor in SafetensorsFile(folder / name).tensors.items():
            if tensor_name in tensors:
                raise LoadError(f"duplicate tensor '{tensor_name}' in {tensors[tensor_name].source} and {tensor.source}")
            tensors[tensor_name] = tensor
    return ModelFiles(str(folder), config_values, tensors)
