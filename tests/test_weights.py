"""Weights: the safetensors container, the folder loader, the binder's single error, random weights (no GPU).

Scenarios of the reference's tests/model/test_safetensors.cpp, test_loader.cpp and test_qwen3_binding.cpp.
"""

import json
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from tie_amd.errors import InvalidArgument, LoadError, UnsupportedError
from tie_amd.models import model_from_config
from tie_amd.weights.binder import check_tensors, place_tensor
from tie_amd.weights.loader import load_model_folder
from tie_amd.weights.random_init import write_random_model
from tie_amd.weights.safetensors_io import SafetensorsFile, StoredTensor, read_safetensors, write_safetensors


def raw_file(path, header, data=b""):
    blob = json.dumps(header).encode() if not isinstance(header, bytes) else header
    path.write_bytes(struct.pack("<Q", len(blob)) + blob + data)
    return path


def test_round_trip_and_interchange_with_the_safetensors_package(tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file

    tensors = [("a", torch.arange(6, dtype=torch.float32).view(2, 3)),
               ("b", torch.randn(4, 5).to(torch.bfloat16)), ("c", torch.tensor([1, 2, 3], dtype=torch.int32))]
    write_safetensors(tmp_path / "m.safetensors", tensors)
    mine = read_safetensors(tmp_path / "m.safetensors")
    assert [(t.dtype, t.shape) for t in mine.values()] == [("F32", (2, 3)), ("BF16", (4, 5)), ("I32", (3,))]
    for name, t in tensors:
        assert torch.equal(mine[name].torch(), t)
    with safe_open(str(tmp_path / "m.safetensors"), framework="pt") as f:       # the package reads what we write
        assert torch.equal(f.get_tensor("b"), tensors[1][1])
    save_file({n: t for n, t in tensors}, str(tmp_path / "theirs.safetensors"))  # and we read what it writes
    theirs = read_safetensors(tmp_path / "theirs.safetensors")
    assert torch.equal(theirs["a"].torch(), tensors[0][1])


def test_header_attacks_are_load_errors(tmp_path):
    p = tmp_path / "x.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(LoadError, match="truncated"):
        SafetensorsFile(p)
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(LoadError, match="runs past the end"):
        SafetensorsFile(p)
    with pytest.raises(LoadError, match="not valid JSON"):
        SafetensorsFile(raw_file(p, b"{not json"))
    with pytest.raises(LoadError, match="not a JSON object"):
        SafetensorsFile(raw_file(p, b"[1, 2]"))
    entry = {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 16]}
    with pytest.raises(LoadError, match="extends past the end"):
        SafetensorsFile(raw_file(p, {"t": entry}, b"\0" * 8))
    with pytest.raises(LoadError, match="needs 16 bytes"):
        SafetensorsFile(raw_file(p, {"t": {**entry, "data_offsets": [0, 12]}}, b"\0" * 16))
    with pytest.raises(LoadError, match="bad data_offsets"):
        SafetensorsFile(raw_file(p, {"t": {**entry, "data_offsets": [16, 0]}}, b"\0" * 16))
    with pytest.raises(LoadError, match="overflowing"):
        SafetensorsFile(raw_file(p, {"t": {**entry, "shape": [2 ** 40, 2 ** 40]}}, b"\0" * 16))
    with pytest.raises(LoadError, match="invalid"):
        SafetensorsFile(raw_file(p, {"t": {**entry, "shape": [-4, -1]}}, b"\0" * 16))
    with pytest.raises(UnsupportedError, match="F64"):
        SafetensorsFile(raw_file(p, {"t": {**entry, "dtype": "F64"}}, b"\0" * 32))
    with pytest.raises(LoadError, match="malformed"):
        SafetensorsFile(raw_file(p, {"t": {"shape": [1]}}, b"\0" * 4))
    ok = SafetensorsFile(raw_file(p, {"__metadata__": {"format": "pt"}, "s": {"dtype": "F32", "shape": [],
                                                                               "data_offsets": [0, 4]}}, b"\0" * 4))
    assert ok.tensors["s"].shape == (1,)                                   # a scalar becomes [1]


def test_folder_loader(tmp_path):
    with pytest.raises(LoadError, match="no such file"):
        load_model_folder(tmp_path / "missing")
    with pytest.raises(LoadError, match="config.json"):
        load_model_folder(tmp_path)
    (tmp_path / "config.json").write_text("{broken")
    with pytest.raises(LoadError, match="not valid JSON"):
        load_model_folder(tmp_path)
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(LoadError, match="model.safetensors"):
        load_model_folder(tmp_path)
    # sharded: only the set of file names of the index is used; duplicates across files are errors
    write_safetensors(tmp_path / "one.safetensors", [("a", torch.zeros(2))])
    write_safetensors(tmp_path / "two.safetensors", [("b", torch.zeros(3))])
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "one.safetensors", "b": "two.safetensors", "c": "two.safetensors"}}))
    files = load_model_folder(tmp_path)
    assert sorted(files.tensors) == ["a", "b"]
    write_safetensors(tmp_path / "two.safetensors", [("a", torch.zeros(3))])
    with pytest.raises(LoadError, match="duplicate tensor 'a'"):
        load_model_folder(tmp_path)
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": [1, 2]}))
    with pytest.raises(LoadError, match="weight_map"):
        load_model_folder(tmp_path)


def stored(cfg, seed=1):
    from tie_amd.weights.random_init import random_tensors

    model = model_from_config(cfg)
    specs = [s for s in model.expected_tensors() if not s.optional]
    return model, {n: StoredTensor.from_tensor(n, t) for n, t in random_tensors(specs, seed, torch.float32)}


def test_one_error_lists_everything_that_does_not_fit():
    model, tensors = stored(TINY_B)
    check_tensors(model.expected_tensors(), tensors)                        # fits as generated
    q = "model.layers.1.self_attn.q_proj.weight"
    tensors[q] = StoredTensor.from_tensor(q, tensors[q].torch().T.contiguous())           # transposed
    del tensors["model.layers.2.mlp.up_proj.weight"]                                       # missing
    del tensors["lm_head.weight"]                                                          # untied needs its head
    tensors["model.layers.0.self_attn.q_proj.bias"] = StoredTensor.from_tensor("b", torch.zeros(192))   # unexpected
    tensors["model.norm.weight"] = StoredTensor.from_tensor("n", torch.zeros(96, dtype=torch.int32))    # wrong dtype
    with pytest.raises(LoadError) as e:
        check_tensors(model.expected_tensors(), tensors)
    text = str(e.value)
    assert "missing (2): model.layers.2.mlp.up_proj.weight, lm_head.weight" in text
    assert "unexpected (1): model.layers.0.self_attn.q_proj.bias" in text
    assert f"{q}: has [96, 192], expected [192, 96]" in text
    assert "model.norm.weight: has I32" in text


def test_tied_head_accepts_a_duplicate_and_untied_requires_one():
    model, tensors = stored(TINY_A)
    assert "lm_head.weight" not in tensors
    check_tensors(model.expected_tensors(), tensors)
    tensors["lm_head.weight"] = StoredTensor.from_tensor("lm_head.weight", torch.zeros(256, 64))
    check_tensors(model.expected_tensors(), tensors)                        # duplicate head of a tied model: accepted
    tensors["lm_head.weight"] = StoredTensor.from_tensor("lm_head.weight", torch.zeros(64, 256))
    with pytest.raises(LoadError, match="lm_head.weight: has \\[64, 256\\]"):
        check_tensors(model.expected_tensors(), tensors)


def test_dtype_policy():
    bf = StoredTensor.from_tensor("m", torch.randn(4, 4).to(torch.bfloat16))
    f32 = StoredTensor.from_tensor("m", torch.randn(4, 4))
    f16 = StoredTensor.from_tensor("m", torch.randn(4, 4).to(torch.float16))
    assert place_tensor(bf, "matrix", "bfloat16", "cpu").dtype == torch.bfloat16      # kept in bfloat16
    assert place_tensor(f32, "matrix", "bfloat16", "cpu").dtype == torch.float32      # stored in 32-bit: stays so
    assert place_tensor(f16, "matrix", "bfloat16", "cpu").dtype == torch.float32      # widened exactly
    assert place_tensor(bf, "matrix", "float32", "cpu").dtype == torch.float32
    assert place_tensor(bf, "vector", "bfloat16", "cpu").dtype == torch.float32       # norm weights: float32
    table = StoredTensor.from_tensor("t", torch.tensor([1, 2 ** 20], dtype=torch.int64))
    assert place_tensor(table, "int_table", "bfloat16", "cpu").dtype == torch.int32
    big = StoredTensor.from_tensor("t", torch.tensor([2 ** 40], dtype=torch.int64))
    with pytest.raises(LoadError, match="outside int32"):
        place_tensor(big, "int_table", "bfloat16", "cpu")


def test_random_weights_mode_writes_a_loadable_folder(tmp_path):
    a = write_random_model(tmp_path / "a", TINY_B, seed=5, dtype="bfloat16")
    b = write_random_model(tmp_path / "b", TINY_B, seed=5, dtype="bfloat16")
    c = write_random_model(tmp_path / "c", TINY_B, seed=6, dtype="float32")
    fa, fb, fc = load_model_folder(a), load_model_folder(b), load_model_folder(c)
    assert json.loads((tmp_path / "a" / "config.json").read_text()) == TINY_B
    model = model_from_config(fa.config_values)
    check_tensors(model.expected_tensors(), fa.tensors)
    q = "model.layers.0.self_attn.q_proj.weight"
    assert fa.tensors[q].dtype == "BF16" and fc.tensors[q].dtype == "F32"
    assert torch.equal(fa.tensors[q].torch(), fb.tensors[q].torch())                  # same seed, same weights
    assert not torch.equal(fa.tensors[q].torch().float(), fc.tensors[q].torch())      # another seed differs
    w = fc.tensors[q].torch()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002        # N(0, 0.02)
    n = fc.tensors["model.layers.1.self_attn.k_norm.weight"].torch()
    assert float(n.min()) >= 0.9 and float(n.max()) <= 1.1 and float(n.std()) > 0.01  # 1 + U(-0.1, 0.1)
    with pytest.raises(InvalidArgument):
        write_random_model(tmp_path / "d", TINY_B, seed=1, dtype="int8")


def test_a_random_element_depends_on_its_key_and_index_alone():
    """The generator is counter-based: element i of a tensor is a function of (seed, name, i), so a tensor's
    prefix does not change with its length, with the pieces it is drawn in or with the other tensors around it,
    and a GPU can draw the same bits element by element (tests/test_gpu_kernels.py checks that it does)."""
    import numpy as np
    from scipy import stats
    from tie_amd.weights import random_init as ri
    from tie_amd.weights.binder import TensorSpec

    long = ri.random_tensor(TensorSpec("w", (3, 50_000), "matrix", ("normal", 0.02)), 9, torch.float32).flatten()
    short = ri.random_tensor(TensorSpec("w", (1000,), "matrix", ("normal", 0.02)), 9, torch.float32)
    assert torch.equal(long[:1000], short)
    old = ri._CHUNK
    try:
        ri._CHUNK = 777                                    # drawn in other pieces: the same values
        pieces = ri.random_tensor(TensorSpec("w", (150_000,), "matrix", ("normal", 0.02)), 9, torch.float32)
    finally:
        ri._CHUNK = old
    assert torch.equal(pieces, long)
    other_name = ri.random_tensor(TensorSpec("v", (1000,), "matrix", ("normal", 0.02)), 9, torch.float32)
    other_seed = ri.random_tensor(TensorSpec("w", (1000,), "matrix", ("normal", 0.02)), 10, torch.float32)
    assert not torch.equal(short, other_name) and not torch.equal(short, other_seed)
    # the distribution: N(0, 0.02) by the inverse distribution function, tails included
    z = long.double().numpy() / 0.02
    assert stats.kstest(z, "norm").pvalue > 1e-3
    assert abs(float((np.abs(z) > 3).mean()) - 0.0027) < 0.001 and float(np.abs(z).max()) > 3.8
    # the inverse distribution function itself against the library's, and the series that stands in for log
    p = np.concatenate([np.logspace(-16, -1, 500), np.linspace(0.05, 0.95, 1001), 1.0 - np.logspace(-15, -1, 500)])
    want = stats.norm.ppf(p)
    assert float(np.max(np.abs(ri._normal_of(p) - want) / np.maximum(1e-3, np.abs(want)))) < 1e-13
    x = np.concatenate([np.logspace(-300, -2, 2000), np.linspace(1e-3, 0.999, 2000)])
    assert float(np.max(np.abs(ri._log(x) - np.log(x)) / np.abs(np.log(x)))) < 1e-15
    u = ri.random_tensor(TensorSpec("n", (20_000,), "vector", ("one_plus_uniform", 0.1)), 9, torch.float32)
    assert 0.9 <= float(u.min()) < 0.9001 and 1.0999 < float(u.max()) <= 1.1 and abs(float(u.mean()) - 1.0) < 2e-3
    assert stats.kstest((u.double().numpy() - 0.9) / 0.2, "uniform").pvalue > 1e-3
