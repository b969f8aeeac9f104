"""Configuration and registry (no GPU). Scenarios of the reference's tests/model/test_config.cpp."""

import pytest

from conftest import TINY_A, TINY_B
from tie_amd.config.qwen3 import Qwen3Config
from tie_amd.config.registry import (register_architecture, resolve_architecture, supported_architectures,
                                     unregister_architecture)
from tie_amd.errors import LoadError, UnsupportedError
from tie_amd.models import model_from_config

QWEN3_06B = {  # the published Qwen3-0.6B config.json values the reference's test reads (test_config.cpp:23-34)
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "vocab_size": 151936, "hidden_size": 1024,
    "intermediate_size": 3072, "num_hidden_layers": 28, "num_attention_heads": 16, "num_key_value_heads": 8,
    "head_dim": 128, "max_position_embeddings": 40960, "rms_norm_eps": 1e-6, "rope_theta": 1000000,
    "tie_word_embeddings": True, "hidden_act": "silu", "torch_dtype": "bfloat16", "sliding_window": None,
    "use_sliding_window": False, "rope_scaling": None, "attention_bias": False, "max_window_layers": 28,
}


def test_reads_the_published_small_config():
    c = Qwen3Config.from_json(QWEN3_06B)
    assert (c.q_dim, c.kv_dim, c.rope_theta, c.tie_word_embeddings) == (2048, 1024, 1e6, True)
    assert c.num_layers == 28 and c.head_dim == 128 and c.rms_norm_eps == 1e-6


def test_defaults_follow_the_reference():
    values = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "num_key_value_heads", "rope_theta",
                                                           "tie_word_embeddings")}
    c = Qwen3Config.from_json(values)
    assert c.head_dim == 64 // 4 and c.num_kv_heads == 4 and c.rope_theta == 10000.0 and c.tie_word_embeddings is False


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "max_position_embeddings", "rms_norm_eps"])
def test_required_keys(key):
    values = dict(TINY_B)
    del values[key]
    with pytest.raises(LoadError, match=key):
        Qwen3Config.from_json(values)


def test_rejections():
    def with_(**kw):
        return {**TINY_B, **kw}

    with pytest.raises(UnsupportedError, match="sliding"):
        Qwen3Config.from_json(with_(use_sliding_window=True))
    with pytest.raises(UnsupportedError, match="rope_scaling"):
        Qwen3Config.from_json(with_(rope_scaling={"type": "yarn", "factor": 4.0}))
    with pytest.raises(UnsupportedError, match="attention_bias"):
        Qwen3Config.from_json(with_(attention_bias=True))
    with pytest.raises(UnsupportedError, match="gelu"):
        Qwen3Config.from_json(with_(hidden_act="gelu"))
    with pytest.raises(LoadError, match="multiple"):
        Qwen3Config.from_json(with_(num_attention_heads=6, num_key_value_heads=4))
    with pytest.raises(LoadError, match="even"):
        Qwen3Config.from_json(with_(head_dim=31))
    with pytest.raises(LoadError, match="positive"):
        Qwen3Config.from_json(with_(vocab_size=0))
    with pytest.raises(LoadError, match="rms_norm_eps"):
        Qwen3Config.from_json(with_(rms_norm_eps=0.0))
    with pytest.raises(LoadError, match="integer"):
        Qwen3Config.from_json(with_(hidden_size="96"))
    # ignored keys stay ignored
    Qwen3Config.from_json(with_(sliding_window=4096, max_window_layers=2, bos_token_id=1, torch_dtype="float16"))


def test_registry_resolves_by_architecture_then_model_type():
    assert resolve_architecture(TINY_A).name == "Qwen3ForCausalLM"
    assert resolve_architecture({"model_type": "qwen3"}).name == "Qwen3ForCausalLM"
    with pytest.raises(UnsupportedError, match="LlamaForCausalLM.*supported: .*Qwen3ForCausalLM"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    with pytest.raises(LoadError):
        resolve_architecture({})
    with pytest.raises(LoadError):
        resolve_architecture({"architectures": "Qwen3ForCausalLM"})


def test_registering_another_architecture():
    arch = resolve_architecture(TINY_A)
    register_architecture("ToyForCausalLM", arch.read_config, arch.build_spec, model_types=("toy",))
    try:
        assert "ToyForCausalLM" in supported_architectures()
        assert resolve_architecture({"architectures": ["ToyForCausalLM"]}).name == "ToyForCausalLM"
        assert resolve_architecture({"model_type": "toy"}).name == "ToyForCausalLM"
    finally:
        unregister_architecture("ToyForCausalLM")
    assert "ToyForCausalLM" not in supported_architectures()


def test_spec_carries_every_size_of_the_config():
    for cfg in (TINY_A, TINY_B):
        model = model_from_config(cfg)
        spec = model.spec
        assert len(spec.layers) == cfg["num_hidden_layers"] and len(spec.order) == cfg["num_hidden_layers"]
        mixer = spec.layers[0].mixer.params
        assert (mixer["num_heads"], mixer["num_kv_heads"], mixer["head_dim"]) == (
            cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"])
        assert mixer["scale"] == pytest.approx(cfg["head_dim"] ** -0.5, rel=1e-6)
        assert mixer["position"].params["theta"] == cfg["rope_theta"]
        assert mixer["qk_norm"]["eps"] == cfg["rms_norm_eps"]
        assert spec.layers[0].feed_forward.params["intermediate"] == cfg["intermediate_size"]
        assert spec.head.params["tied_to"] == ("model.embed_tokens.weight" if cfg["tie_word_embeddings"] else None)
        group = model.cache_plan.groups[0]
        assert group.num_planes == cfg["num_hidden_layers"] and group.need.window is None
