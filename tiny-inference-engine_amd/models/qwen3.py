"""Qwen3 dense as a ModelSpec.

A pre-norm decoder: token embedding; ``num_layers`` identical layers of
grouped-query attention (per-head q/k RMSNorm before rotate-half rotary, full
causal attention) and a SwiGLU feed-forward; a final RMSNorm; a vocabulary
projection that is the embedding matrix when ``tie_word_embeddings`` is set.
Tensor names are HuggingFace's, exactly those the reference binds
(``src/model/qwen3.cpp:75-100``). The attention scale is ``1 / sqrt(head_dim)``
in float32 (``qwen3.cpp:195``); one ``rms_norm_eps`` serves all five norms
(``qwen3.cpp:193,218,222,223,234,258``).
"""

from __future__ import annotations

import numpy as np

from ..config.qwen3 import Qwen3Config
from ..config.registry import register_architecture
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec


def build_qwen3_spec(config: Qwen3Config) -> ModelSpec:
    scale = float(np.float32(1.0) / np.sqrt(np.float32(config.head_dim)))
    layers = []
    for l in range(config.num_layers):
        p = f"model.layers.{l}."
        norm = lambda name: PartSpec("rms_norm", {"dim": config.hidden_size, "eps": config.rms_norm_eps,
                                                  "weight": p + name})
        mixer = PartSpec("paged_attention", {
            "hidden": config.hidden_size,
            "num_heads": config.num_heads,
            "num_kv_heads": config.num_kv_heads,
            "head_dim": config.head_dim,
            "scale": scale,
            "window": None,
            "qk_norm": {"eps": config.rms_norm_eps,
                        "q_weight": p + "self_attn.q_norm.weight",
                        "k_weight": p + "self_attn.k_norm.weight"},
            "position": PartSpec("rope_neox", {"head_dim": config.head_dim, "theta": config.rope_theta}),
            "names": {"q": p + "self_attn.q_proj.weight", "k": p + "self_attn.k_proj.weight",
                      "v": p + "self_attn.v_proj.weight", "o": p + "self_attn.o_proj.weight"},
        })
        feed_forward = PartSpec("swiglu", {
            "hidden": config.hidden_size,
            "intermediate": config.intermediate_size,
            "names": {"gate": p + "mlp.gate_proj.weight", "up": p + "mlp.up_proj.weight",
                      "down": p + "mlp.down_proj.weight"},
        })
        layers.append(LayerSpec(
            block=PartSpec("pre_norm"),
            mixer=mixer,
            feed_forward=feed_forward,
            norms={"pre_mixer": norm("input_layernorm.weight"),
                   "pre_feed_forward": norm("post_attention_layernorm.weight")},
        ))
    embed_name = "model.embed_tokens.weight"
    return ModelSpec(
        architecture="Qwen3ForCausalLM",
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        max_positions=config.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab": config.vocab_size, "hidden": config.hidden_size,
                                               "weight": embed_name}),
        layers=tuple(layers),
        order=tuple(LayerCall(l) for l in range(config.num_layers)),
        head=PartSpec("lm_head", {
            "vocab": config.vocab_size,
            "hidden": config.hidden_size,
            "norm": PartSpec("rms_norm", {"dim": config.hidden_size, "eps": config.rms_norm_eps,
                                          "weight": "model.norm.weight"}),
            "weight": "lm_head.weight",
            "tied_to": embed_name if config.tie_word_embeddings else None,
        }),
    )


register_architecture("Qwen3ForCausalLM", Qwen3Config.from_json, build_qwen3_spec, model_types=("qwen3",))
