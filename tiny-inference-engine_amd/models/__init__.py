"""Model descriptions and the builder that turns them into runnable models."""

from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec
from .builder import Model, expected_tensors_for_config, load_model, load_model_from_tensors, model_from_config
from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
