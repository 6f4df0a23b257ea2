"""Model descriptions and the builder that turns them into runnable models."""

from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec
from .builder import Model, expected_tensors_for_config, load_model, load_model_from_tensors, model_from_config
from . import duzozen, minerax, qwen3, topapel, zovudra  # noqa: F401  (register Duzozen, Minerax, Qwen3ForCausalLM, Topapel, Zovudra)
