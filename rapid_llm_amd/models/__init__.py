from .causal_lm import CausalLM, model_param_specs
from .spec import IgnoreRule, LayerSpec, ModelSpec, PartSpec

__all__ = ["CausalLM", "IgnoreRule", "LayerSpec", "ModelSpec", "PartSpec", "model_param_specs"]
