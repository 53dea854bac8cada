from .causal_lm import CausalLM, model_param_specs
from .spec import IgnoreRule, LayerSpec, ModelSpec, PartSpec, linear_output, token_embedding

__all__ = [
    "CausalLM", "IgnoreRule", "LayerSpec", "ModelSpec", "PartSpec", "linear_output", "model_param_specs",
    "token_embedding",
]
