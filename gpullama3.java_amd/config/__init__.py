from .registry import (ConfigError, config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .specs import (AttentionSpec, BlockSpec, GatedFeedForwardSpec, Llama3RopeScaling, ModelSpec,
                    NormSpec, RotarySpec, Run)
from .llama import LlamaConfiguration

__all__ = ["ConfigError", "config_from_dict", "load_config", "register_architecture",
           "registered_architectures", "AttentionSpec", "BlockSpec", "GatedFeedForwardSpec",
           "Llama3RopeScaling", "ModelSpec", "NormSpec", "RotarySpec", "Run", "LlamaConfiguration"]
