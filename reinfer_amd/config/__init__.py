from .schema import (BlockSpec, ConfigError, FeedForwardSpec, MixerSpec, ModelSpec, NormSpec,
                     PositionSpec, RunEntry, UnknownArchitecture)
from .registry import (architecture_name, config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .qwen3 import Qwen3Config

register_architecture("Qwen3ForCausalLM", Qwen3Config, "qwen3")

__all__ = [
    "BlockSpec", "ConfigError", "FeedForwardSpec", "MixerSpec", "ModelSpec", "NormSpec",
    "PositionSpec", "RunEntry", "UnknownArchitecture", "architecture_name", "config_from_dict",
    "load_config", "register_architecture", "registered_architectures", "Qwen3Config",
]
