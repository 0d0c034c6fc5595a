from .registry import (ConfigError, config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .specs import (AttentionSpec, BlockSpec, DistanceBias, GatedDeltaSpec, GatedFeedForwardSpec, Inject,
                    Llama3RopeScaling, LinearRopeScaling, MinGRUSpec, ModelSpec, NormSpec, PairEmbedding, Remix,
                    RotarySpec, Run, SideBySideSpec, TimeMixSpec)
from .llama import LlamaConfiguration
from .melizen import MelizenConfiguration
from .nodupel import NodupelConfiguration
from .nolatar import NolatarConfiguration
from .dotanex import DotanexConfiguration

__all__ = ["ConfigError", "config_from_dict", "load_config", "register_architecture",
           "registered_architectures", "AttentionSpec", "BlockSpec", "GatedFeedForwardSpec",
           "Llama3RopeScaling", "ModelSpec", "NormSpec", "RotarySpec", "Run", "LlamaConfiguration", "DistanceBias", "GatedDeltaSpec", "Inject",
           "MelizenConfiguration", "NodupelConfiguration", "LinearRopeScaling", "MinGRUSpec", "PairEmbedding", "Remix",
           "SideBySideSpec", "TimeMixSpec", "NolatarConfiguration", "DotanexConfiguration"]
