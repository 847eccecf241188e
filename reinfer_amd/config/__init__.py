from .schema import (BlockSpec, ConfigError, FeedForwardSpec, InputSpec, LatentAttentionSpec, MixerSpec,
                     ModelSpec, MoESpec, NormSpec, PairHashSpec, PositionSpec, RunEntry, StreamAdd,
                     UnknownArchitecture)
from .registry import (architecture_name, config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .qwen3 import Qwen3Config
from .puresun import PuresunConfig

register_architecture("Qwen3ForCausalLM", Qwen3Config, "qwen3")
register_architecture("Puresun", PuresunConfig, "puresun")

__all__ = [
    "BlockSpec", "ConfigError", "FeedForwardSpec", "MixerSpec", "ModelSpec", "NormSpec",
    "PositionSpec", "RunEntry", "UnknownArchitecture", "architecture_name", "config_from_dict",
    "load_config", "register_architecture", "registered_architectures", "Qwen3Config", "PuresunConfig",
    "InputSpec", "LatentAttentionSpec", "MoESpec", "PairHashSpec", "StreamAdd",
]
