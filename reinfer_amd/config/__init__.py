from .schema import (BlockSpec, ConfigError, DecayMemorySpec, DeltaRuleSpec, FeedForwardSpec, InputSpec, LatentAttentionSpec,
                     MatrixMemorySpec, MixerSpec, ModelSpec, MoESpec, NormSpec, PairHashSpec, PositionSpec, RunEntry,
                     ParallelSpec, SideBySideSpec, StreamAdd, UnknownArchitecture, WKVSpec)
from .registry import (architecture_name, config_from_dict, load_config, register_architecture,
                       registered_architectures)
from .qwen3 import Qwen3Config
from .puresun import PuresunConfig
from .kobolix import KobolixConfig
from .detatar import DetatarConfig
from .gibavik import GibavikConfig

register_architecture("Qwen3ForCausalLM", Qwen3Config, "qwen3")
register_architecture("Puresun", PuresunConfig, "puresun")
register_architecture("Kobolix", KobolixConfig, "kobolix")
register_architecture("Detatar", DetatarConfig, "detatar")
register_architecture("Gibavik", GibavikConfig, "gibavik")

__all__ = [
    "BlockSpec", "ConfigError", "FeedForwardSpec", "MixerSpec", "ModelSpec", "NormSpec",
    "PositionSpec", "RunEntry", "UnknownArchitecture", "architecture_name", "config_from_dict",
    "load_config", "register_architecture", "registered_architectures", "Qwen3Config", "PuresunConfig", "KobolixConfig", "DetatarConfig", "GibavikConfig", "DecayMemorySpec", "ParallelSpec", "WKVSpec",
    "InputSpec", "LatentAttentionSpec", "DeltaRuleSpec", "MatrixMemorySpec", "SideBySideSpec", "MoESpec", "PairHashSpec", "StreamAdd",
]
