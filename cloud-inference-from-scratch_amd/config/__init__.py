from .engine_config import EngineConfig, build_engine_config, canonical_dtype
from .givizen import GivizenConfig
from .nokipel import NokipelConfig
from .polosun import PolosunConfig
from .qwen2 import Qwen2Config
from .senuvik import SenuvikConfig
from .registry import (
    ARCHITECTURES,
    Architecture,
    architecture_of,
    config_from_dict,
    load_config,
    register_architecture,
)
from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

# the architectures this package brings; others register themselves the same way from outside
register_architecture("Qwen2ForCausalLM", Qwen2Config, model_type="qwen2")
register_architecture("Polosun", PolosunConfig)
register_architecture("Givizen", GivizenConfig)
register_architecture("Nokipel", NokipelConfig)
register_architecture("Senuvik", SenuvikConfig)

__all__ = [
    "ARCHITECTURES", "Architecture", "ConfigError", "EngineConfig", "GivizenConfig", "LayerCall", "LayerSpec",
    "ModelSpec", "NokipelConfig", "PartSpec", "PolosunConfig", "Qwen2Config", "SenuvikConfig", "architecture_of", "build_engine_config",
    "canonical_dtype", "config_from_dict", "load_config", "register_architecture",
]
