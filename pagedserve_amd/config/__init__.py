from .base import ConfigError, read_config_json
from .gpt2 import GPT2Config
from .registry import ARCHITECTURES, Architecture, register_architecture, resolve_architecture
from .spec import BlockSpec, LayerCall, ModelSpec, PartSpec

__all__ = [
    "ARCHITECTURES", "Architecture", "BlockSpec", "ConfigError", "GPT2Config", "LayerCall",
    "ModelSpec", "PartSpec", "read_config_json", "register_architecture", "resolve_architecture",
]
