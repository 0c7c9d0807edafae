from .engine_config import EngineConfig
from .model_config import LlamaConfig, resolve_dtype
from .registry import ARCHITECTURES, Architecture, lookup_architecture, register_architecture, read_config_json

__all__ = ["EngineConfig", "LlamaConfig", "resolve_dtype", "ARCHITECTURES", "Architecture",
           "lookup_architecture", "register_architecture", "read_config_json"]
