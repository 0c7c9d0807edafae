from .dtypes import resolve_dtype
from .engine_config import EngineConfig
from .registry import ARCHITECTURES, Architecture, lookup_architecture, register_architecture, read_config_json

__all__ = ["EngineConfig", "resolve_dtype", "ARCHITECTURES", "Architecture",
           "lookup_architecture", "register_architecture", "read_config_json"]
