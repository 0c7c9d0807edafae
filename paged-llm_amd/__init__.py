"""A paged Llama inference engine for one AMD MI355X (gfx950): model folder in, tokens out.

    from paged_llm_amd import EngineConfig, SamplingParams
    from paged_llm_amd.engine.llm_engine import LLMEngine
"""
from .config.engine_config import EngineConfig
from .engine.request import SamplingParams

__all__ = ["EngineConfig", "SamplingParams"]
