"""``from paged_llm_amd.engine.engine import LLMEngine`` mirrors the reference's import path."""
from .llm_engine import EngineStats, LLMEngine, RequestOutput, StepOutput

__all__ = ["EngineStats", "LLMEngine", "RequestOutput", "StepOutput"]
