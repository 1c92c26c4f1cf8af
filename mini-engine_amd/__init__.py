"""mini-engine for one AMD MI355X: a small, whole LLM inference engine for the Qwen3 dense decoder,
with hand-written HIP kernels for gfx950."""

from .config.engine_config import EngineConfig
from .engine.llm_engine import EngineStats, LLMEngine, kv_cache_bytes_per_token
from .engine.sequence import SamplingParams, Sequence

__all__ = ["EngineConfig", "EngineStats", "LLMEngine", "SamplingParams", "Sequence", "kv_cache_bytes_per_token"]
