"""A single-GPU inference engine for MI355X (gfx950): paged cache, one mixed-batch step function,
continuous batching with chunked prefill, hand-written HIP kernels, a true 32-bit path."""
from .config import EngineConfig, Qwen2Config, load_config, register_architecture
from .engine import LLM, Engine, GenerationResult, Request, generate
from .loading import load_model
from .sampling import SamplingParams
from .weights import load_random_model, write_random_model

__all__ = ["EngineConfig", "Qwen2Config", "load_config", "register_architecture", "LLM", "Engine",
           "GenerationResult", "Request", "generate", "load_model", "SamplingParams", "write_random_model",
           "load_random_model"]
