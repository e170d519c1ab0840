"""mercury_amd: a single-GPU inference engine for MI355X (gfx950), hand-written HIP kernels.

    from mercury_amd import Engine, EngineConfig, SamplingParams
    engine = Engine(EngineConfig(model="/path/to/model", dtype="bfloat16"))
    tokens = engine.generate([[1, 2, 3]], SamplingParams(temperature=0.0), max_tokens=16)
"""

from .cache import CacheManager, PagePool
from .config import EngineConfig, Qwen2Config, build_model, register_architecture
from .engine import Engine, Plan, Request, RequestState, SamplingParams, Scheduler, StreamEvent

__version__ = "0.1.0"

__all__ = [
    "CacheManager", "Engine", "EngineConfig", "PagePool", "Plan", "Qwen2Config", "Request",
    "RequestState", "SamplingParams", "Scheduler", "StreamEvent", "build_model",
    "register_architecture", "__version__",
]
