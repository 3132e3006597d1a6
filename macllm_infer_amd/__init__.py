"""A Falcon-H1 inference engine for one AMD MI355X (gfx950): typed configuration and
architecture registry, safetensors weights, layers composed from parts, a paged cache
manager with state slots, one step function over mixed batches, a continuous-batching
scheduler, GPU sampling, and hand-written HIP kernels with a true float32 path."""
from .cache import CacheExhausted
from .config import ConfigError, FalconH1Config, load_config, register_architecture
from .engine import (LLM, Engine, EngineConfig, GenerationResult, Lane, Scheduler, StepError, StepFailed,
                     generate)
from .sampling import GREEDY, Sampler, SamplingParams
from .weights import WeightError

__version__ = "0.1.0"

__all__ = ["CacheExhausted", "ConfigError", "Engine", "EngineConfig", "FalconH1Config", "GREEDY",
           "GenerationResult", "LLM", "Lane", "Sampler", "SamplingParams", "Scheduler", "StepError", "StepFailed",
           "WeightError", "generate", "load_config", "register_architecture"]
