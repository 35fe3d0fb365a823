"""A single-GPU inference engine for AMD Instinct MI355X (gfx950).

Everything between a request's tokens and its next token: typed configuration and
architecture registry, safetensors weights by name, layers put together from parts,
a paged cache manager, one step function over mixed batches, a scheduler, sampling,
and hand-written HIP kernels.
"""

from . import models  # registers the architectures
from .cache import BlockPoolExhaustedError, CacheManager, PagedKVSpec, SlotStateSpec
from .config import ConfigError, ModelConfig, Qwen2Config
from .engine import (
    BatchingPolicy,
    ContinuousBatchEngine,
    EngineConfig,
    EngineStepResult,
    ModelRunner,
    PageAdmission,
    Request,
    Scheduler,
    StepEntry,
    generate,
    greedy_generate,
    load_model,
    make_cache,
)
from .models import ARCHITECTURES, build_model, load_config, register_architecture
from .parts import DecoderModel, register_part
from .sampling import Sampler, SamplingParams
from .weights import WeightsError, load_weights, write_random_model

__version__ = "0.1.0"

__all__ = [
    "ARCHITECTURES",
    "BatchingPolicy",
    "BlockPoolExhaustedError",
    "CacheManager",
    "ConfigError",
    "ContinuousBatchEngine",
    "EngineConfig",
    "DecoderModel",
    "EngineStepResult",
    "ModelConfig",
    "ModelRunner",
    "PageAdmission",
    "PagedKVSpec",
    "Qwen2Config",
    "Request",
    "Scheduler",
    "Sampler",
    "SamplingParams",
    "SlotStateSpec",
    "StepEntry",
    "WeightsError",
    "build_model",
    "generate",
    "greedy_generate",
    "load_config",
    "load_model",
    "load_weights",
    "make_cache",
    "register_architecture",
    "register_part",
    "write_random_model",
]
