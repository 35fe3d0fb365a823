"""Step function, scheduler, admission and the continuous-batching engine."""

from .admission import PageAdmission, PagePromise
from .config import EngineConfig, GraphLimits
from .engine import ContinuousBatchEngine, EngineBrokenError, EngineStepResult
from .factory import load_model, make_cache, parse_dtype
from .generation import GenerationOutput, generate, greedy_generate
from .metrics import RequestTimes, summarize
from .request import EndReason, Phase, Request, Timeline
from .runner import ModelRunner, StepEntry, StepOutput
from .scheduler import BatchingPolicy, Scheduler, Slice, StepPlan, StepReport

__all__ = [
    "BatchingPolicy",
    "ContinuousBatchEngine",
    "EndReason",
    "EngineBrokenError",
    "EngineConfig",
    "EngineStepResult",
    "GenerationOutput",
    "GraphLimits",
    "ModelRunner",
    "PageAdmission",
    "PagePromise",
    "Phase",
    "Request",
    "RequestTimes",
    "Scheduler",
    "Slice",
    "StepEntry",
    "StepOutput",
    "StepPlan",
    "StepReport",
    "Timeline",
    "generate",
    "greedy_generate",
    "load_model",
    "make_cache",
    "parse_dtype",
    "summarize",
]
