"""Step function, scheduler, admission and the continuous-batching engine."""

from .admission import BlockReservation, PagedBlockAdmissionController
from .config import EngineConfig, GraphLimits
from .engine import ContinuousBatchEngine, EngineStepResult
from .factory import load_model, make_cache, parse_dtype
from .generation import GenerationOutput, generate, greedy_generate
from .metrics import RequestMetrics, RequestMetricsCollector, TokenEvent
from .runner import ModelRunner, StepEntry, StepOutput
from .scheduler import (
    BatchingPolicy,
    FinishReason,
    RequestScheduler,
    RequestState,
    RequestStatus,
    ScheduledRequest,
    SchedulerBatch,
    SchedulerStepUpdate,
    WorkKind,
)

__all__ = [
    "BatchingPolicy",
    "BlockReservation",
    "ContinuousBatchEngine",
    "EngineConfig",
    "GraphLimits",
    "EngineStepResult",
    "FinishReason",
    "GenerationOutput",
    "ModelRunner",
    "PagedBlockAdmissionController",
    "RequestMetrics",
    "RequestMetricsCollector",
    "RequestScheduler",
    "RequestState",
    "RequestStatus",
    "ScheduledRequest",
    "SchedulerBatch",
    "SchedulerStepUpdate",
    "StepEntry",
    "StepOutput",
    "TokenEvent",
    "WorkKind",
    "generate",
    "greedy_generate",
    "load_model",
    "make_cache",
    "parse_dtype",
]
