from .engine import EngineMetrics, EngineResult, InferenceEngine, StreamUpdate
from .scheduler import GenerationScheduler
from .step import ModelRunner, StepEntry
from .types import GenerationRequest, RequestPhase, SchedulerResult

__all__ = ["EngineMetrics", "EngineResult", "GenerationRequest", "GenerationScheduler", "InferenceEngine",
           "ModelRunner", "RequestPhase", "SchedulerResult", "StepEntry", "StreamUpdate"]
