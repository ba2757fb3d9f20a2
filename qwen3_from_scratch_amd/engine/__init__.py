from .batch import StepBatch, StepEntry, pack_step
from .runner import ModelRunner
from .loading import load_model, load_runner, random_model
from .scheduler import Request, RequestStatus, Scheduled, Scheduler
from .sync_engine import BatchPerfMetrics, PerfMetrics, StreamChunk, SyncEngine
from .llm_engine import LLMEngine

__all__ = [
    "StepBatch", "StepEntry", "pack_step", "ModelRunner", "load_model", "load_runner", "random_model",
    "Request", "RequestStatus", "Scheduled", "Scheduler",
    "BatchPerfMetrics", "PerfMetrics", "StreamChunk", "SyncEngine", "LLMEngine",
]
