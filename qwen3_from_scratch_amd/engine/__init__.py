from .batch import StepBatch, StepEntry, pack_step
from .runner import ModelRunner
from .loading import load_model, load_runner

__all__ = ["StepBatch", "StepEntry", "pack_step", "ModelRunner", "load_model", "load_runner"]
