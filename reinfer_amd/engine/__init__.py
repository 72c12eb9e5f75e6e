from .batch import StepBatch, StepEntry, build_step_batch
from .runner import ModelRunner, StepError, parse_dtype

__all__ = ["StepBatch", "StepEntry", "build_step_batch", "ModelRunner", "StepError", "parse_dtype"]
