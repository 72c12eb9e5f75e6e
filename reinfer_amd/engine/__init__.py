from .batch import StepBatch, StepEntry, build_step_batch
from .llm import LLMEngine, RequestOutput
from .runner import ModelRunner, StepError, parse_dtype
from .scheduler import Portion, Request, RequestRefused, Scheduler, StepPlan

__all__ = ["StepBatch", "StepEntry", "build_step_batch", "LLMEngine", "RequestOutput", "ModelRunner",
           "StepError", "parse_dtype", "Portion", "Request", "RequestRefused", "Scheduler", "StepPlan"]
