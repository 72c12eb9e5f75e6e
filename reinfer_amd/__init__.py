"""reinfer_amd: a small, whole inference engine for one MI355X (gfx950)."""
from .config import Qwen3Config, load_config, register_architecture
from .engine import LLMEngine, ModelRunner, RequestOutput, StepEntry
from .sampling import SamplingParams

__version__ = "0.1.0"
__all__ = ["Qwen3Config", "load_config", "register_architecture", "LLMEngine", "ModelRunner",
           "RequestOutput", "StepEntry", "SamplingParams"]
