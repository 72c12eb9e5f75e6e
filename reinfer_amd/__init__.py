"""reinfer_amd: a small, whole inference engine for one MI355X (gfx950)."""
from .config import Qwen3Config, load_config, register_architecture
from .engine import ModelRunner, StepEntry

__version__ = "0.1.0"
__all__ = ["Qwen3Config", "load_config", "register_architecture", "ModelRunner", "StepEntry"]
