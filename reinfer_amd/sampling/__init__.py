from .params import SamplingParams
from .sampler import Sampler, SamplingError, derive_seed

__all__ = ["SamplingParams", "Sampler", "SamplingError", "derive_seed"]
