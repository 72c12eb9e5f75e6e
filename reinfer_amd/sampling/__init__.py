from .params import SamplingParams
from .sampler import Sampler, SamplingError, as_int64, derive_seed

__all__ = ["SamplingParams", "Sampler", "SamplingError", "as_int64", "derive_seed"]
