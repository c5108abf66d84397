from .params import SamplingParams
from .sampler import Sampler, request_seed

__all__ = ["Sampler", "SamplingParams", "request_seed"]
