from .params import SamplingParams, ScoringParams
from .sampler import Sampler, request_seed

__all__ = ["SamplingParams", "ScoringParams", "Sampler", "request_seed"]
