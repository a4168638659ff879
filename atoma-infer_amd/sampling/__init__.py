"""Generation parameters and the sampler."""
from .params import DEFAULT_RANDOM_SEED, GenerateParameters, SamplingPlan, ValidationError, validate
from .sampler import Pending, Sampler, uniform

__all__ = ["DEFAULT_RANDOM_SEED", "GenerateParameters", "SamplingPlan", "ValidationError", "validate", "Sampler",
           "uniform"]
