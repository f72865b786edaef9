from .rng import splitmix64, uniform
from .sampler import SamplerError, SamplingParams, apply_penalties, argmax, distribution, sample, select
