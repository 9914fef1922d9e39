"""Sampling: parameters, the seeded draw, and the device sampler."""
from .rng import request_key, splitmix64, uniform
from .sampler import (DEFAULT_MAX_NEW_TOKENS, DEFAULT_TEMPERATURE, DEFAULT_TOP_K, DEFAULT_TOP_P, GREEDY_BELOW,
                      MAX_TOP_K, Draw, Sampler, SamplingParams)
