"""Sampling: greedy, temperature, top-k, top-p, repetition penalty."""
from .sampler import GREEDY_BELOW, Sampler, SamplerConfig, TokenLog, request_seed, uniform

__all__ = ["GREEDY_BELOW", "Sampler", "SamplerConfig", "TokenLog", "request_seed", "uniform"]
