"""Sampling options and the sampler that chooses next tokens on the device."""
from .params import GREEDY, SamplingError, SamplingParams
from .sampler import DeviceSampler, SequenceSampling, penalty_counts, uniform

__all__ = ["GREEDY", "SamplingError", "SamplingParams", "DeviceSampler", "SequenceSampling", "penalty_counts", "uniform"]
