"""Greedy, temperature, top-k and top-p sampling."""

from .params import SamplingParams
from .rng import RandomStream
from .sampler import DeviceSampler, sample
