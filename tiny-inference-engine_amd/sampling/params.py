"""Sampling parameters of one request, with the reference's meanings and defaults.

``src/sampling/sampler.h:11-17`` and ``sampler.cpp:10-16``: temperature 0 is greedy;
top_k 0 and top_p 1 switch those filters off; max_tokens counts generated tokens
including a final stop token.
"""

from __future__ import annotations

import dataclasses
import math

from ..errors import InvalidArgument


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 0
    max_tokens: int = 256

    def validate(self) -> None:
        """Raises InvalidArgument naming the first impossible field."""
        if not (isinstance(self.temperature, (int, float)) and math.isfinite(self.temperature)
                and self.temperature >= 0.0):
            raise InvalidArgument(f"temperature must be finite and >= 0, got {self.temperature}")
        if not isinstance(self.top_k, int) or self.top_k < 0:
            raise InvalidArgument(f"top_k must be >= 0, got {self.top_k}")
        if not (isinstance(self.top_p, (int, float)) and 0.0 < self.top_p <= 1.0):
            raise InvalidArgument(f"top_p must be in (0, 1], got {self.top_p}")
        if not isinstance(self.seed, int) or not 0 <= self.seed < 2 ** 64:
            raise InvalidArgument(f"seed must be an unsigned 64-bit integer, got {self.seed}")
        if not isinstance(self.max_tokens, int) or self.max_tokens < 1:
            raise InvalidArgument(f"max_tokens must be >= 1, got {self.max_tokens}")

    @property
    def greedy(self) -> bool:
        """Whether every draw is the argmax: temperature 0, or so small that its reciprocal overflows."""
        import numpy as np

        if self.temperature == 0.0:
            return True
        with np.errstate(divide="ignore", over="ignore"):
            return not np.isfinite(np.float32(1.0) / np.float32(self.temperature))
