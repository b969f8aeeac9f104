"""The shape of one step, shared by the scheduler and the engine.

``src/engine/serving_config.h:12-22`` and ``serving_config.cpp:7-25`` of the
reference: a token budget per step and a cap on sequences per step, with
``max_seqs <= max_tokens_per_step`` so that every running sequence can decode
one token in the same step. ``prefill_chunk`` is an addition: the most prompt
tokens one sequence runs in one step (0 = only the budget limits it).
"""

from __future__ import annotations

import dataclasses

from ..errors import InvalidArgument


@dataclasses.dataclass
class ServingConfig:
    max_tokens_per_step: int = 512
    max_seqs: int = 64
    prefill_chunk: int = 0

    def validate(self) -> None:
        if self.max_tokens_per_step <= 0:
            raise InvalidArgument(f"max_tokens_per_step must be positive, got {self.max_tokens_per_step}")
        if self.max_seqs <= 0:
            raise InvalidArgument(f"max_seqs must be positive, got {self.max_seqs}")
        if self.max_seqs > self.max_tokens_per_step:
            raise InvalidArgument(
                f"max_seqs ({self.max_seqs}) cannot exceed max_tokens_per_step ({self.max_tokens_per_step}): "
                f"every sequence must decode each step")
        if self.prefill_chunk < 0:
            raise InvalidArgument(f"prefill_chunk must be >= 0, got {self.prefill_chunk}")
