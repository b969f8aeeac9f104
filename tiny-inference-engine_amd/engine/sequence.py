"""Per-request state of the engine (``src/engine/sequence.h:12-30`` of the reference)."""

from __future__ import annotations

import enum
from typing import List

from ..cache.manager import RequestCache
from ..sampling.params import SamplingParams
from ..sampling.rng import RandomStream


class SeqState(enum.Enum):
    WAITING = "waiting"
    PREFILLING = "prefilling"
    DECODING = "decoding"
    FINISHED = "finished"


class FinishReason(enum.Enum):
    NONE = "none"
    STOP = "stop"
    LENGTH = "length"
    ERROR = "error"
    CANCELLED = "cancelled"


UNREAD = -1      # stands in ``Sequence.tokens`` for a token the GPU has chosen and the host has not read yet


class Sequence:
    """One request: its tokens (prompt, then generated), how many are cached, and what it holds."""

    def __init__(self, seq_id: int, prompt: List[int], params: SamplingParams, cache: RequestCache):
        self.id = seq_id
        self.tokens: List[int] = list(prompt)
        self.prompt_len = len(prompt)
        self.num_computed = 0                  # tokens whose keys and values are in the cache
        self.cache = cache
        self.params = params
        self.rng = RandomStream(params.seed)
        self.state = SeqState.WAITING
        self.finish_reason = FinishReason.NONE
        self.waiting_since_step = 0            # scheduler step at which it last entered the waiting queue
        self.num_preemptions = 0
        self.in_flight = False                 # part of a planned step that has neither run nor been abandoned

    @property
    def num_generated(self) -> int:
        return len(self.tokens) - self.prompt_len

    @property
    def num_pending(self) -> int:
        return len(self.tokens) - self.num_computed

    @property
    def generated(self) -> List[int]:
        """The generated tokens the host knows (a last one still on its way from the GPU is left out)."""
        out = self.tokens[self.prompt_len:]
        if out and out[-1] == UNREAD:
            out.pop()
        return out
