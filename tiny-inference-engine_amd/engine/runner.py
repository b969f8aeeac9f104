"""The step function: run exactly the tokens given, from the cache, and return the wanted logits.

``ModelRunner.step(entries)`` is the one way tokens pass through a model here:
generation, the scheduler's engine and trace replay all call it. It builds the
step's arrays, runs embedding, the run order and the head on the wanted rows,
and leaves the keys and values of the new tokens in the cache
(``src/model/qwen3.cpp:160-263`` is the reference's step). Pages must have been
reserved by the caller; nothing is sampled here.
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..errors import InvalidArgument
from ..models.builder import Model
from ..parts.base import StepContext, Workspace
from .batch import BatchBuilder, StepEntry


class ModelRunner:
    def __init__(self, model: Model, cache: CacheManager, max_seq_len: Optional[int] = None):
        if model.mode is None:
            raise InvalidArgument("the model has no weights loaded")
        if cache.plan is not model.cache_plan and cache.plan != model.cache_plan:
            raise InvalidArgument("the cache was not planned for this model")
        self.model = model
        self.cache = cache
        self.device = model.device
        limit = model.spec.max_positions
        self.max_seq_len = min(limit, max_seq_len) if max_seq_len else limit
        self.max_blocks_per_seq = cache.blocks_for(self.max_seq_len)
        self.builder = BatchBuilder(cache, model.spec.vocab_size, self.max_blocks_per_seq, self.device)
        self.workspace = Workspace(self.device)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Runs one batch; returns float32 logits ``[wanted rows, vocab]`` on the device, or None."""
        for e in entries:
            if e.start + len(e.tokens) > self.max_seq_len:
                raise InvalidArgument(
                    f"a request would reach {e.start + len(e.tokens)} tokens; the limit is {self.max_seq_len}")
        batch = self.builder.build(entries)
        ctx = StepContext(batch, self.model.mode, self.device, self.workspace, self.cache, self.model.cache_plan)
        return self.model.forward(ctx)
