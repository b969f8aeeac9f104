"""Trace replay: given token ids go through the model step by step; logits come out.

Nothing is sampled and nothing is scheduled: a trace says which tokens of which
request run in which step and where logits are wanted. The replayer owns only
the bookkeeping of a trace (which request holds how many tokens); the model,
the step function, the cache manager and the kernels are the ones generation
uses. The reference has the same idea as a test helper that drives one sequence
through ``forward`` with its own block table (``tests/support/sequence_runner.h:13-46``).

A step is a dictionary::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

``entries`` is one batch; ``want`` lists the places among an entry's tokens whose
logits are returned, in the order of the entries and of ``want``; ``end`` lists
requests that are finished after the step, whose pages go back to the pool.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import kernels
from ..cache.manager import CacheManager, RequestCache
from ..errors import CapacityError, InvalidArgument
from ..models.builder import Model, load_model
from ..weights.binder import normalize_mode
from .batch import StepEntry
from .runner import ModelRunner


class TraceReplayer:
    def __init__(self, model: Model, max_tokens: int, block_size: int = 16, use_graphs=None, kv_dtype=None):
        """``max_tokens``: the most tokens live requests hold at any time, each request's
        count rounded up to a multiple of 64 (of the block size if that is larger); the page pool
        is made for exactly this many, so pages are used again. ``kv_dtype``: the cache's precision if it is
        to differ from the model's (float32 arithmetic over bfloat16 or float16 pages)."""
        if max_tokens <= 0:
            raise InvalidArgument(f"max_tokens must be positive, got {max_tokens}")
        self.model = model
        cache_dtype = kernels.cache_dtype_for(model.mode, kv_dtype)
        num_blocks = math.ceil(max_tokens / block_size)
        self.cache = CacheManager(model.cache_plan, block_size=block_size, num_blocks=num_blocks,
                                  dtype=cache_dtype, device=model.device, max_state_slots=8)
        # A request may outgrow the pool where windows give pages back, so only the model's context limits it.
        self.runner = ModelRunner(model, self.cache, use_graphs=use_graphs)
        self.requests: Dict[str, RequestCache] = {}
        self.lengths: Dict[str, int] = {}

    @classmethod
    def from_folder(cls, folder, dtype: str, max_tokens: int, block_size: int = 16, device="cuda:0",
                    use_graphs=None, kv_dtype=None):
        mode = normalize_mode(dtype)
        kernels.cache_dtype_for(mode, kv_dtype)        # a pair no kernel takes fails before the weights are read
        model = load_model(folder, mode, device)
        return cls(model, max_tokens, block_size, use_graphs, kv_dtype)

    def run_step(self, step: dict) -> Optional[torch.Tensor]:
        """Runs one step of a trace; returns float32 logits ``[wanted, vocab]`` (on the device) or None."""
        entries = step.get("entries", [])
        if not isinstance(entries, list):
            raise InvalidArgument("'entries' must be a list")
        batch: List[StepEntry] = []
        seen = set()
        grown = []
        try:
            for e in entries:
                rid = str(e["id"])
                tokens = [int(t) for t in e["tokens"]]
                want = [int(w) for w in e.get("want", [])]
                if rid in seen:
                    raise InvalidArgument(f"request '{rid}' appears twice in one step")
                seen.add(rid)
                if not tokens:
                    raise InvalidArgument(f"request '{rid}' brings no tokens")
                req = self.requests.get(rid)
                if req is None:
                    req = self.requests[rid] = self.cache.new_request()
                    self.lengths[rid] = 0
                start = self.lengths[rid]
                if not self.cache.reserve(req, start + len(tokens)):
                    raise CapacityError(
                        f"request '{rid}' needs {self.cache.blocks_for(start + len(tokens))} pages for "
                        f"{start + len(tokens)} tokens but only {self.cache.num_free()} of {self.cache.num_blocks} "
                        f"are free; raise --max-tokens")
                grown.append((rid, start))
                batch.append(StepEntry(req, start, tokens, want))
            logits = self.runner.step(batch) if batch else None
        except Exception:
            for rid, start in grown:           # the step never ran: give back what it reserved
                self.cache.truncate(self.requests[rid], start)
            raise
        for entry, (rid, start) in zip(batch, grown):
            self.lengths[rid] = start + len(entry.tokens)
            self.cache.trim(entry.cache, self.lengths[rid])
        for rid in step.get("end", []):
            rid = str(rid)
            req = self.requests.pop(rid, None)
            if req is None:
                raise InvalidArgument(f"request '{rid}' ends but was never seen")
            self.cache.release(req)
            del self.lengths[rid]
        return logits
