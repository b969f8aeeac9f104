"""The step function: run exactly the tokens given, from the cache, and return the wanted logits.

``ModelRunner.step(entries)`` is the one way tokens pass through a model here:
generation, the scheduler's engine and trace replay all call it. It builds the
step's arrays, runs embedding, the run order and the head on the wanted rows,
and leaves the keys and values of the new tokens in the cache
(``src/model/qwen3.cpp:160-263`` is the reference's step). Pages must have been
reserved by the caller; nothing is sampled here.

Steps that hold only decoded tokens (one new row per sequence) are launch-bound:
a few hundred small kernels. In bfloat16 mode such a step is recorded once per
shape (sequences, wanted rows, context bucket) into a HIP graph and replayed
afterwards; the step's arrays live at fixed addresses in the staging buffer,
so a replay reads the new step's tokens, positions, slots and block tables.
The reference gets the same effect by recording every op of a step into one
command buffer (``src/backend/metal/metal_backend.mm:95-109``).
"""

from __future__ import annotations

from typing import Dict, Optional, Sequence, Tuple

import torch

from .. import kernels
from ..cache.manager import CacheManager
from ..errors import CapacityError, InvalidArgument
from ..models.builder import Model
from ..parts.base import StepContext, Workspace
from ..weights.binder import BFLOAT16
from .batch import BatchBuilder, StepBatch, StepEntry


class _RecordedStep:
    def __init__(self, graph, logits, staging_ptr, generation):
        self.graph = graph
        self.logits = logits
        self.staging_ptr = staging_ptr
        self.generation = generation


class ModelRunner:
    def __init__(self, model: Model, cache: CacheManager, max_seq_len: Optional[int] = None,
                 use_graphs: Optional[bool] = None):
        if model.mode is None:
            raise InvalidArgument("the model has no weights loaded")
        if cache.plan is not model.cache_plan and cache.plan != model.cache_plan:
            raise InvalidArgument("the cache was not planned for this model")
        self.model = model
        self.cache = cache
        self.device = torch.device(model.device)
        limit = model.spec.max_positions
        self.max_seq_len = min(limit, max_seq_len) if max_seq_len else limit
        self.max_blocks_per_seq = cache.blocks_for(self.max_seq_len)
        self.builder = BatchBuilder(cache, model.spec.vocab_size, self.max_blocks_per_seq, self.device)
        self.workspace = Workspace(self.device)
        # Recording needs every part's consent: one part that reads the step's host-side values would
        # bake them into the recording (see Part.capturable). ``use_graphs`` can only switch it off.
        wanted = (model.mode == BFLOAT16) if use_graphs is None else bool(use_graphs)
        self.use_graphs = wanted and self.device.type == "cuda" and model.capturable()
        self._recorded: Dict[Tuple, _RecordedStep] = {}
        self.graph_replays = 0

    def _forward(self, batch: StepBatch) -> Optional[torch.Tensor]:
        ctx = StepContext(batch, self.model.mode, self.device, self.workspace, self.cache, self.model.cache_plan)
        return self.model.forward(ctx)

    def step(self, entries: Sequence[StepEntry], device_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """Runs one batch; returns float32 logits ``[wanted rows, vocab]`` on the device, or None.

        The returned tensor is scratch memory of the runner: it is valid until the next step.

        ``device_tokens`` (int32 on the device): tokens the host does not know yet - an earlier step's sampling
        kernel left them there. An entry with ``token_from >= 0`` brings one token, whose value is
        ``device_tokens[token_from]``; the value the entry itself names is ignored.
        """
        total = 0
        for e in entries:
            if e.start + len(e.tokens) > self.max_seq_len:
                raise InvalidArgument(
                    f"a request would reach {e.start + len(e.tokens)} tokens; the limit is {self.max_seq_len}")
            total += len(e.tokens)
        if total > kernels.MAX_STEP_TOKENS:
            raise CapacityError(f"a step of {total} tokens exceeds the {kernels.MAX_STEP_TOKENS} the kernels take; "
                                f"cut the prompt into portions")
        batch = self.builder.build(entries)
        if batch.takes_device_tokens:
            if device_tokens is None or device_tokens.dtype != torch.int32 or \
                    max(e.token_from for e in entries) >= device_tokens.numel():
                raise InvalidArgument("an entry takes its token from the device: the step needs the int32 tokens an "
                                      "earlier step left there, as many as the entries point into")
            # queued behind the copy of the step's arrays, before any kernel of the step
            kernels.take_tokens(batch.tokens, batch.token_sources, device_tokens)
        if not (self.use_graphs and batch.all_decode and self.model.layer_hook is None):
            return self._forward(batch)

        # A decode-only step: replay its recording, or run it eagerly once and record it for next time.
        key = (batch.num_seqs, batch.num_logit_rows, batch.plan_context, batch.share_key)
        staging_ptr = self.builder.staging_ptr
        recorded = self._recorded.get(key)
        if recorded is not None and recorded.staging_ptr == staging_ptr and \
                recorded.generation == self.workspace.generation:
            recorded.graph.replay()
            self.graph_replays += 1
            return recorded.logits
        logits = self._forward(batch)                    # eager: does the step and settles the workspace
        generation = self.workspace.generation
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):                    # records the same launches; nothing runs here
            recorded_logits = self._forward(batch)
        if self.workspace.generation == generation and self.builder.staging_ptr == staging_ptr:
            self._recorded[key] = _RecordedStep(graph, recorded_logits, staging_ptr, generation)
        return logits
