"""The engine: requests in, tokens out, one step at a time.

The scheduler picks the work, the engine builds the batch, runs the step
function, samples, and finishes sequences (``src/engine/engine.cpp:26-235`` of
the reference, whose behaviour this follows):

* ``add_request`` rejects only what can never run - an empty prompt, a token id
  outside the vocabulary, a prompt that leaves no room for one generated token
  in the context, the page pool or a block-table row - and clamps ``max_tokens``
  to the room that is left;
* a step that fails before progress is recorded gives back the pages reserved
  for it and is offered again; a failure while sampling finishes the affected
  sequences with an error and frees what they hold;
* a sequence samples once all its known tokens are cached; it finishes on a
  stop token (kept in the output) or at ``max_tokens``.
"""

from __future__ import annotations

import dataclasses
import time
from typing import Callable, Dict, List, Optional, Sequence as Seq

import torch

from ..cache.manager import CacheManager
from ..errors import CapacityError, InvalidArgument
from ..models.builder import Model
from ..sampling.params import SamplingParams
from ..sampling.sampler import DeviceSampler
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import BatchScheduler, ScheduledBatch, SchedulerConfig
from .sequence import FinishReason, SeqState, Sequence
from .serving import ServingConfig


@dataclasses.dataclass
class EngineStats:
    steps: int = 0
    seqs_scheduled: int = 0      # summed over steps; divided by steps it is the mean batch size
    prefill_tokens: int = 0      # prompt tokens, and tokens recomputed after preemption
    decode_tokens: int = 0
    step_seconds: float = 0.0    # time in the model's step function
    preemptions: int = 0


class Engine:
    def __init__(self, model: Model, cache: CacheManager, scheduler=None, serving: Optional[ServingConfig] = None,
                 stop_tokens: Seq[int] = (), max_seq_len: Optional[int] = None, use_graphs: Optional[bool] = None):
        self.model = model
        self.cache = cache
        self.serving = serving or ServingConfig()
        self.serving.validate()
        self.scheduler = scheduler or BatchScheduler(cache, SchedulerConfig(serving=self.serving))
        self.stop_tokens = set(int(t) for t in stop_tokens)
        self.runner = ModelRunner(model, cache, max_seq_len, use_graphs=use_graphs)
        self.sampler = DeviceSampler(model.device)
        self.sequences: Dict[int, Sequence] = {}
        self.on_token: Optional[Callable[[int, int], None]] = None
        self._stats = EngineStats()
        self._next_id = 0
        self._stepping = False

    # -------------------------------------------------------------- requests
    def add_request(self, prompt: Seq[int], params: Optional[SamplingParams] = None) -> int:
        params = dataclasses.replace(params) if params is not None else SamplingParams()
        params.validate()
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise InvalidArgument("prompt is empty")
        vocab = self.model.spec.vocab_size
        for t in prompt:
            if not 0 <= t < vocab:
                raise InvalidArgument(f"prompt token {t} outside vocabulary of {vocab}")
        # Most tokens (prompt included) one sequence can hold: the context, the whole pool, one block-table row.
        bs = self.cache.block_size
        context_cap = self.model.spec.max_positions
        pool_cap = self.cache.num_blocks * bs
        row_cap = self.runner.max_blocks_per_seq * bs
        n = len(prompt)
        if n >= context_cap:
            raise CapacityError(f"prompt of {n} tokens leaves no room to generate in the model context of {context_cap}")
        if n >= pool_cap:
            raise CapacityError(
                f"prompt of {n} tokens plus one generated token needs {self.cache.blocks_for(n + 1)} KV blocks "
                f"but the cache holds {self.cache.num_blocks}; raise --kv-mem")
        if n >= row_cap:
            raise CapacityError(
                f"prompt of {n} tokens needs {self.cache.blocks_for(n + 1)} KV blocks but a sequence may hold "
                f"{self.runner.max_blocks_per_seq}")
        params.max_tokens = min(params.max_tokens, min(context_cap, pool_cap, row_cap) - n)
        seq = Sequence(self._next_id, prompt, params, self.cache.new_request())
        self._next_id += 1
        self.scheduler.add(seq)
        self.sequences[seq.id] = seq
        return seq.id

    def sequence(self, seq_id: int) -> Sequence:
        try:
            return self.sequences[seq_id]
        except KeyError:
            raise InvalidArgument(f"no sequence with id {seq_id}") from None

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def cancel(self, seq_id: int) -> None:
        seq = self.sequence(seq_id)
        if seq.state != SeqState.FINISHED:
            self._finish(seq, FinishReason.CANCELLED)

    def release(self, seq_id: int) -> None:
        if self._stepping:
            raise InvalidArgument(f"cannot release sequence {seq_id} during a step")
        if self.sequence(seq_id).state != SeqState.FINISHED:
            raise InvalidArgument(f"sequence {seq_id} is still running")
        del self.sequences[seq_id]

    def stats(self) -> EngineStats:
        s = dataclasses.replace(self._stats)
        s.preemptions = self.scheduler.num_preemptions
        return s

    # ------------------------------------------------------------------ step
    def _check_batch(self, batch: ScheduledBatch) -> None:
        """A scheduler's mistake must fail loudly before any compute or progress (engine.cpp:65-92)."""
        if len(batch.seqs) > self.serving.max_seqs:
            raise InvalidArgument(f"scheduler gave {len(batch.seqs)} sequences; a step allows at most {self.serving.max_seqs}")
        seen = set()
        total = 0
        for s in batch.seqs:
            seq = s.seq
            if s.num_tokens <= 0 or s.num_tokens > seq.num_pending:
                raise InvalidArgument(
                    f"scheduler gave sequence {seq.id} {s.num_tokens} tokens; it has {seq.num_pending} pending")
            if id(seq) in seen:
                raise InvalidArgument(f"scheduler gave sequence {seq.id} twice in one step")
            seen.add(id(seq))
            end = seq.num_computed + s.num_tokens
            need = self.cache.blocks_for(end)
            for g in self.cache.plan.paged_groups:
                have = len(seq.cache.tables[g])
                if have < need or have > self.runner.max_blocks_per_seq:
                    raise InvalidArgument(
                        f"sequence {seq.id} has {have} KV blocks reserved; {end} tokens need {need} and a row holds "
                        f"at most {self.runner.max_blocks_per_seq}")
            total += s.num_tokens
        if total > self.serving.max_tokens_per_step:
            raise InvalidArgument(f"scheduler gave {total} tokens; a step allows at most {self.serving.max_tokens_per_step}")

    def step(self) -> None:
        if self._stepping:
            raise InvalidArgument("step() called during a step (e.g. from a token callback)")
        batch = self.scheduler.schedule()
        if not batch:
            return
        self._stepping = True
        try:
            self._run(batch)
        finally:
            self._stepping = False

    def _run(self, batch: ScheduledBatch) -> None:
        sampled: List[Sequence] = []
        prefill_tokens = decode_tokens = 0
        try:
            self._check_batch(batch)
            entries = []
            for s in batch.seqs:
                seq = s.seq
                begin, end = seq.num_computed, seq.num_computed + s.num_tokens
                # A decode is the single newest token of a sequence that was already decoding; a prompt
                # portion, or tokens recomputed after preemption, is prefill (engine.cpp:121-124).
                if seq.state == SeqState.DECODING and s.num_tokens == 1:
                    decode_tokens += 1
                else:
                    prefill_tokens += s.num_tokens
                want = ()
                if end == len(seq.tokens):     # a sequence samples once its whole pending input is cached
                    want = (s.num_tokens - 1,)
                    sampled.append(seq)
                entries.append(StepEntry(seq.cache, begin, seq.tokens[begin:end], want))
            started = time.perf_counter()
            logits = self.runner.step(entries)      # queued on the GPU; sampling below is queued right behind it
            self._stats.steps += 1
            self._stats.seqs_scheduled += len(batch.seqs)
            self._stats.prefill_tokens += prefill_tokens
            self._stats.decode_tokens += decode_tokens
        except BaseException:
            # The step never ran: give back what the scheduler reserved for it, and let it be scheduled again.
            for s in batch.seqs:
                self.cache.truncate(s.seq.cache, s.seq.num_computed)
            self.scheduler.abandon(batch)
            raise

        for s in batch.seqs:
            s.seq.num_computed += s.num_tokens
            self.cache.trim(s.seq.cache, s.seq.num_computed)
        self.scheduler.complete(batch)
        if not sampled:
            self._stats.step_seconds += time.perf_counter() - started
            return

        try:
            tokens = self.sampler.sample_rows(logits, [q.params for q in sampled], [q.rng for q in sampled])
        except BaseException:
            for seq in sampled:
                if seq.state != SeqState.FINISHED:
                    self._finish(seq, FinishReason.ERROR)
            raise
        self._stats.step_seconds += time.perf_counter() - started   # reading the tokens waited for the GPU
        for i, seq in enumerate(sampled):
            if seq.state == SeqState.FINISHED:      # cancelled by an earlier token callback of this step
                continue
            token = tokens[i]
            try:
                seq.tokens.append(token)
                seq.state = SeqState.DECODING
                if self.on_token is not None:
                    self.on_token(seq.id, token)
            except BaseException:
                # Sequences after it already count this step as computed but will never get its token.
                for later in sampled[i:]:
                    if later.state != SeqState.FINISHED:
                        self._finish(later, FinishReason.ERROR)
                raise
            if seq.state == SeqState.FINISHED:      # its own callback cancelled it
                continue
            if token in self.stop_tokens:
                self._finish(seq, FinishReason.STOP)
            elif seq.num_generated >= seq.params.max_tokens:
                self._finish(seq, FinishReason.LENGTH)

    def _finish(self, seq: Sequence, reason: FinishReason) -> None:
        seq.state = SeqState.FINISHED
        seq.finish_reason = reason
        self.cache.release(seq.cache)
        self.scheduler.finish(seq)

    # -------------------------------------------------------------- generate
    def generate(self, prompt: Seq[int], params: Optional[SamplingParams] = None) -> List[int]:
        """Runs one request to completion; returns its generated tokens, a final stop token included."""
        seq_id = self.add_request(prompt, params)
        try:
            while self.sequence(seq_id).state != SeqState.FINISHED:
                self.step()
        except BaseException:
            seq = self.sequences.get(seq_id)
            if seq is not None:
                if seq.state != SeqState.FINISHED:
                    self._finish(seq, FinishReason.ERROR)
                del self.sequences[seq_id]
            raise
        out = self.sequence(seq_id).generated
        self.release(seq_id)
        return out
