"""The engine: requests in, tokens out, one step at a time.

One ``step()`` is: the scheduler plans (which sequence, how many tokens); the plan becomes the
entries of one batch; the step function runs them; progress is recorded; the sequences whose
whole input is now cached sample their next token. The behaviour towards the caller is the
reference engine's (``src/engine/engine.cpp:26-235``):

* ``add_request`` turns away only what could never run - no tokens, a token id the vocabulary does
  not have, a prompt that leaves no room for a single generated token in the context, in the page
  pool or in a block-table row - and shortens ``max_tokens`` to the room there is;
* a step that fails before its progress is recorded gives its pages back and will be planned
  again; a failure after that (sampling, a token callback) ends the affected sequences with
  ``FinishReason.ERROR`` and frees what they hold, since their cache already counts the step;
* a sequence ends on a stop token (which stays in its output) or after ``max_tokens`` tokens.

Reading ahead (``launch_ahead``, not in the reference). A step's host work - planning, the batch arrays,
the launches - lies between two steps while the GPU idles, because the next step's tokens are the ones just
sampled. With ``launch_ahead`` a step only queues its sampling kernels and leaves the tokens unread; the next
call to ``step()`` plans and queues the next step first - the rows that continue a sequence whose token is
unread take it on the GPU from the sampling kernels' own output - and reads the earlier step's tokens while
that one runs. Nothing in a plan depends on the value of an unread token, only on its existence: which
sequences decode, which prompts go on, who is admitted. Two things need the token itself and are read before
planning: a sequence whose unread token is its last (it ends, and planning it again would be wrong), and rows
that draw from a random stream unless the step is the steady repetition of the one before (they carry both
uniform numbers their stream may be at, see ``DeviceSampler``, which asks for the same rows in the same order).
A sequence that turns out to have met a stop token has then run a token too many for each step queued behind
its last, which are dropped. ``launch_ahead`` is also the number of steps that may stay unread once a step is
queued (True: 1). More than one lets the host's quick steps run further ahead of its slow ones; measured on 64
requests through a small cache it gains nothing over one (the GPU is then the limit) and makes the slowest
gaps between a request's tokens longer, so one is the default. Tokens (and callbacks) appear that many
``step()`` calls later; ``has_work()`` stays true until they have.
"""

from __future__ import annotations

import collections
import dataclasses
import time
from typing import Callable, Deque, Dict, List, Optional, Sequence as Seq, Tuple, Union

from .. import kernels
from ..cache.manager import CacheManager
from ..errors import CapacityError, InvalidArgument
from ..models.builder import Model
from ..sampling.params import SamplingParams
from ..sampling.sampler import DeviceSampler
from .batch import StepEntry
from .runner import ModelRunner
from .scheduler import BatchScheduler, SchedulerConfig, StepPlan
from .sequence import UNREAD, FinishReason, SeqState, Sequence
from .serving import ServingConfig


@dataclasses.dataclass
class EngineStats:
    steps: int = 0
    seqs_scheduled: int = 0      # summed over steps; divided by steps it is the mean batch size
    prefill_tokens: int = 0      # prompt tokens, and tokens recomputed after preemption
    decode_tokens: int = 0
    step_seconds: float = 0.0    # from handing a batch to the step function until its tokens are read
    preemptions: int = 0


class _PlanAgain(Exception):
    """A plan was overtaken by what reading the unread steps showed; nothing of it has run."""


class _Unread:
    """A launched step whose sampled tokens the host has not read: who sampled, where each token goes."""

    __slots__ = ("sampling", "places", "ticket")

    def __init__(self, sampling, places, ticket):
        self.sampling = sampling      # the sequences that sampled, in the order of the step's rows
        self.places = places          # per sequence, the index in its tokens that holds UNREAD
        self.ticket = ticket


class Engine:
    def __init__(self, model: Model, cache: CacheManager, scheduler=None, serving: Optional[ServingConfig] = None,
                 stop_tokens: Seq[int] = (), max_seq_len: Optional[int] = None, use_graphs: Optional[bool] = None,
                 launch_ahead: Union[bool, int] = False, runner=None, sampler=None):
        """``runner`` / ``sampler``: stand-ins with the interface of ``ModelRunner`` (``step``,
        ``max_blocks_per_seq``) and ``DeviceSampler`` (``launch_greedy``, ``launch``, ``collect``,
        ``sample_rows``), for driving the engine's bookkeeping without a GPU; the default builds the real ones."""
        self.model = model
        self.cache = cache
        self.serving = serving or ServingConfig()
        self.serving.validate()
        if self.serving.max_tokens_per_step > kernels.MAX_STEP_TOKENS:
            raise InvalidArgument(f"max_tokens_per_step of {self.serving.max_tokens_per_step} exceeds the "
                                  f"{kernels.MAX_STEP_TOKENS} rows the kernels take in one step")
        self.scheduler = scheduler or BatchScheduler(cache, SchedulerConfig(serving=self.serving))
        self.stop_tokens = frozenset(int(t) for t in stop_tokens)
        self.runner = runner if runner is not None else ModelRunner(model, cache, max_seq_len, use_graphs=use_graphs)
        self.sampler = sampler if sampler is not None else DeviceSampler(model.device)
        self.sequences: Dict[int, Sequence] = {}
        self.on_token: Optional[Callable[[int, int], None]] = None     # (sequence id, token), as each token is known
        self._stats = EngineStats()
        self._ids = 0
        self._inside_step = False
        # How many launched steps may stay unread after a step has been queued (0: every step is read at once).
        self.launch_ahead = 1 if launch_ahead is True else max(0, int(launch_ahead))
        if self.launch_ahead and hasattr(self.sampler, "keep_apart"):
            self.sampler.keep_apart(self.launch_ahead + 2)      # result buffers of the unread steps and the next
        self._unread: Deque[_Unread] = collections.deque()      # oldest first
        self.steps_launched_ahead = 0
        self.ahead_replans = 0      # steps planned over unread tokens whose plan was not the steady one after all

    # -------------------------------------------------------------- requests
    def _token_limits(self) -> List[Tuple[int, str]]:
        """The three ceilings on a sequence's length (prompt and generated together), each with its name."""
        page = self.cache.block_size
        return [(self.model.spec.max_positions, "the model's context"),
                (self.cache.capacity_tokens, f"the cache of {self.cache.num_blocks} pages (see --kv-mem)"),
                (self.runner.max_blocks_per_seq * page, f"a block-table row of {self.runner.max_blocks_per_seq} pages")]

    def add_request(self, prompt: Seq[int], params: Optional[SamplingParams] = None) -> int:
        params = dataclasses.replace(params) if params is not None else SamplingParams()
        params.validate()
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise InvalidArgument("a request needs at least one prompt token")
        vocab = self.model.spec.vocab_size
        if not params.greedy:
            filtered = 0 < params.top_k < vocab or params.top_p < 1.0
            most = kernels.MAX_FILTERED_VOCAB if filtered else kernels.MAX_SAMPLED_VOCAB
            if vocab > most:
                raise InvalidArgument(f"the sampling kernel for {'top-k / top-p' if filtered else 'a temperature'} takes "
                                      f"vocabularies of up to {most} tokens, this model has {vocab}")
        if min(prompt) < 0 or max(prompt) >= vocab:
            bad = next(t for t in prompt if not 0 <= t < vocab)
            raise InvalidArgument(f"prompt token {bad} is not in the vocabulary of {vocab}")
        n = len(prompt)
        ceiling, what = min(self._token_limits(), key=lambda limit: limit[0])    # ties: the first named
        if n + 1 > ceiling:
            raise CapacityError(f"a prompt of {n} tokens and one generated token make {n + 1}; {what} holds "
                                f"{ceiling}")
        params.max_tokens = min(params.max_tokens, ceiling - n)
        seq = Sequence(self._ids, prompt, params, self.cache.new_request())
        self._ids += 1
        self.sequences[seq.id] = seq
        self.scheduler.add(seq)
        return seq.id

    def sequence(self, seq_id: int) -> Sequence:
        seq = self.sequences.get(seq_id)
        if seq is None:
            raise InvalidArgument(f"the engine knows no sequence {seq_id}")
        return seq

    def has_work(self) -> bool:
        return self.scheduler.has_work() or bool(self._unread)

    def cancel(self, seq_id: int) -> None:
        seq = self.sequence(seq_id)
        if seq.state != SeqState.FINISHED:
            self._end(seq, FinishReason.CANCELLED)

    def release(self, seq_id: int) -> None:
        """Forgets a finished sequence (its tokens with it)."""
        if self._inside_step:
            raise InvalidArgument(f"sequence {seq_id} cannot be released from inside a step")
        if self.sequence(seq_id).state != SeqState.FINISHED:
            raise InvalidArgument(f"sequence {seq_id} has not finished; cancel it first")
        del self.sequences[seq_id]

    def stats(self) -> EngineStats:
        return dataclasses.replace(self._stats, preemptions=self.scheduler.num_preemptions)

    def _end(self, seq: Sequence, reason: FinishReason) -> None:
        while seq.tokens and seq.tokens[-1] == UNREAD:      # tokens of steps that ran past its end
            seq.tokens.pop()
        seq.state = SeqState.FINISHED
        seq.finish_reason = reason
        self.cache.release(seq.cache)
        self.scheduler.finish(seq)

    # ------------------------------------------------------------------ step
    def step(self) -> None:
        if self._inside_step:
            raise InvalidArgument("step() was called from inside a step (a token callback?)")
        self._inside_step = True
        try:
            while self._unread and not self._may_plan_over():
                self._read_oldest()                # a token is needed for the plan itself: know it first
            plan = self.scheduler.schedule()
            if plan:
                self._carry_out(plan)
            else:
                self._read_all()
        finally:
            self._inside_step = False

    def _may_plan_over(self) -> bool:
        """Whether the next step can be planned while the tokens of the unread steps are still on the GPU."""
        if any(not seq.params.greedy for unread in self._unread for seq in unread.sampling):
            # rows that draw: only the same rows again, in the same order, and one step of them at a time
            return len(self._unread) == 1 and self._steady(self._unread[0])
        for unread in self._unread:
            for seq in unread.sampling:
                if seq.state == SeqState.FINISHED:     # cancelled meanwhile: its token will be dropped
                    continue
                if seq.state != SeqState.DECODING or seq.tokens[-1] != UNREAD:
                    return False
                if len(seq.tokens) - seq.prompt_len >= seq.params.max_tokens:    # an unread token is its last
                    return False
        return True

    def _steady(self, unread: _Unread) -> bool:
        """Whether the next step is the one before once more: the very same sequences decode, nobody waits."""
        running = self.scheduler.running
        if self.scheduler.waiting or len(running) != len(unread.sampling):
            return False
        for seq, sampled in zip(running, unread.sampling):
            if seq is not sampled or len(seq.tokens) - seq.num_computed != 1:
                return False
            if len(seq.tokens) - seq.prompt_len >= seq.params.max_tokens:    # the unread token is its last
                return False
        return True

    def _entries_of(self, plan: StepPlan, unread_rows: Optional[Dict[int, int]] = None):
        """The plan as batch entries, checked on the way: a planner's mistake stops here, before any compute.

        ``unread_rows``: for the sequences whose last token is still on the GPU, its place among the tokens the
        step before left there. Returns (entries, the sequences that sample after this step, prompt tokens,
        decoded tokens).
        """
        serving = self.serving
        if len(plan.seqs) > serving.max_seqs or plan.total_tokens > serving.max_tokens_per_step:
            raise InvalidArgument(f"the plan holds {len(plan.seqs)} sequences and {plan.total_tokens} tokens; a step "
                                  f"takes {serving.max_seqs} and {serving.max_tokens_per_step}")
        entries, sampling, seen = [], [], set()
        prompt_tokens = decoded_tokens = 0
        groups = self.cache.plan.paged_groups
        row_pages = self.runner.max_blocks_per_seq
        for share in plan.seqs:
            seq, n = share.seq, share.num_tokens
            if not 0 < n <= seq.num_pending or id(seq) in seen:
                raise InvalidArgument(f"the plan gives sequence {seq.id} {n} tokens (it has {seq.num_pending} to run), "
                                      f"or names it twice")
            seen.add(id(seq))
            first, last = seq.num_computed, seq.num_computed + n
            pages = self.cache.blocks_for(last)
            for g in groups:
                held = len(seq.cache.tables[g])
                if not pages <= held <= row_pages:
                    raise InvalidArgument(f"sequence {seq.id} holds {held} pages of cache group {g}: {last} tokens "
                                          f"take {pages}, a block-table row {row_pages}")
            # One new token of a sequence that has sampled before is a decode; everything else (prompt portions,
            # tokens computed again after an eviction) counts as prefill (engine.cpp:121-124).
            if n == 1 and seq.state == SeqState.DECODING:
                decoded_tokens += 1
            else:
                prompt_tokens += n
            tokens = seq.tokens[first:last]
            token_from = -1
            if tokens[-1] == UNREAD:             # the GPU knows it, the host does not: the step takes it from there
                token_from = -1 if unread_rows is None else unread_rows.get(id(seq), -1)
                if n != 1 or token_from < 0:
                    raise InvalidArgument(f"sequence {seq.id} would run {n} tokens, one of them not read yet")
                tokens = (0,)
            if last == len(seq.tokens):          # all it has is cached after this step: it samples
                entries.append(StepEntry(seq.cache, first, tokens, (n - 1,), token_from))
                sampling.append(seq)
            else:
                entries.append(StepEntry(seq.cache, first, tokens, (), token_from))
        return entries, sampling, prompt_tokens, decoded_tokens

    def _carry_out(self, plan: StepPlan) -> None:
        """Runs a plan, over the unread steps if it can: the rows that continue a sequence whose last token is
        still on the GPU take it from the latest unread step's sampling output."""
        try:
            latest = self._unread[-1] if self._unread else None
            unread_rows, repeats = None, False
            if latest is not None:
                unread_rows = {id(seq): row for row, seq in enumerate(latest.sampling)}
                repeats = len(plan.seqs) == len(latest.sampling) and all(
                    share.seq is seq and share.num_tokens == 1 for share, seq in zip(plan.seqs, latest.sampling))
                if not repeats:
                    self.ahead_replans += 1        # (an eviction to make room, a prompt beside the decoders, ...)
                # The plan can run over the unread tokens if every share that ends in one is that one token of a
                # sequence of the latest unread step; rows that draw need that step alone, repeated exactly.
                def continues_latest(share) -> bool:
                    row = unread_rows.get(id(share.seq))
                    return share.num_tokens == 1 and row is not None and \
                        latest.places[row] == share.seq.num_computed == len(share.seq.tokens) - 1
                fits = all(share.seq.tokens[share.seq.num_computed + share.num_tokens - 1] != UNREAD or
                           continues_latest(share) for share in plan.seqs)
                draws = any(not seq.params.greedy for unread in self._unread for seq in unread.sampling)
                if not fits or (draws and not (repeats and len(self._unread) == 1)):
                    self._read_all()
                    latest = unread_rows = None
                    repeats = False
                    for share in [s for s in plan.seqs if s.seq.state == SeqState.FINISHED]:
                        plan.seqs.remove(share)      # it met a stop token; what was reserved for it went back with it
                        plan.total_tokens -= share.num_tokens
                    if not plan.seqs:
                        self.scheduler.complete(plan)
                        return
            entries, sampling, prompt_tokens, decoded_tokens = self._entries_of(plan, unread_rows)
            if latest is not None and any(not seq.params.greedy for seq in sampling) and \
                    not (repeats and len(self._unread) == 1):
                # Rows that begin to draw in this step: their streams stand where the host's do only once
                # everything before has been read (nothing of this step is queued yet).
                self._read_all()
                if any(share.seq.state == SeqState.FINISHED for share in plan.seqs):
                    raise _PlanAgain()
                latest = None
                entries, sampling, prompt_tokens, decoded_tokens = self._entries_of(plan, None)
            began = time.perf_counter()
            # Queued on the GPU; the sampling kernels queue right behind.
            logits = self.runner.step(entries, None if latest is None else latest.ticket.device_tokens)
        except BaseException as error:
            # Nothing of the step counts: the pages reserved for it go back and the plan's sequences are free
            # to be planned again.
            for share in plan.seqs:
                if share.seq.state != SeqState.FINISHED:
                    self.cache.truncate(share.seq.cache, share.seq.num_computed)
            self.scheduler.abandon(plan)
            if isinstance(error, _PlanAgain):
                return                             # the next step() plans afresh, everything read
            raise
        stats = self._stats
        stats.steps += 1
        stats.seqs_scheduled += len(plan.seqs)
        stats.prefill_tokens += prompt_tokens
        stats.decode_tokens += decoded_tokens
        windows = self.cache.has_windows
        for share in plan.seqs:
            seq = share.seq
            seq.num_computed += share.num_tokens
            if windows:
                self.cache.trim(seq.cache, seq.num_computed)     # pages a window has passed go back now
        self.scheduler.complete(plan)
        if latest is not None:
            self.steps_launched_ahead += 1
        tokens: List[int] = []
        if sampling and self.launch_ahead:
            try:
                if all(s.params.greedy for s in sampling):
                    ticket = self.sampler.launch_greedy(logits)
                else:
                    # Rows that drew in the unread step (it is then this step's like: see above) take the number
                    # their stream will be at once that step is read.
                    ticket = self.sampler.launch(logits, [s.params for s in sampling], [s.rng for s in sampling],
                                                 latest.ticket if latest is not None else None)
            except BaseException:
                self._end_all(sampling, FinishReason.ERROR)
                raise
            for seq in sampling:
                seq.tokens.append(UNREAD)
                seq.state = SeqState.DECODING
            self._unread.append(_Unread(sampling, [len(seq.tokens) - 1 for seq in sampling], ticket))
            sampling = []
        elif sampling:
            try:
                tokens = self.sampler.sample_rows(logits, [s.params for s in sampling], [s.rng for s in sampling])
            except BaseException:
                self._end_all(sampling, FinishReason.ERROR)
                raise
        stats.step_seconds += time.perf_counter() - began     # reading the tokens waited for the GPU
        while len(self._unread) > self.launch_ahead:
            self._read_oldest()                                # earlier steps, while this one runs
        if sampling:
            self._deliver(sampling, tokens)

    def _read_oldest(self) -> None:
        """Waits for the oldest unread step's tokens, puts them where UNREAD stands, and delivers them."""
        unread = self._unread.popleft()
        began = time.perf_counter()
        try:
            tokens = self.sampler.collect(unread.ticket)
        except BaseException:
            self._end_all(unread.sampling, FinishReason.ERROR)
            raise
        self._stats.step_seconds += time.perf_counter() - began
        self._deliver(unread.sampling, tokens, unread.places)

    def _read_all(self) -> None:
        while self._unread:
            self._read_oldest()

    def _end_all(self, seqs: Seq[Sequence], reason: FinishReason) -> None:
        for seq in seqs:
            if seq.state != SeqState.FINISHED:
                self._end(seq, reason)

    def _deliver(self, sampling: List[Sequence], tokens: List[int], places: Optional[List[int]] = None) -> None:
        """Hands each sequence its token: appended, or (``places``) written where UNREAD stood for it."""
        callback, stop = self.on_token, self.stop_tokens
        for i, seq in enumerate(sampling):
            if seq.state == SeqState.FINISHED:       # cancelled meanwhile, or by a callback earlier in this loop
                continue
            token = tokens[i]
            if places is None:
                seq.tokens.append(token)
                count = len(seq.tokens) - seq.prompt_len
            else:
                seq.tokens[places[i]] = token
                count = places[i] + 1 - seq.prompt_len       # a later token may stand behind it, still unread
            if seq.state != SeqState.WAITING:    # WAITING: evicted while this token was unread; it stays in the
                seq.state = SeqState.DECODING    # scheduler's waiting queue and is computed again with the token
            if callback is not None:
                try:
                    callback(seq.id, token)
                except BaseException:
                    # The sequences from here on have this step in their cache and will never see its token.
                    self._end_all(sampling[i:], FinishReason.ERROR)
                    raise
                if seq.state == SeqState.FINISHED:   # its own callback cancelled it
                    continue
            if token in stop:
                self._end(seq, FinishReason.STOP)
            elif count >= seq.params.max_tokens:
                self._end(seq, FinishReason.LENGTH)

    # -------------------------------------------------------------- generate
    def generate(self, prompt: Seq[int], params: Optional[SamplingParams] = None) -> List[int]:
        """One request from its prompt to its end; returns the generated tokens (a stop token included)."""
        seq_id = self.add_request(prompt, params)
        seq = self.sequences[seq_id]
        try:
            while seq.state != SeqState.FINISHED:
                self.step()
        except BaseException:
            if seq.state != SeqState.FINISHED:
                self._end(seq, FinishReason.ERROR)
            self.sequences.pop(seq_id, None)
            raise
        self.release(seq_id)
        return seq.generated
