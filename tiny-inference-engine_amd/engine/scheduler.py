"""Continuous batching with chunked prefill, admission by free pages, and preemption by recompute.

The policy is the reference's ``BatchScheduler`` (``src/engine/batch_scheduler.cpp:78-174``).
Each step, under the token budget, the cap on sequences and the free pages:

1. every decoding sequence (one pending token) advances, oldest first. One that needs a page
   when none is free preempts the newest sequence admitted after it that is idle and holds
   pages; if there is none but a newer one is in flight it sits this step out; it preempts
   itself only when no newer sequence holds pages or is in flight;
2. partially prefilled sequences continue in admission order with as much as budget, chunk cap
   and free pages allow;
3. waiting sequences are admitted in policy order (first come first served, or least remaining
   work first with aging). A watermark of pages stays free for running sequences to grow into,
   and admission stops at the first sequence that does not fit, so a large request is not
   overtaken forever. A sequence preempted in this step waits at least one step;
4. if nothing could run, the oldest running sequence preempts newer ones until it can.

When pages run out the answer is therefore preemption by recompute: the victim's pages and state
slot go back, its tokens (prompt and generated) stay, and on re-admission all of them are
prefilled again before it samples its next token. The oldest running sequence is never
preempted, so it always finishes.

Deciding a step (``schedule``) is separate from finishing it (``complete`` / ``abandon``); a
sequence in a batch that is neither completed nor abandoned is not scheduled again.
"""

from __future__ import annotations

import dataclasses
from typing import List, Optional

from ..cache.manager import CacheManager
from ..errors import InvalidArgument
from .sequence import SeqState, Sequence
from .serving import ServingConfig

FCFS = "fcfs"
SRPT_AGING = "srpt-aging"


def parse_policy(name: str) -> str:
    if name not in (FCFS, SRPT_AGING):
        raise InvalidArgument(f"scheduling policy must be fcfs or srpt-aging, got '{name}'")
    return name


@dataclasses.dataclass
class SchedulerConfig:
    serving: ServingConfig = dataclasses.field(default_factory=ServingConfig)
    policy: str = SRPT_AGING
    aging: int = 16                # srpt-aging: priority (in tokens) gained per step waited
    watermark_blocks: int = -1     # pages admission leaves free; -1 = max(1, 1% of the pool)


@dataclasses.dataclass
class ScheduledSeq:
    seq: Sequence
    num_tokens: int


@dataclasses.dataclass
class ScheduledBatch:
    id: int = 0
    seqs: List[ScheduledSeq] = dataclasses.field(default_factory=list)

    def __bool__(self) -> bool:
        return bool(self.seqs)

    def tokens_of(self, seq: Sequence) -> int:
        return next((s.num_tokens for s in self.seqs if s.seq is seq), 0)

    @property
    def total_tokens(self) -> int:
        return sum(s.num_tokens for s in self.seqs)


class BatchScheduler:
    def __init__(self, cache: CacheManager, config: Optional[SchedulerConfig] = None):
        self.cache = cache
        self.config = config or SchedulerConfig()
        self.config.serving.validate()
        parse_policy(self.config.policy)
        if self.config.aging < 0:
            raise InvalidArgument(f"aging must be non-negative, got {self.config.aging}")
        wm = self.config.watermark_blocks
        if wm < -1 or wm >= cache.num_blocks:
            raise InvalidArgument(
                f"watermark of {wm} blocks must be -1 (auto) or below the pool's {cache.num_blocks} blocks")
        self.watermark = wm if wm >= 0 else max(1, cache.num_blocks // 100)
        self.waiting: List[Sequence] = []
        self.running: List[Sequence] = []      # admission order, oldest first
        self._in_flight = set()
        self._step = 0
        self._next_batch_id = 1
        self.num_preemptions = 0

    # ------------------------------------------------------------- interface
    def add(self, seq: Sequence) -> None:
        seq.state = SeqState.WAITING
        seq.waiting_since_step = self._step
        self.waiting.append(seq)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def complete(self, batch: ScheduledBatch) -> None:
        for s in batch.seqs:
            self._in_flight.discard(id(s.seq))

    def abandon(self, batch: ScheduledBatch) -> None:
        for s in batch.seqs:
            self._in_flight.discard(id(s.seq))

    def finish(self, seq: Sequence) -> None:
        self.waiting = [s for s in self.waiting if s is not seq]
        self.running = [s for s in self.running if s is not seq]
        self._in_flight.discard(id(seq))

    # --------------------------------------------------------------- helpers
    def _busy(self, seq: Sequence) -> bool:
        return id(seq) in self._in_flight

    def _order_key(self, seq: Sequence):
        if self.config.policy == SRPT_AGING:
            score = seq.num_pending - self.config.aging * (self._step - seq.waiting_since_step)
            return (score, seq.waiting_since_step, seq.id)
        return (0, seq.waiting_since_step, seq.id)

    def _fit(self, seq: Sequence, want: int) -> int:
        return self.cache.fit(seq.cache, seq.num_computed, want)

    def _chunk(self, seq: Sequence, budget: int) -> int:
        n = min(seq.num_pending, budget)
        cap = self.config.serving.prefill_chunk
        return min(n, cap) if cap > 0 else n

    def _newest_after(self, index: int) -> Optional[Sequence]:
        """The newest running sequence admitted after ``index`` that is idle and holds pages."""
        for j in range(len(self.running) - 1, index, -1):
            cand = self.running[j]
            if not self._busy(cand) and cand.cache.num_held() > 0:
                return cand
        return None

    def _newer_busy(self, index: int) -> bool:
        return any(self._busy(s) for s in self.running[index + 1:])

    def _preempt(self, seq: Sequence) -> None:
        self.cache.release(seq.cache)
        seq.num_computed = 0               # its tokens stay and are recomputed on re-admission
        seq.state = SeqState.WAITING
        seq.waiting_since_step = self._step
        seq.num_preemptions += 1
        self.num_preemptions += 1
        self.running = [s for s in self.running if s is not seq]
        self.waiting.append(seq)

    # -------------------------------------------------------------- schedule
    def schedule(self) -> ScheduledBatch:
        self._step += 1
        batch = ScheduledBatch(id=self._next_batch_id)
        self._next_batch_id += 1
        serving = self.config.serving
        budget = serving.max_tokens_per_step

        def full() -> bool:
            return budget == 0 or len(batch.seqs) == serving.max_seqs

        def take(seq: Sequence, n: int) -> None:
            nonlocal budget
            if not self.cache.reserve(seq.cache, seq.num_computed + n):
                raise InvalidArgument(
                    f"scheduler bug: {n} tokens of sequence {seq.id} do not fit the blocks it counted")
            batch.seqs.append(ScheduledSeq(seq, n))
            budget -= n

        # 1. decodes, oldest first
        i = 0
        while i < len(self.running) and not full():
            seq = self.running[i]
            if self._busy(seq) or seq.num_pending != 1:
                i += 1
                continue
            preempted_self = deferred = False
            while self._fit(seq, 1) == 0:
                victim = self._newest_after(i)
                if victim is None and self._newer_busy(i):
                    deferred = True
                    break
                self._preempt(victim if victim is not None else seq)
                if victim is None:
                    preempted_self = True
                    break
            if deferred:
                i += 1
                continue
            if preempted_self:
                continue                   # running[i] is now the next sequence
            take(seq, 1)
            i += 1

        # 2. partial prefills continue in admission order
        for seq in list(self.running):
            if full():
                break
            if self._busy(seq) or seq.num_pending <= 1 or batch.tokens_of(seq):
                continue
            n = self._fit(seq, self._chunk(seq, budget))
            if n > 0:
                take(seq, n)

        # 3. admission in policy order
        self.waiting.sort(key=self._order_key)
        admitted = []
        for seq in self.waiting:
            if full() or len(self.running) >= serving.max_seqs:
                break
            if seq.num_preemptions > 0 and seq.waiting_since_step == self._step:
                continue                   # preempted in this very step: waits one step
            n = self._chunk(seq, budget)
            keep_free = self.watermark if self.running else 0
            if not self.cache.can_admit(n, keep_free):
                break
            seq.state = SeqState.PREFILLING
            self.running.append(seq)
            take(seq, n)
            admitted.append(seq)
        if admitted:
            self.waiting = [s for s in self.waiting if not any(s is a for a in admitted)]

        # 4. never stall
        if not batch.seqs:
            for i, seq in enumerate(self.running):
                if self._busy(seq):
                    continue
                want = self._chunk(seq, budget)
                while self._fit(seq, want) == 0:
                    victim = self._newest_after(i)
                    if victim is None:
                        break
                    self._preempt(victim)
                n = self._fit(seq, want)
                if n > 0:
                    take(seq, n)
                break

        for s in batch.seqs:
            self._in_flight.add(id(s.seq))
        return batch
