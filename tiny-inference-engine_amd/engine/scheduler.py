"""Which request runs how many tokens in the next step.

The policy is the one of the reference's scheduler (``src/engine/batch_scheduler.cpp:78-174``:
continuous batching, prompts in portions, admission by free pages, preemption by recompute); the
code is organised around three small things of its own:

* a ``StepPlan``: the shares (sequence, number of tokens) of one step;
* a ``_Budget``: what a step may still take, in tokens and in sequences;
* ``_make_room``: the one place that decides what happens when pages run out.

A step is planned in rounds, each a method, each spending the same budget:

``_advance_decoders``  every sequence with exactly one token to run (a decode) goes first, oldest
                       first, so that a running request never waits behind new prompts;
``_continue_prompts``  sequences in the middle of their prompt take the next portion, as large as the
                       budget, the portion cap (``prefill_chunk``) and the free pages allow;
``_admit``             waiting sequences enter in policy order (first come first served, or least
                       remaining work first where a waiting step counts ``aging`` tokens). Admission
                       keeps ``watermark`` pages free for the running ones to grow into and stops at the
                       first sequence that does not fit: a large request is not overtaken for ever.
                       What has to fit is the first portion, as in the reference, or with ``admit_whole``
                       all of the sequence's pending input: a long prompt then enters only when the pool
                       can hold it, instead of entering on its first portion and being evicted, or evicting
                       others, on a later one;
``_unblock_oldest``    only if all of that produced nothing: the oldest idle running sequence takes
                       pages from newer ones until it can move, so the engine never stalls.

When pages run out (``_make_room``), the sequence that needs one evicts the NEWEST sequence admitted
after it that is idle and holds pages: the victim's pages and state slot go back, its tokens
(prompt and generated) stay, and it waits to be admitted and computed again from its first token.
With nobody to evict but a newer sequence still in an unfinished step, the sequence sits this step
out (that step's end will free or advance something); otherwise it evicts itself. Sequences older
than the one in need are never touched, so the oldest running sequence always finishes.

When the engine is in its steady state - nobody waiting, every running sequence decoding, pages
for all of them - the rounds would hand every sequence one token; ``_steady_decode`` sees that
without walking through them.

Deciding a step (``schedule``) is separate from ending it (``complete`` after it ran, ``abandon`` if
it never did): a sequence of a planned step that has not ended is "in flight" and is left alone.
"""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional

from ..cache.manager import CacheManager
from ..errors import InvalidArgument
from .sequence import SeqState, Sequence
from .serving import ServingConfig

FCFS = "fcfs"
SRPT_AGING = "srpt-aging"
POLICIES = (FCFS, SRPT_AGING)


def parse_policy(name: str) -> str:
    if name not in POLICIES:
        raise InvalidArgument(f"unknown scheduling policy '{name}': choose one of {', '.join(POLICIES)}")
    return name


@dataclasses.dataclass
class SchedulerConfig:
    serving: ServingConfig = dataclasses.field(default_factory=ServingConfig)
    policy: str = SRPT_AGING
    aging: int = 16                # srpt-aging: tokens of priority a sequence gains per step it waits
    watermark_blocks: int = -1     # pages that admission leaves free; -1 picks max(1, 1 % of the pool)
    admit_whole: bool = False      # admission counts pages for all of a sequence's pending input, not its first portion


class Share:
    """One sequence's part of a step."""

    __slots__ = ("seq", "num_tokens")

    def __init__(self, seq: Sequence, num_tokens: int):
        self.seq = seq
        self.num_tokens = num_tokens


class StepPlan:
    """The shares of one step, in the order they were granted."""

    def __init__(self, plan_id: int = 0):
        self.id = plan_id
        self.seqs: List[Share] = []
        self._tokens: Dict[int, int] = {}      # id(sequence) -> tokens granted
        self.total_tokens = 0

    def grant(self, seq: Sequence, num_tokens: int) -> None:
        self.seqs.append(Share(seq, num_tokens))
        self._tokens[id(seq)] = num_tokens
        self.total_tokens += num_tokens

    def tokens_of(self, seq: Sequence) -> int:
        return self._tokens.get(id(seq), 0)

    def __bool__(self) -> bool:
        return bool(self.seqs)

    def __len__(self) -> int:
        return len(self.seqs)


class _Budget:
    """What the step being planned may still take."""

    __slots__ = ("tokens", "seats")

    def __init__(self, tokens: int, seats: int):
        self.tokens = tokens
        self.seats = seats

    def spent(self) -> bool:
        return self.tokens <= 0 or self.seats <= 0


# outcomes of _make_room
_ROOM, _SIT_OUT, _EVICTED_ITSELF, _NO_ROOM = range(4)


class BatchScheduler:
    def __init__(self, cache: CacheManager, config: Optional[SchedulerConfig] = None):
        self.cache = cache
        self.config = config or SchedulerConfig()
        self.config.serving.validate()
        parse_policy(self.config.policy)
        if self.config.aging < 0:
            raise InvalidArgument(f"aging counts tokens per waited step and cannot be negative ({self.config.aging})")
        asked = self.config.watermark_blocks
        if asked < -1 or asked >= cache.num_blocks:
            raise InvalidArgument(f"a watermark of {asked} pages is neither -1 (choose for me) nor smaller than "
                                  f"the pool of {cache.num_blocks} pages")
        self.watermark = asked if asked >= 0 else max(1, cache.num_blocks // 100)
        self.waiting: List[Sequence] = []
        self.running: List[Sequence] = []      # in order of admission: the oldest first
        self.num_preemptions = 0
        self.steady_steps = 0                  # steps planned by _steady_decode
        self._clock = 0                        # counts planned steps; waiting times are measured in it
        self._next_plan_id = 1

    # ------------------------------------------------------------- interface
    def add(self, seq: Sequence) -> None:
        seq.state = SeqState.WAITING
        seq.waiting_since_step = self._clock
        seq.in_flight = False
        self.waiting.append(seq)

    def has_work(self) -> bool:
        return bool(self.waiting) or bool(self.running)

    def complete(self, plan: StepPlan) -> None:
        """The step ran: its sequences may be planned again."""
        for share in plan.seqs:
            share.seq.in_flight = False

    def abandon(self, plan: StepPlan) -> None:
        """The step never ran (the caller has given its pages back): its sequences may be planned again."""
        for share in plan.seqs:
            share.seq.in_flight = False

    def finish(self, seq: Sequence) -> None:
        """Forgets a sequence wherever it is; the caller gives back what it holds."""
        for queue in (self.waiting, self.running):
            for i, other in enumerate(queue):
                if other is seq:
                    del queue[i]
                    break
        seq.in_flight = False

    # -------------------------------------------------------------- planning
    def schedule(self) -> StepPlan:
        self._clock += 1
        plan = StepPlan(self._next_plan_id)
        self._next_plan_id += 1
        serving = self.config.serving
        budget = _Budget(serving.max_tokens_per_step, serving.max_seqs)
        if not self._steady_decode(plan, budget):
            self._advance_decoders(plan, budget)
            self._continue_prompts(plan, budget)
            self._admit(plan, budget)
            if not plan:
                self._unblock_oldest(plan, budget)
        for share in plan.seqs:
            share.seq.in_flight = True
        return plan

    def _grant(self, plan: StepPlan, budget: _Budget, seq: Sequence, num_tokens: int) -> None:
        if not self.cache.reserve(seq.cache, seq.num_computed + num_tokens):
            raise InvalidArgument(f"internal error of the scheduler: it granted sequence {seq.id} {num_tokens} tokens "
                                  f"after counting pages for them, and the cache has no room for them")
        plan.grant(seq, num_tokens)
        budget.tokens -= num_tokens
        budget.seats -= 1

    def _portion(self, seq: Sequence, budget: _Budget) -> int:
        """How much of its pending input a sequence would take if pages were no concern."""
        cap = self.config.serving.prefill_chunk
        n = min(seq.num_pending, budget.tokens)
        return min(n, cap) if cap > 0 else n

    def _steady_decode(self, plan: StepPlan, budget: _Budget) -> bool:
        """Every running sequence decodes, nobody waits, and there is a page for each that needs one."""
        running = self.running
        if self.waiting or not running or len(running) > min(budget.seats, budget.tokens):
            return False
        block_size = self.cache.block_size
        at_page_edge = 0
        for seq in running:
            if seq.in_flight or len(seq.tokens) - seq.num_computed != 1:
                return False
            if seq.num_computed % block_size == 0:
                at_page_edge += 1
        if at_page_edge and not self.cache.has_free_pages(at_page_edge):
            return False
        for seq in running:
            if seq.num_computed % block_size == 0:     # the others' last page has room: nothing to reserve
                self._grant(plan, budget, seq, 1)
            else:
                plan.grant(seq, 1)
        self.steady_steps += 1
        return True

    def _advance_decoders(self, plan: StepPlan, budget: _Budget) -> None:
        for seq in list(self.running):
            if budget.spent():
                return
            if seq.in_flight or seq.num_pending != 1 or seq.state == SeqState.WAITING:   # WAITING: evicted just now
                continue
            if self._make_room(seq, 1, may_give_way=True) == _ROOM:
                self._grant(plan, budget, seq, 1)

    def _continue_prompts(self, plan: StepPlan, budget: _Budget) -> None:
        for seq in list(self.running):
            if budget.spent():
                return
            if seq.in_flight or seq.num_pending <= 1 or plan.tokens_of(seq):
                continue
            n = self.cache.fit(seq.cache, seq.num_computed, self._portion(seq, budget))
            if n > 0:
                self._grant(plan, budget, seq, n)

    def _priority(self, seq: Sequence):
        waited = self._clock - seq.waiting_since_step
        work = seq.num_pending - self.config.aging * waited if self.config.policy == SRPT_AGING else 0
        return (work, seq.waiting_since_step, seq.id)

    def _admit(self, plan: StepPlan, budget: _Budget) -> None:
        if not self.waiting:
            return
        self.waiting.sort(key=self._priority)
        entered = set()
        for seq in self.waiting:
            if budget.spent() or len(self.running) >= self.config.serving.max_seqs:
                break
            if seq.num_preemptions and seq.waiting_since_step == self._clock:
                continue                       # evicted while this very step was planned: it waits a step
            n = self._portion(seq, budget)
            counted = seq.num_pending if self.config.admit_whole else n
            if not self.cache.can_admit(counted, self.watermark if self.running else 0):
                break
            seq.state = SeqState.PREFILLING
            self.running.append(seq)
            self._grant(plan, budget, seq, n)
            entered.add(id(seq))
        if entered:         # by identity, not by state: nothing but admission takes a sequence out of this queue
            self.waiting = [s for s in self.waiting if id(s) not in entered]

    def _unblock_oldest(self, plan: StepPlan, budget: _Budget) -> None:
        for seq in self.running:
            if seq.in_flight:
                continue
            want = self._portion(seq, budget)
            self._make_room(seq, want, may_give_way=False)
            n = self.cache.fit(seq.cache, seq.num_computed, want)
            if n > 0:
                self._grant(plan, budget, seq, n)
            return

    # ------------------------------------------------------------- out of pages
    def _make_room(self, seq: Sequence, want: int, may_give_way: bool) -> int:
        """Evicts newer sequences until ``seq`` can run at least one of ``want`` tokens.

        ``may_give_way``: with nobody left to evict, the sequence itself yields - it sits the step out if a
        newer sequence is in flight, else it is evicted. Without it the answer is just _NO_ROOM.
        """
        while self.cache.fit(seq.cache, seq.num_computed, want) == 0:
            victim, newer_in_flight = None, False
            for other in reversed(self.running):
                if other is seq:
                    break
                if other.in_flight:
                    newer_in_flight = True
                elif self.cache.holds_pages(other.cache):
                    victim = other
                    break
            if victim is not None:
                self._evict(victim)
                continue
            if not may_give_way:
                return _NO_ROOM
            if newer_in_flight:
                return _SIT_OUT
            self._evict(seq)
            return _EVICTED_ITSELF
        return _ROOM

    def _evict(self, seq: Sequence) -> None:
        self.cache.release(seq.cache)
        seq.num_computed = 0                   # prompt and generated tokens stay: all are computed again
        seq.state = SeqState.WAITING
        seq.waiting_since_step = self._clock
        seq.num_preemptions += 1
        self.num_preemptions += 1
        for i, other in enumerate(self.running):
            if other is seq:
                del self.running[i]
                break
        self.waiting.append(seq)
