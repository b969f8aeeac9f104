"""The scheduler's decisions over a real page pool and no model (no GPU).

The scenarios are those of the reference's tests/engine/test_batch_scheduler.cpp and the randomized
simulation of tests/engine/test_batch_scheduler_sim.cpp; the fixture plays the engine's part
between steps (advance num_computed, append a sampled token).
"""

import random

import pytest

from tie_amd.cache.manager import CacheManager
from tie_amd.cache.spec import FixedState, PagedKV, plan_cache
from tie_amd.engine.scheduler import FCFS, SRPT_AGING, BatchScheduler, SchedulerConfig, parse_policy
from tie_amd.engine.sequence import SeqState, Sequence
from tie_amd.engine.serving import ServingConfig
from tie_amd.errors import InvalidArgument
from tie_amd.sampling.params import SamplingParams

PLAN = plan_cache([PagedKV(1, 8)], [None])


def config(max_tokens_per_step, max_seqs, policy=FCFS, watermark=0, aging=16, prefill_chunk=0, admit_whole=False):
    return SchedulerConfig(ServingConfig(max_tokens_per_step, max_seqs, prefill_chunk), policy, aging, watermark,
                           admit_whole)


class Fixture:
    def __init__(self, blocks, cfg, plan=PLAN, state_slots=64):
        self.cache = CacheManager(plan, block_size=4, num_blocks=blocks, max_state_slots=state_slots)
        self.sched = BatchScheduler(self.cache, cfg)
        self.seqs = []

    def add(self, prompt_len, max_tokens=256):
        s = Sequence(len(self.seqs), [1] * prompt_len, SamplingParams(max_tokens=max_tokens), self.cache.new_request())
        self.seqs.append(s)
        self.sched.add(s)
        return s

    def run(self):
        """One engine step: schedule, record progress, complete, append a token where the input is all computed."""
        b = self.sched.schedule()
        for s in b.seqs:
            s.seq.num_computed += s.num_tokens
        self.sched.complete(b)
        for s in b.seqs:
            if s.seq.num_pending == 0:
                s.seq.tokens.append(2)
                s.seq.state = SeqState.DECODING
        return b

    def finish(self, s):
        self.cache.release(s.cache)
        s.state = SeqState.FINISHED
        self.sched.finish(s)

    def blocks(self, s):
        return len(s.cache.tables[0])


def test_decodes_run_first_and_prefill_fills_the_budget():
    f = Fixture(64, config(8, 4))
    a, b = f.add(3), f.add(3)
    s1 = f.run()
    assert s1.tokens_of(a) == 3 and s1.tokens_of(b) == 3
    c = f.add(20)
    for _ in range(3):
        s = f.run()
        assert [(x.seq, x.num_tokens) for x in s.seqs] == [(a, 1), (b, 1), (c, 6)]
        assert s.total_tokens <= 8
    for x in f.run().seqs:
        assert f.blocks(x.seq) == f.cache.blocks_for(x.seq.num_computed)


def test_max_seqs_caps_running_sequences_and_the_rest_wait():
    f = Fixture(64, config(16, 2))
    a, b, c = f.add(2), f.add(2), f.add(2)
    s = f.run()
    assert (s.tokens_of(a), s.tokens_of(b), s.tokens_of(c)) == (2, 2, 0)
    assert c.state == SeqState.WAITING and len(f.sched.running) == 2
    f.finish(a)
    s = f.run()
    assert s.tokens_of(c) == 2 and s.tokens_of(b) == 1


def test_a_one_token_prompt_is_admitted_and_sampled():
    f = Fixture(16, config(8, 2))
    a = f.add(1)
    assert f.run().tokens_of(a) == 1 and a.num_generated == 1
    assert f.run().tokens_of(a) == 1


def test_a_prefill_portion_shrinks_to_the_free_pages():
    f = Fixture(4, config(8, 2))
    x, a = f.add(4), f.add(16)
    s = f.run()
    assert s.tokens_of(x) == 4 and s.tokens_of(a) == 4
    s = f.run()                      # x decodes into a second page, leaving one free
    assert s.tokens_of(x) == 1 and s.tokens_of(a) == 4      # 7 fit the budget; one more page holds only 4
    assert f.cache.num_free() == 0


def test_watermark_stays_free_and_admission_stops_at_a_head_that_does_not_fit():
    f = Fixture(8, config(64, 8, FCFS, watermark=2))
    a = f.add(16)
    assert f.run().tokens_of(a) == 16                       # 4 pages, 4 free
    b, c = f.add(12), f.add(2)                              # c would fit, but b is ahead of it
    s = f.run()                                             # a's decode takes a 5th page, 3 free
    assert (s.tokens_of(a), s.tokens_of(b), s.tokens_of(c)) == (1, 0, 0)
    assert b.state == SeqState.WAITING and c.state == SeqState.WAITING


@pytest.mark.parametrize("admit_whole", [False, True])
def test_admission_by_the_first_portion_or_by_the_whole_pending_input(admit_whole):
    """Not in the reference, whose admission counts the first portion (src/engine/batch_scheduler.cpp:143-146)."""
    f = Fixture(8, config(8, 4, FCFS, watermark=0, prefill_chunk=8, admit_whole=admit_whole))
    a = f.add(8)
    assert f.run().tokens_of(a) == 8                        # 2 pages, 6 free
    b = f.add(28)                                           # 7 pages in all, 2 for what the budget leaves this step
    s = f.run()                                             # a's decode takes a 3rd page
    assert s.tokens_of(a) == 1
    if admit_whole:
        assert s.tokens_of(b) == 0 and b.state == SeqState.WAITING and f.sched.num_preemptions == 0
        f.finish(a)
        assert f.run().tokens_of(b) == 8                    # the pool is b's alone now
        while b.num_pending > 1:
            f.run()
        assert f.sched.num_preemptions == 0
    else:
        assert s.tokens_of(b) == 7 and b.state == SeqState.PREFILLING
        for _ in range(8):
            f.run()                                         # b's portions fill the pool; a's next page evicts b
        assert f.sched.num_preemptions >= 1 and b.num_preemptions >= 1


def test_the_head_is_admitted_past_the_watermark_when_nothing_runs():
    f = Fixture(4, config(64, 4, FCFS, watermark=3))
    a = f.add(12)
    assert f.run().tokens_of(a) == 12


@pytest.mark.parametrize("policy,expected", [(SRPT_AGING, 18), (FCFS, 1)])
def test_shortest_first_with_aging_lets_a_long_waiter_in(policy, expected):
    f = Fixture(256, config(8, 1, policy, 0, aging=2))
    lng = f.add(40)
    admitted_at = -1
    for step in range(1, 41):
        f.add(6)                                            # a fresh short request arrives every step
        f.run()
        if lng.state != SeqState.WAITING:
            admitted_at = step
            break
        for s in f.seqs:
            if s is not lng and s.state == SeqState.DECODING:
                f.finish(s)                                 # shorts leave after one token
    # score = pending - aging * steps waited: 40 - 2t ties a fresh short's 6 - 2 = 4 at t = 18
    assert admitted_at == expected


def test_a_decode_that_needs_a_page_preempts_the_newest_which_keeps_its_tokens():
    f = Fixture(4, config(64, 4))
    a, b = f.add(8), f.add(7)
    f.run()                                                 # both prefill and sample: a has 9 tokens, b has 8
    assert f.cache.num_free() == 0
    s = f.run()                                             # a's 9th token needs a 3rd page
    assert s.tokens_of(a) == 1 and s.tokens_of(b) == 0
    assert b.state == SeqState.WAITING and b.num_computed == 0 and f.blocks(b) == 0
    assert len(b.tokens) == 8 and b.num_preemptions == 1 and f.sched.num_preemptions == 1
    f.finish(a)
    s = f.run()
    assert s.tokens_of(b) == 8 and b.num_generated == 2     # recompute, then sample the next token


def test_a_decode_with_nobody_newer_preempts_itself():
    f = Fixture(3, config(64, 4))
    a, b = f.add(3), f.add(8)
    f.run()
    assert f.cache.num_free() == 0
    s = f.run()
    assert s.tokens_of(a) == 1 and s.tokens_of(b) == 0
    assert b.num_preemptions == 1 and a.num_preemptions == 0


def test_in_flight_sequences_are_skipped_and_an_abandoned_batch_is_offered_again():
    f = Fixture(16, config(8, 2))
    a = f.add(4)
    b1 = f.sched.schedule()
    assert b1.tokens_of(a) == 4
    assert not f.sched.schedule()
    f.cache.truncate(a.cache, a.num_computed)               # what the engine does when the step fails
    f.sched.abandon(b1)
    assert f.sched.schedule().tokens_of(a) == 4


def test_the_oldest_of_several_stalled_prefills_preempts_newer_ones():
    f = Fixture(4, config(8, 2))
    a, b = f.add(12), f.add(12)
    b1 = f.sched.schedule()                                 # a: 8 tokens, 2 pages
    b2 = f.sched.schedule()                                 # a in flight; b admitted: 8 tokens, 2 pages
    assert b1.tokens_of(a) == 8 and b2.tokens_of(b) == 8
    for batch in (b1, b2):
        for s in batch.seqs:
            s.seq.num_computed += s.num_tokens
        f.sched.complete(batch)
    assert f.cache.num_free() == 0                          # both mid-prefill on a full pool
    s = f.sched.schedule()
    assert s.tokens_of(a) == 4 and b.num_preemptions == 1


def test_finish_forgets_a_sequence_waiting_running_or_preempted():
    f = Fixture(16, config(16, 1))
    a, b = f.add(3), f.add(3)
    f.run()
    f.finish(b)                                             # waiting
    assert f.sched.has_work()
    f.finish(a)                                             # running
    assert not f.sched.has_work() and f.cache.num_free() == 16
    g = Fixture(4, config(64, 4))
    p, q = g.add(8), g.add(7)
    g.run()
    g.run()                                                 # p's decode needs a 3rd page and preempts q
    assert q.num_preemptions == 1
    g.finish(q)
    assert g.run().tokens_of(q) == 0
    g.finish(p)
    assert not g.sched.has_work() and g.cache.num_free() == 4


def test_config_is_validated_and_policy_names_are_parsed():
    cache = CacheManager(PLAN, block_size=4, num_blocks=8)
    assert parse_policy("fcfs") == FCFS and parse_policy("srpt-aging") == SRPT_AGING
    with pytest.raises(InvalidArgument, match="lifo"):
        parse_policy("lifo")
    assert BatchScheduler(cache, config(8, 2, FCFS, -1)).watermark == 1
    for bad in (config(8, 9), config(8, 2, FCFS, 8), config(8, 2, FCFS, -2), config(8, 2, SRPT_AGING, 0, -1),
                config(0, 0), config(8, 2, "lifo"), config(8, 2, prefill_chunk=-1)):
        with pytest.raises(InvalidArgument):
            BatchScheduler(cache, bad)


def test_a_decode_defers_while_a_newer_sequence_is_in_flight():
    f = Fixture(3, config(64, 4))
    a, b = f.add(4), f.add(6)                               # 1 page and 2 pages: the pool is full
    b1 = f.sched.schedule()
    assert b1.tokens_of(a) == 4 and b1.tokens_of(b) == 6
    for x in b1.seqs:
        x.seq.num_computed += x.num_tokens
    f.sched.complete(b1)
    b.tokens.append(2)                                      # b sampled and decodes; a has not sampled yet
    b.state = SeqState.DECODING
    assert f.cache.num_free() == 0
    b2 = f.sched.schedule()
    assert [x.seq for x in b2.seqs] == [b]
    a.tokens.append(2)                                      # now a's decode needs a 2nd page; only in-flight b is newer
    a.state = SeqState.DECODING
    b3 = f.sched.schedule()
    assert b3.tokens_of(a) == 0 and a.num_computed == 4 and a.num_preemptions == 0 and b.num_preemptions == 0
    b.num_computed += 1
    f.sched.complete(b2)
    b4 = f.sched.schedule()
    assert b4.tokens_of(a) == 1 and b.num_preemptions == 1 and a.num_preemptions == 0


def test_no_preemption_is_counted_for_a_newer_sequence_without_pages():
    f = Fixture(2, config(64, 4))
    a, c = f.add(4), f.add(4)
    f.run()                                                 # one page each; both sample
    f.cache.release(c.cache)                                # c's step failed and its table was truncated to nothing
    c.num_computed = 0
    while a.num_computed < 8:
        f.run()                                             # a grows into the pool; c cannot get a page
    assert f.blocks(a) == 2
    s = f.run()                                             # a's 9th token needs a 3rd page that does not exist
    assert s.tokens_of(a) == 0 and c.num_preemptions == 0 and a.num_preemptions == 1
    assert f.sched.num_preemptions == 1


def test_a_sequence_preempted_this_step_is_not_readmitted_in_the_same_step():
    f = Fixture(3, config(5, 2))
    a, b = f.add(3), f.add(6)
    f.run()                                                 # a: 3 tokens, b: first 2 of its prompt
    f.run()                                                 # a decodes; b finishes its prompt and samples
    assert f.cache.num_free() == 0 and f.blocks(b) == 2
    s = f.run()                                             # a needs a page: b is preempted, freeing two
    assert s.tokens_of(a) == 1 and s.tokens_of(b) == 0
    assert b.state == SeqState.WAITING and b.num_preemptions == 1
    assert f.run().tokens_of(b) == 4                        # readmitted the step after


def test_prefill_chunk_caps_each_sequences_portion():
    f = Fixture(64, config(32, 4, prefill_chunk=13))
    a, b = f.add(40), f.add(5)
    s = f.run()
    assert s.tokens_of(a) == 13 and s.tokens_of(b) == 5
    s = f.run()
    assert s.tokens_of(a) == 13 and s.tokens_of(b) == 1
    f.run()
    s = f.run()
    assert s.tokens_of(a) == 1 and a.num_computed == 40 and a.num_generated == 1


def test_admission_needs_a_free_state_slot():
    plan = plan_cache([PagedKV(1, 8), FixedState((2,))], [None, None])
    f = Fixture(32, config(16, 4), plan=plan, state_slots=1)
    a, b = f.add(3), f.add(3)
    s = f.run()
    assert s.tokens_of(a) == 3 and s.tokens_of(b) == 0 and a.cache.state_slot == 0
    f.finish(a)
    assert f.run().tokens_of(b) == 3 and b.cache.state_slot == 0


@pytest.mark.parametrize("seed", range(300))
def test_randomized_everything_finishes_and_no_page_is_shared_or_lost(seed):
    rng = random.Random(seed)
    blocks = rng.randint(3, 16)
    pool_tokens = blocks * 4
    budget = rng.randint(4, 32)
    cfg = config(budget, rng.randint(1, min(8, budget)), FCFS if seed % 2 else SRPT_AGING,
                 rng.randint(-1, blocks - 1), rng.randint(0, 8), prefill_chunk=rng.choice([0, 0, 3, 7]),
                 admit_whole=seed % 3 == 0)
    f = Fixture(blocks, cfg)
    requests = []
    for _ in range(rng.randint(1, 20)):
        prompt = rng.randint(1, pool_tokens - 1)            # like add_request: each fits the whole pool alone
        requests.append((rng.randint(0, 40), prompt, rng.randint(1, pool_tokens - prompt)))
    requests.sort(key=lambda r: r[0])
    live, nxt, empty_streak, step = [], 0, 0, 0

    def finish(s):
        f.finish(s)
        live.remove(s)

    while step < 20000 and (nxt < len(requests) or live):
        while nxt < len(requests) and requests[nxt][0] <= step:
            live.append(f.add(requests[nxt][1], requests[nxt][2]))
            nxt += 1
        if live and rng.randint(0, 49) == 0:
            finish(rng.choice(live))                        # cancel
        oldest = f.sched.running[0] if f.sched.running else None
        oldest_preemptions = oldest.num_preemptions if oldest else 0
        batch = f.sched.schedule()
        if oldest is not None:
            assert oldest.num_preemptions == oldest_preemptions
        for s in batch.seqs:
            assert 0 < s.num_tokens <= s.seq.num_pending
            assert f.blocks(s.seq) >= f.cache.blocks_for(s.seq.num_computed + s.num_tokens)
        assert batch.total_tokens <= cfg.serving.max_tokens_per_step and len(batch.seqs) <= cfg.serving.max_seqs
        # an empty step is allowed only right after a preemption made the waiter sit out one step
        empty_streak = empty_streak + 1 if (not batch and f.sched.has_work()) else 0
        assert empty_streak <= 1
        for s in batch.seqs:
            s.seq.num_computed += s.num_tokens
        f.sched.complete(batch)
        for s in batch.seqs:
            if s.seq.num_pending != 0:
                continue
            s.seq.tokens.append(3)
            s.seq.state = SeqState.DECODING
            if s.seq.num_generated >= s.seq.params.max_tokens:
                finish(s.seq)
        f.cache.audit([s.cache for s in live])
        for s in live:
            assert f.blocks(s) == f.cache.blocks_for(s.num_computed)
        step += 1
    assert not live and nxt == len(requests)
    assert f.cache.num_free() == blocks and not f.sched.has_work()
    test_randomized_everything_finishes_and_no_page_is_shared_or_lost.preemptions += f.sched.num_preemptions


test_randomized_everything_finishes_and_no_page_is_shared_or_lost.preemptions = 0


@pytest.mark.parametrize("seed", range(40))
def test_the_shortcut_for_steady_decoding_plans_what_the_rounds_would(seed):
    """Two schedulers over equal pools and equal requests, one with the shortcut switched off: equal plans."""
    rng = random.Random(1000 + seed)
    blocks, budget = rng.randint(6, 40), rng.randint(4, 32)
    cfg = lambda: config(budget, rng_seats, FCFS if seed % 2 else SRPT_AGING, 0, 4)
    rng_seats = rng.randint(1, min(8, budget))
    fast, slow = Fixture(blocks, cfg()), Fixture(blocks, cfg())
    slow.sched._steady_decode = lambda plan, budget: False
    arrivals = sorted((rng.randint(0, 30), rng.randint(1, blocks * 4 - 1)) for _ in range(rng.randint(1, 10)))
    arrivals = [(at, n, rng.randint(1, blocks * 4 - n)) for at, n in arrivals]
    step = nxt = 0
    while step < 3000 and (nxt < len(arrivals) or fast.sched.has_work()):
        while nxt < len(arrivals) and arrivals[nxt][0] <= step:
            for f in (fast, slow):
                f.add(arrivals[nxt][1], arrivals[nxt][2])
            nxt += 1
        plans = [f.run() for f in (fast, slow)]
        assert [(x.seq.id, x.num_tokens) for x in plans[0].seqs] == [(x.seq.id, x.num_tokens) for x in plans[1].seqs]
        for f in (fast, slow):
            for s in f.seqs:
                if s.state == SeqState.DECODING and s.num_generated >= s.params.max_tokens:
                    f.finish(s)
        assert fast.cache.num_free() == slow.cache.num_free()
        step += 1
    assert not fast.sched.has_work() and not slow.sched.has_work()
    test_the_shortcut_for_steady_decoding_plans_what_the_rounds_would.taken += fast.sched.steady_steps


test_the_shortcut_for_steady_decoding_plans_what_the_rounds_would.taken = 0


def test_the_shortcut_was_taken():
    assert test_the_shortcut_for_steady_decoding_plans_what_the_rounds_would.taken > 100


def test_the_randomized_runs_did_preempt():
    assert test_randomized_everything_finishes_and_no_page_is_shared_or_lost.preemptions > 0
