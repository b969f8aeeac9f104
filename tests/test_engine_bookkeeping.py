"""The engine's bookkeeping over a real scheduler and page pool, with a stand-in model and sampler (no GPU).

The stand-in "model" remembers, per request, the tokens that went through ``step`` (what a cache of
keys and values amounts to) and its "logits" name the token that follows a history: a hash of that
history. Whatever the engine does between a request's tokens and its next token - portions, evictions
and recomputation, steps queued ahead of the tokens they depend on - every request must end with
exactly the chain of hashes of its own prompt, every page must come back, and no request may be lost.
"""

import random
import types

import pytest

from tie_amd.cache.manager import CacheManager
from tie_amd.cache.spec import PagedKV, plan_cache
from tie_amd.engine.engine import Engine
from tie_amd.engine.scheduler import FCFS, SRPT_AGING, BatchScheduler, SchedulerConfig
from tie_amd.engine.sequence import UNREAD, SeqState
from tie_amd.engine.serving import ServingConfig
from tie_amd.sampling.params import SamplingParams

VOCAB = 97
PLAN = plan_cache([PagedKV(1, 8)], [None])


def next_token(history):
    h = 1469598103
    for t in history:
        h = (h * 1099511 + t + 1) % 2147483647
    return h % VOCAB


def expected(prompt, count, stop=()):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(next_token(tokens))
        if tokens[-1] in stop:
            break
    return tokens[len(prompt):]


class FakeRunner:
    """Keeps every request's history as a cache would; a step's 'logits' are the next tokens of the wanted rows."""

    def __init__(self, max_blocks_per_seq):
        self.max_blocks_per_seq = max_blocks_per_seq
        self.history = {}
        self.steps = 0

    def step(self, entries, device_tokens=None):
        self.steps += 1
        out = []
        for i, e in enumerate(entries):
            tokens = list(e.tokens)
            if e.token_from >= 0:                   # the token an earlier step's sampling left "on the device"
                assert len(tokens) == 1 and device_tokens is not None
                tokens = [device_tokens[e.token_from]]
            assert all(0 <= t < VOCAB for t in tokens), "a token the host never read went into a step as it stood"
            past = self.history.setdefault(id(e.cache), [])
            assert len(past) >= e.start, "a step began beyond what the cache holds"
            del past[e.start:]                      # recomputation after an eviction starts over
            past.extend(tokens)
            for w in e.want:
                out.append(next_token(past[:e.start + w + 1]))
        return out


class FakeTicket:
    def __init__(self, tokens):
        self.device_tokens = list(tokens)
        self.rows = len(tokens)


class FakeSampler:
    def launch_greedy(self, logits):
        return FakeTicket(logits)

    def launch(self, logits, params, rngs, previous=None):
        return FakeTicket(logits)

    def collect(self, ticket):
        return list(ticket.device_tokens)

    def sample_rows(self, logits, params, rngs):
        return list(logits)


def make_engine(blocks, max_tokens_per_step, max_seqs, policy, launch_ahead, prefill_chunk=0, stop=(), admit_whole=False):
    cache = CacheManager(PLAN, block_size=4, num_blocks=blocks, max_state_slots=64)
    serving = ServingConfig(max_tokens_per_step, max_seqs, prefill_chunk)
    model = types.SimpleNamespace(spec=types.SimpleNamespace(max_positions=4096, vocab_size=VOCAB), device="cpu")
    runner = FakeRunner(max_blocks_per_seq=cache.blocks_for(4096))
    sched = BatchScheduler(cache, SchedulerConfig(serving, policy, 16, 0, admit_whole))
    return Engine(model, cache, sched, serving, stop_tokens=stop, launch_ahead=launch_ahead, runner=runner,
                  sampler=FakeSampler())


def run_all(engine, requests, arrivals=None, limit=20000):
    """Adds the requests (``arrivals``: the step at which each enters) and steps until nothing is left."""
    ids, step = {}, 0
    pending = sorted(range(len(requests)), key=lambda i: 0 if arrivals is None else arrivals[i])
    while pending or engine.has_work():
        while pending and (arrivals is None or arrivals[pending[0]] <= step):
            i = pending.pop(0)
            prompt, count = requests[i]
            ids[i] = engine.add_request(prompt, SamplingParams(max_tokens=count))
        engine.step()
        step += 1
        for seq in engine.sequences.values():          # a request is in exactly one place
            queues = sum(seq is s for s in engine.scheduler.waiting) + sum(seq is s for s in engine.scheduler.running)
            assert queues == (0 if seq.state == SeqState.FINISHED else 1), \
                f"sequence {seq.id} ({seq.state}) is in {queues} queues after step {step}"
            assert (seq.state == SeqState.WAITING) == any(seq is s for s in engine.scheduler.waiting)
        assert step < limit, "the engine does not come to an end"
    return {i: engine.sequences[ids[i]] for i in ids}


@pytest.mark.parametrize("policy", [FCFS, SRPT_AGING])
@pytest.mark.parametrize("launch_ahead", [False, True, 2, 3])
def test_random_workloads_over_small_pools_lose_nobody(policy, launch_ahead):
    evictions = ahead = mixed_ahead = steps = 0
    for seed in range(300):
        rng = random.Random(seed)
        n = rng.randint(2, 6)
        requests = [([rng.randrange(VOCAB) for _ in range(rng.randint(1, 14))], rng.randint(1, 12)) for _ in range(n)]
        arrivals = [rng.randint(0, 8) for _ in range(n)]
        longest = max(len(p) + c for p, c in requests)
        blocks = (longest + 3) // 4 + rng.randint(0, 5)            # the longest fits alone, little more
        # every other workload has stop tokens: a sequence that meets one has run ahead, and what it ran is dropped
        stop = tuple(rng.sample(range(VOCAB), 6)) if seed % 2 else ()
        engine = make_engine(blocks, rng.randint(4, 12), rng.randint(2, 4), policy, launch_ahead,
                             prefill_chunk=rng.choice([0, 3, 5]), stop=stop, admit_whole=seed % 5 == 0)
        done = run_all(engine, requests, arrivals)
        for i, (prompt, count) in enumerate(requests):
            assert done[i].state == SeqState.FINISHED
            assert done[i].generated == expected(prompt, count, stop), f"seed {seed}, request {i}"
            assert UNREAD not in done[i].tokens
        assert engine.cache.all_free()
        evictions += engine.stats().preemptions
        ahead += engine.steps_launched_ahead
        mixed_ahead += engine.ahead_replans
        steps += engine.stats().steps
    assert evictions > 100
    # Queued ahead are not only the steady repetitions of a decode step but most steps: prompts beside decoders,
    # admissions, steps after an eviction.
    assert (ahead > 0.6 * steps and mixed_ahead > 0.2 * steps) if launch_ahead else ahead == mixed_ahead == 0


def test_an_eviction_while_tokens_are_unread_keeps_the_evicted_request():
    """All decoding, nobody waiting, tokens unread, and the pool runs dry at a page's edge: newer requests are
    evicted with their last token still on the GPU. Each must stay in the waiting queue (and only there, as a
    waiting request), be computed again with that token, and end like the others."""
    # Four prompts of 3 tokens in pages of 4: each holds one page and needs a second at its fifth token, all in
    # the same step, and the pool has one spare page: two or more requests wait afterwards.
    requests = [([1, 2, 3], 9), ([4, 5, 6], 9), ([7, 8, 9], 9), ([10, 11, 12], 9)]
    engine = make_engine(5, 16, 4, FCFS, launch_ahead=True)
    most_waiting = 0
    real_read = engine._read_oldest

    def counting_read():
        real_read()
        nonlocal most_waiting
        most_waiting = max(most_waiting, sum(s.num_preemptions > 0 for s in engine.scheduler.waiting))
    engine._read_oldest = counting_read
    done = run_all(engine, requests)          # checks after every step that a request is in exactly one place
    assert engine.ahead_replans > 0, "no plan was changed by an eviction while tokens were unread"
    assert most_waiting >= 2 and engine.stats().preemptions >= 2 and engine.steps_launched_ahead > 0
    for i, (prompt, count) in enumerate(requests):
        assert done[i].generated == expected(prompt, count)
    assert engine.cache.all_free()


def test_stop_tokens_met_in_a_step_queued_ahead_drop_the_token_that_ran_past():
    prompt = [5, 6, 7]
    chain = expected(prompt, 12)
    stop = chain[6]
    first = chain.index(stop)
    for launch_ahead in (False, True):
        engine = make_engine(32, 16, 4, FCFS, launch_ahead, stop=(stop,))
        out = engine.generate(prompt, SamplingParams(max_tokens=12))
        assert out == chain[:first + 1]
        assert engine.cache.all_free()
