"""Feeds a workload to an engine and records when every token appears.

The reference declares this runner's inputs and outputs (``src/bench/report.h:12-23``: per request the
arrival, the prompt length and the times of its tokens; the wall time; the engine's statistics) and
parses its options, but never wrote the loop. Here it is: requests enter the engine when their arrival
time has come, the engine steps while it has work, and a token callback notes the time of every token.
"""

from __future__ import annotations

import time
from typing import Callable, List, Optional, Sequence

from ..engine.engine import Engine
from ..sampling.params import SamplingParams
from .report import BenchRun, RequestTiming
from .workload import BenchRequest


def run_workload(engine: Engine, requests: Sequence[BenchRequest], sampling: Optional[SamplingParams] = None,
                 clock: Callable[[], float] = time.perf_counter,
                 progress: Optional[Callable[[str], None]] = None) -> BenchRun:
    """Runs ``requests`` to their ends; returns the timings. The engine's own token callback is put back after."""
    import dataclasses

    sampling = sampling or SamplingParams(temperature=0.0)
    order = sorted(range(len(requests)), key=lambda i: (requests[i].arrival, i))
    timings: List[RequestTiming] = [RequestTiming(r.arrival, len(r.prompt)) for r in requests]
    of_sequence = {}
    before = engine.stats()
    started = clock()
    last_report = started

    def on_token(seq_id: int, token: int) -> None:
        timings[of_sequence[seq_id]].token_times.append(clock() - started)

    previous, engine.on_token = engine.on_token, on_token
    try:
        nxt = 0
        while nxt < len(order) or engine.has_work():
            now = clock() - started
            while nxt < len(order) and requests[order[nxt]].arrival <= now:
                i = order[nxt]
                params = dataclasses.replace(sampling, max_tokens=requests[i].max_tokens, seed=sampling.seed + i)
                of_sequence[engine.add_request(requests[i].prompt, params)] = i
                nxt += 1
            if engine.has_work():
                engine.step()
            else:                                   # nothing to do until the next request arrives
                time.sleep(min(1e-3, max(0.0, requests[order[nxt]].arrival - now)))
            if progress is not None and clock() - last_report > 15:
                done = sum(1 for s in engine.sequences.values() if s.finish_reason.value != "none")
                progress(f"{done} of {len(requests)} requests finished, {engine.stats().steps - before.steps} steps")
                last_report = clock()
    finally:
        engine.on_token = previous
    wall = clock() - started
    after = engine.stats()
    for seq_id in list(of_sequence):
        engine.release(seq_id)
    return BenchRun(timings, wall, after.steps - before.steps, after.seqs_scheduled - before.seqs_scheduled,
                    after.preemptions - before.preemptions, tokens_read_late=bool(getattr(engine, "launch_ahead", False)))
