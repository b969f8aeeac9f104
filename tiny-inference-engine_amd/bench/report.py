"""What a serving run is summed up to.

The fields are those of the reference's report (``src/bench/report.h:29-36``, computed as in
``report.cpp:34-59``): requests, prompt and output tokens, wall time, requests / output tokens / all
tokens a second, steps, mean sequences a step, preemptions, and the 50th / 90th / 99th percentile of
the time to the first token (arrival to first token), of the gaps between consecutive tokens of a
request, and of the whole request (arrival to last token), in milliseconds. Percentiles interpolate
linearly between the closest ranks (``report.cpp:24-32``).
"""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Sequence

import numpy as np

from ..errors import InvalidArgument


@dataclasses.dataclass
class RequestTiming:
    arrival: float = 0.0                  # seconds after the run started
    prompt_len: int = 0
    token_times: List[float] = dataclasses.field(default_factory=list)


@dataclasses.dataclass
class BenchRun:
    requests: List[RequestTiming]
    wall_seconds: float
    steps: int
    seqs_scheduled: int
    preemptions: int
    tokens_read_late: bool = False        # the engine queued decode steps ahead: a token's time is one step late


@dataclasses.dataclass
class BenchReport:
    requests: int = 0
    prompt_tokens: int = 0
    output_tokens: int = 0
    wall_s: float = 0.0
    requests_per_s: float = 0.0
    output_tok_per_s: float = 0.0
    total_tok_per_s: float = 0.0
    ttft_ms: Dict[str, float] = dataclasses.field(default_factory=dict)
    itl_ms: Dict[str, float] = dataclasses.field(default_factory=dict)
    e2e_ms: Dict[str, float] = dataclasses.field(default_factory=dict)
    mean_seqs_per_step: float = 0.0
    steps: int = 0
    preemptions: int = 0
    # Not among the reference's fields: whether the engine read a decode step's tokens while the next step ran
    # (``launch_ahead``). Token times (ttft, itl, e2e) then carry one step of delay that throughput does not.
    tokens_read_late: bool = False


def percentile(values: Sequence[float], p: float) -> float:
    if not 0.0 <= p <= 100.0:
        raise InvalidArgument(f"a percentile lies between 0 and 100, not {p}")
    if len(values) == 0:
        return 0.0
    ordered = np.sort(np.asarray(values, dtype=np.float64))
    rank = p / 100.0 * (ordered.size - 1)
    below = int(rank)
    above = min(below + 1, ordered.size - 1)
    return float(ordered[below] + (ordered[above] - ordered[below]) * (rank - below))


def _p50_p90_p99_ms(seconds: Sequence[float]) -> Dict[str, float]:
    ms = [s * 1e3 for s in seconds]
    return {"p50": percentile(ms, 50), "p90": percentile(ms, 90), "p99": percentile(ms, 99)}


def summarize(run: BenchRun) -> BenchReport:
    first, gaps, whole = [], [], []
    report = BenchReport(requests=len(run.requests), wall_s=run.wall_seconds, steps=run.steps,
                         preemptions=run.preemptions, tokens_read_late=run.tokens_read_late)
    for timing in run.requests:
        report.prompt_tokens += timing.prompt_len
        report.output_tokens += len(timing.token_times)
        if not timing.token_times:
            continue
        times = np.asarray(timing.token_times)
        first.append(float(times[0]) - timing.arrival)
        whole.append(float(times[-1]) - timing.arrival)
        gaps.extend(np.diff(times).tolist())
    if run.wall_seconds > 0:
        report.requests_per_s = report.requests / run.wall_seconds
        report.output_tok_per_s = report.output_tokens / run.wall_seconds
        report.total_tok_per_s = (report.prompt_tokens + report.output_tokens) / run.wall_seconds
    report.mean_seqs_per_step = run.seqs_scheduled / run.steps if run.steps else 0.0
    report.ttft_ms, report.itl_ms, report.e2e_ms = _p50_p90_p99_ms(first), _p50_p90_p99_ms(gaps), _p50_p90_p99_ms(whole)
    return report


def format_report(r: BenchReport) -> str:
    def row(name, p):
        return f"  {name:<5} ms   p50 {p['p50']:>9.1f}   p90 {p['p90']:>9.1f}   p99 {p['p99']:>9.1f}\n"

    return (f"requests {r.requests}  |  wall {r.wall_s:.2f} s  |  {r.requests_per_s:.2f} req/s\n"
            f"tokens   {r.prompt_tokens} prompt + {r.output_tokens} output  |  output {r.output_tok_per_s:.1f} tok/s"
            f"  |  total {r.total_tok_per_s:.1f} tok/s\n"
            + row("ttft", r.ttft_ms) + row("itl", r.itl_ms) + row("e2e", r.e2e_ms) +
            f"steps    {r.steps}  |  {r.mean_seqs_per_step:.2f} sequences/step  |  {r.preemptions} preemptions\n"
            + ("note     decode steps were queued ahead: every token above is timed one step after it existed "
               "(--no-launch-ahead times them as they appear)\n" if r.tokens_read_late else ""))


def report_json(r: BenchReport) -> dict:
    return dataclasses.asdict(r)
