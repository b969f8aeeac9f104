"""The requests of a serving benchmark.

What the reference's bench helpers make (``src/bench/workload.cpp:46-82``): ``n`` requests of
uniformly random token ids whose prompt and output lengths are drawn uniformly from two ranges, all from
one seed, and Poisson arrivals at a given rate (an infinite rate puts every request at time 0). The
streams here are Python's ``random.Random``; the reference draws from ``std::mt19937_64`` through
distributions whose algorithms the C++ standard leaves open, so equal seeds do not give equal workloads
across the two programs (only equal statistics).

A workload file is JSON lines ``{"prompt_ids": [...], "max_tokens": N}``. The reference's files hold
prompt TEXT (``workload.cpp:14-44``); this engine has no tokenizer, so such a line is refused.
"""

from __future__ import annotations

import dataclasses
import json
import math
import random
from typing import List, Optional, Tuple

from ..errors import InvalidArgument


@dataclasses.dataclass
class BenchRequest:
    prompt: List[int]
    max_tokens: int
    arrival: float = 0.0       # seconds after the run starts


def parse_range(flag: str, text: str) -> Tuple[int, int]:
    """"A:B" or "A" with 1 <= A <= B."""
    low, _, high = text.partition(":")
    try:
        lo = int(low)
        hi = int(high) if high else lo
    except ValueError:
        raise InvalidArgument(f"{flag} takes A:B or A in whole numbers, not '{text}'") from None
    if lo < 1 or hi < lo:
        raise InvalidArgument(f"{flag} takes A:B with 1 <= A <= B, not '{text}'")
    return lo, hi


def synthetic_requests(n: int, prompt_len: Tuple[int, int], output_len: Tuple[int, int], vocab_size: int,
                       seed: int) -> List[BenchRequest]:
    if n < 1:
        raise InvalidArgument(f"a synthetic workload has at least one request, not {n}")
    if vocab_size < 1:
        raise InvalidArgument(f"a vocabulary of {vocab_size} tokens cannot be drawn from")
    for what, (lo, hi) in (("prompt", prompt_len), ("output", output_len)):
        if lo < 1 or hi < lo:
            raise InvalidArgument(f"{what} lengths {lo}:{hi} are no range with 1 <= low <= high")
    rng = random.Random(seed)
    requests = []
    for _ in range(n):
        length = rng.randint(*prompt_len)
        prompt = [rng.randrange(vocab_size) for _ in range(length)]
        requests.append(BenchRequest(prompt, rng.randint(*output_len)))
    return requests


def assign_arrivals(requests: List[BenchRequest], rate: float, seed: int) -> None:
    """Poisson arrivals at ``rate`` requests a second, in the order given; ``inf`` means all at time 0."""
    if not rate > 0:
        raise InvalidArgument(f"an arrival rate must be positive, not {rate}")
    if math.isinf(rate):
        for r in requests:
            r.arrival = 0.0
        return
    rng = random.Random(seed)
    now = 0.0
    for r in requests:
        now += rng.expovariate(rate)
        r.arrival = now


def read_requests_jsonl(path: str, default_max_tokens: int, vocab_size: Optional[int] = None) -> List[BenchRequest]:
    requests = []
    try:
        with open(path) as f:
            lines = f.read().splitlines()
    except OSError as e:
        raise InvalidArgument(f"cannot read {path}: {e.strerror or e}") from None
    for number, line in enumerate(lines, 1):
        if not line.strip():
            continue
        try:
            item = json.loads(line)
        except json.JSONDecodeError as e:
            raise InvalidArgument(f"{path}:{number}: not JSON ({e.msg})") from None
        if not isinstance(item, dict) or "prompt_ids" not in item:
            hint = " (prompt text needs a tokenizer, which this engine does not have)" if isinstance(item, dict) and \
                "prompt" in item else ""
            raise InvalidArgument(f"{path}:{number}: a line is an object with \"prompt_ids\"{hint}")
        ids = item["prompt_ids"]
        if not isinstance(ids, list) or not ids or not all(isinstance(t, int) and not isinstance(t, bool) for t in ids):
            raise InvalidArgument(f"{path}:{number}: \"prompt_ids\" is a non-empty list of token ids")
        if vocab_size is not None and not all(0 <= t < vocab_size for t in ids):
            raise InvalidArgument(f"{path}:{number}: a token id lies outside the vocabulary of {vocab_size}")
        max_tokens = item.get("max_tokens", default_max_tokens)
        if not isinstance(max_tokens, int) or isinstance(max_tokens, bool) or max_tokens < 1:
            raise InvalidArgument(f"{path}:{number}: \"max_tokens\" is a positive whole number")
        requests.append(BenchRequest(list(ids), max_tokens))
    if not requests:
        raise InvalidArgument(f"{path}: no requests")
    return requests
