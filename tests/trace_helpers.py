"""Building traces (lists of steps) that cut the same requests in different ways."""

import random
from typing import Dict, List, Sequence


def make_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def round64(n: int) -> int:
    return (n + 63) // 64 * 64


def whole(requests):
    """Each request alone and whole, every position wanted."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
    return steps


def prefill_then_decode(requests, tail=32):
    """Most of a request in one step, its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=(13, 7, 2, 5, 3, 2, 11, 4)):
    """Each request alone in portions of changing size, down to two tokens."""
    steps = []
    k = 0
    for rid, toks in requests.items():
        pos = 0
        while pos < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - pos)
            k += 1
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[pos:pos + n],
                                                           "want": list(range(n))}], "end": []})
            pos += n
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests, max_live=4, seed=0, tail=8, sizes=(13, 7, 2, 5, 3, 2, 9)):
    """Up to ``max_live`` requests at a time: portions of some beside single tokens of others.

    A request runs its last ``tail`` tokens one by one; now and then a live request sits a step
    out. Returns (steps, max_tokens) where max_tokens is the most that live requests hold at any
    time with each request's count rounded up to a multiple of 64.
    """
    rng = random.Random(seed)
    waiting = list(requests)
    live: Dict[str, int] = {}
    steps = []
    peak = 0
    k = 0
    while waiting or live:
        while waiting and len(live) < max_live:
            live[waiting.pop(0)] = 0
        entries, ended = [], []
        for rid in list(live):
            toks, pos = requests[rid], live[rid]
            if len(live) > 1 and len(entries) > 0 and rng.random() < 0.2:
                continue                                    # sits this step out
            remaining = len(toks) - pos
            if remaining <= tail:
                n = 1
            else:
                n = min(sizes[k % len(sizes)], remaining - tail)
                k += 1
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))})
            live[rid] = pos + n
            if live[rid] == len(toks):
                ended.append(rid)
        peak = max(peak, sum(round64(v) for v in live.values()))
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        for rid in ended:
            del live[rid]
    return steps, peak


def collect(replayer, steps):
    """Runs steps in-process; returns {request id: {position: logits row (CPU float32 tensor)}}."""
    out: Dict[str, Dict[int, object]] = {}
    position: Dict[str, int] = {}
    for step in steps:
        logits = replayer.run_step(step)
        rows = logits.float().cpu() if logits is not None else None
        r = 0
        for e in step["entries"]:
            start = position.get(e["id"], 0)
            for w in e["want"]:
                out.setdefault(e["id"], {})[start + w] = rows[r]
                r += 1
            position[e["id"]] = start + len(e["tokens"])
        for rid in step["end"]:
            position.pop(rid, None)
    return out
