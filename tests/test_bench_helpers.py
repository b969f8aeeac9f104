"""The serving benchmark's helpers (no GPU): the workload, the percentiles, the report.

The percentile vectors are those the reference's own test holds (tests/bench/test_report.cpp, read, not run)."""

import json
import math

import pytest

from tie_amd.bench import (BenchRequest, BenchRun, RequestTiming, assign_arrivals, format_report, parse_range, percentile,
                           read_requests_jsonl, report_json, summarize, synthetic_requests)
from tie_amd.errors import InvalidArgument


def test_synthetic_requests_are_seeded_and_inside_their_ranges():
    a = synthetic_requests(50, (3, 9), (2, 5), 100, seed=7)
    b = synthetic_requests(50, (3, 9), (2, 5), 100, seed=7)
    c = synthetic_requests(50, (3, 9), (2, 5), 100, seed=8)
    assert [r.prompt for r in a] == [r.prompt for r in b] and [r.prompt for r in a] != [r.prompt for r in c]
    assert all(3 <= len(r.prompt) <= 9 and 2 <= r.max_tokens <= 5 and all(0 <= t < 100 for t in r.prompt) for r in a)
    assert {len(r.prompt) for r in a} == set(range(3, 10))          # both ends of the range are reached
    assert all(r.arrival == 0.0 for r in a)
    for bad in ((0, (1, 2), (1, 2), 10), (3, (0, 2), (1, 2), 10), (3, (1, 2), (5, 2), 10), (3, (1, 2), (1, 2), 0)):
        with pytest.raises(InvalidArgument):
            synthetic_requests(*bad, seed=0)


def test_arrivals_are_poisson_in_order_or_all_at_once():
    requests = [BenchRequest([1], 1) for _ in range(4000)]
    assign_arrivals(requests, 50.0, seed=3)
    times = [r.arrival for r in requests]
    assert times == sorted(times) and times[0] > 0
    assert abs(times[-1] / len(times) - 1 / 50.0) < 0.1 / 50.0       # the mean gap is 1 / rate
    assign_arrivals(requests, math.inf, seed=3)
    assert all(r.arrival == 0.0 for r in requests)
    with pytest.raises(InvalidArgument):
        assign_arrivals(requests, 0.0, seed=3)


def test_ranges_and_workload_files(tmp_path):
    assert parse_range("--prompt-len", "3:9") == (3, 9) and parse_range("--output-len", "7") == (7, 7)
    for bad in ("9:3", "0", "a:b", "3:", ":3", ""):
        if bad == "3:":
            assert parse_range("--x", bad) == (3, 3)
            continue
        with pytest.raises(InvalidArgument):
            parse_range("--x", bad)
    path = tmp_path / "w.jsonl"
    path.write_text('{"prompt_ids": [1, 2, 3], "max_tokens": 4}\n\n{"prompt_ids": [5]}\n')
    got = read_requests_jsonl(str(path), default_max_tokens=9, vocab_size=10)
    assert [(r.prompt, r.max_tokens) for r in got] == [([1, 2, 3], 4), ([5], 9)]
    for text, match in (('{"prompt": "hello"}', "tokenizer"), ('{"prompt_ids": []}', "non-empty"), ("[1]", "prompt_ids"),
                        ('{"prompt_ids": [1], "max_tokens": 0}', "max_tokens"), ("{", "not JSON"), ("\n", "no requests"),
                        ('{"prompt_ids": [11]}', "vocabulary")):
        path.write_text(text + "\n")
        with pytest.raises(InvalidArgument, match=match):
            read_requests_jsonl(str(path), 9, 10)


def test_percentiles_interpolate_between_the_closest_ranks():
    values = [10.0, 20.0, 30.0, 40.0]
    assert percentile(values, 0) == 10.0 and percentile(values, 100) == 40.0
    assert percentile(values, 50) == 25.0                               # rank 1.5
    assert percentile([3.0, 1.0, 2.0], 50) == 2.0                       # sorted first
    assert math.isclose(percentile(values, 90), 37.0) and percentile([], 50) == 0.0 and percentile([7.0], 99) == 7.0
    # the reference's own vectors (tests/bench/test_bench.cpp:67-73, 109-113)
    assert percentile([], 50) == 0.0 and percentile([4.0], 99) == 4.0 and math.isclose(percentile([1, 2, 3, 4], 50), 2.5)
    assert percentile([4, 3, 2, 1], 0) == 1.0 and percentile([1, 2, 3, 4], 100) == 4.0
    assert math.isclose(percentile([1, 2, 3, 4, 5], 90), 4.6)
    for bad in (100.5, -1, math.nan, 101):
        with pytest.raises(InvalidArgument):
            percentile([1, 2, 3] if bad != 101 else [], bad)


def test_the_report_sums_up_a_run():
    run = BenchRun([RequestTiming(0.0, 10, [1.0, 1.5, 2.5]), RequestTiming(0.5, 20, [2.0]), RequestTiming(1.0, 5, [])],
                   wall_seconds=4.0, steps=8, seqs_scheduled=12, preemptions=2)
    r = summarize(run)
    assert (r.requests, r.prompt_tokens, r.output_tokens, r.steps, r.preemptions) == (3, 35, 4, 8, 2)
    assert r.requests_per_s == 0.75 and r.output_tok_per_s == 1.0 and r.total_tok_per_s == 39 / 4.0
    assert r.mean_seqs_per_step == 1.5
    assert r.ttft_ms["p50"] == 1250.0                 # first tokens 1.0 and 1.5 s after arrival
    assert r.itl_ms["p50"] == 750.0                   # gaps of 0.5 and 1.0 s
    assert r.e2e_ms["p50"] == 2000.0                  # 2.5 and 1.5 s from arrival to the last token
    # the reference's own vector (tests/bench/test_bench.cpp:76-94)
    theirs = summarize(BenchRun([RequestTiming(0.0, 10, [0.1, 0.2, 0.3]), RequestTiming(0.5, 20, [1.0, 1.5])],
                                wall_seconds=2.0, steps=4, seqs_scheduled=6, preemptions=1))
    assert (theirs.requests, theirs.output_tokens, theirs.prompt_tokens, theirs.preemptions) == (2, 5, 30, 1)
    assert math.isclose(theirs.output_tok_per_s, 2.5) and math.isclose(theirs.total_tok_per_s, 17.5)
    assert math.isclose(theirs.requests_per_s, 1.0) and math.isclose(theirs.mean_seqs_per_step, 1.5)
    assert math.isclose(theirs.ttft_ms["p50"], 300.0) and math.isclose(theirs.e2e_ms["p50"], 650.0)
    assert math.isclose(theirs.itl_ms["p50"], 100.0)
    text = format_report(r)
    assert "requests 3" in text and "2 preemptions" in text and "1.50 sequences/step" in text and "ttft" in text
    assert set(json.loads(json.dumps(report_json(r)))) == {
        "requests", "prompt_tokens", "output_tokens", "wall_s", "requests_per_s", "output_tok_per_s", "total_tok_per_s",
        "ttft_ms", "itl_ms", "e2e_ms", "mean_seqs_per_step", "steps", "preemptions",      # report.cpp:73-86
        "tokens_read_late"}                                # ours: the token times carry one step of delay
    assert "queued ahead" not in text
    late = summarize(BenchRun([RequestTiming(0.0, 10, [1.0, 1.5])], 2.0, 2, 2, 0, tokens_read_late=True))
    assert late.tokens_read_late and "queued ahead" in format_report(late)


def test_kernel_trace_summaries(tmp_path):
    """Totals, a decode step's average and the busy share, from a hand-made trace: three steps of an embedding
    kernel (1 us) and a product (10 us) with 4 us between the steps."""
    import sqlite3

    from tie_amd.bench import kernel_trace

    path = str(tmp_path / "trace.db")
    db = sqlite3.connect(path)
    db.execute("create table kernels (name text, start integer, end integer, grid_x integer, grid_y integer, grid_z integer)")
    t = 1_000_000
    for _ in range(3):
        db.execute("insert into kernels values ('void embed_kernel<float>(int*)', ?, ?, 256, 1, 1)", (t, t + 1000))
        db.execute("insert into kernels values ('void product<1, 2>(float const*)', ?, ?, 512, 2, 1)", (t + 1000, t + 11000))
        t += 15000
    db.commit()
    db.close()
    launches = kernel_trace.read_launches(path)
    assert len(launches) == 6 and launches[1][3] == 1024
    text = kernel_trace.totals(launches)
    assert "product<1, 2>" in text and "embed_kernel<float>" in text and "(" not in text.split("\n")[1]
    assert "kernel time 0.0 ms" in text
    steps = kernel_trace.last_steps(launches, 2, "embed_kernel")
    assert "2 steps: kernel span 11.0 us/step, kernel busy 11.0 us/step, step period 15.0 us" in steps
    # the last 30 us: two whole steps' kernels less the first's first microsecond... exactly: from 11 us before the
    # first of them ends; 4 us of every 15 idle
    share = kernel_trace.busy_share(launches, 30e-6)
    assert "= 0.733" in share and "shorter: 2 totalling" in share
    assert kernel_trace.main([path, "--steps", "2", "--window", "0.00003", "--by-grid"]) == 0
