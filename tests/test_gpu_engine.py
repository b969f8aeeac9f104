"""Generation through the engine on the GPU: the entry points, chunked prefill, batching, preemption.

Scenarios of the reference's tests/engine/test_engine.cpp and test_engine_batching.cpp, with the plain
implementation in place of the fixtures the reference downloads.
"""

import subprocess
import sys

import pytest
import torch

import plain_qwen3 as plain
import tolerances
from conftest import BLOCK_SIZE, ROOT, load_plain_weights

pytestmark = pytest.mark.gpu


def prompt_of(n, vocab, salt=0):
    return [(i * 5 + 1 + salt * 13) % vocab for i in range(n)]


def make_engine(folder, block_size, **kw):
    import tie_amd

    kw.setdefault("kv_blocks", 256)
    kw.setdefault("dtype", "float32")
    return tie_amd.create_engine(folder, block_size=block_size, **kw)


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point_matches_the_plain_implementation(model_folders, name):
    import tie_amd

    folder, cfg = model_folders[name]
    weights = load_plain_weights(folder)
    for n in (1, 9, 30):
        prompt = prompt_of(n, cfg["vocab_size"], n)
        want = plain.greedy(weights, cfg, prompt, 12)
        got = tie_amd.generate(folder, prompt, tie_amd.SamplingParams(max_tokens=12), dtype="float32",
                               block_size=BLOCK_SIZE[name], kv_blocks=64)
        assert got == want


@pytest.mark.parametrize("name", ["A", "B"])
def test_bfloat16_greedy_generation_follows_the_plain_implementation(model_folders_bf16, name):
    """Every token of a bfloat16 greedy run is, given the tokens before it, the plain logits' maximum or within the
    fixture's bound of it (a near-tie may fall either way, after which the two runs go their own ways: so each
    token is judged against the plain logits of the engine's own prefix, not against the plain run's tokens)."""
    import tie_amd

    folder, cfg = model_folders_bf16[name]
    weights = load_plain_weights(folder)
    bound = tolerances.BFLOAT16["tiny " + name]
    agree = 0
    for n in (1, 9, 23):
        prompt = prompt_of(n, cfg["vocab_size"], n)
        got = tie_amd.generate(folder, prompt, tie_amd.SamplingParams(max_tokens=8), dtype="bfloat16",
                               block_size=BLOCK_SIZE[name], kv_blocks=64)
        assert len(got) == 8
        logits = plain.forward(weights, cfg, prompt + got)
        for k, token in enumerate(got):
            row = logits[len(prompt) + k - 1]
            assert float(row.max() - row[token]) <= bound * float(row.abs().max()), \
                f"prompt of {n}: token {k} ({token}) is not what the plain logits favour ({int(row.argmax())})"
            agree += int(token == int(row.argmax()))
    assert agree >= 20, f"only {agree} of 24 tokens are the plain logits' maxima"


def test_the_command_line_generates_the_same_tokens(model_folders):
    folder, cfg = model_folders["B"]
    prompt = prompt_of(11, cfg["vocab_size"])
    want = plain.greedy(load_plain_weights(folder), cfg, prompt, 6)
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "tie"), "generate", "-m", folder, "-p",
                           ",".join(map(str, prompt)), "--temp", "0", "--max-tokens", "6", "--dtype", "float32",
                           "--kv-mem", "16M"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == want
    assert "[tie] hip | load" in proc.stderr and "6 tok generated" in proc.stderr
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "tie"), "generate", "-m", folder + "/missing", "-p", "1"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 1 and "tie: error:" in proc.stderr


def test_the_command_line_runs_a_workload_and_prints_its_report(model_folders, tmp_path):
    import json

    folder, cfg = model_folders["A"]
    run = lambda *a: subprocess.run([sys.executable, str(ROOT / "bin" / "tie"), "bench", "-m", folder, "--dtype", "float32",
                                     "--block-size", "4", "--kv-blocks", "20", "--max-seqs", "4",
                                     "--max-tokens-per-step", "16", *a], capture_output=True, text=True, timeout=600)
    proc = run("--synthetic", "9", "--prompt-len", "3:20", "--output-len", "2:6", "--seed", "3", "--json")
    assert proc.returncode == 0, proc.stderr[-2000:]
    report = json.loads(proc.stdout)
    assert report["requests"] == 9 and 18 <= report["output_tokens"] <= 54 and report["steps"] > 0
    assert report["total_tok_per_s"] > 0 and set(report["ttft_ms"]) == {"p50", "p90", "p99"}
    workload = tmp_path / "w.jsonl"
    workload.write_text('{"prompt_ids": [1, 2, 3], "max_tokens": 4}\n{"prompt_ids": [9, 8]}\n')
    proc = run("--prompts", str(workload), "--max-tokens", "3", "--rate", "50")
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "requests 2" in proc.stdout and "5 prompt + 7 output" in proc.stdout and "ttft" in proc.stdout
    workload.write_text('{"prompt": "text"}\n')
    proc = run("--prompts", str(workload))
    assert proc.returncode == 1 and "tokenizer" in proc.stderr


def test_stop_token_max_tokens_and_pages_returned(model_folders):
    import tie_amd

    folder, cfg = model_folders["A"]
    engine = make_engine(folder, 4)
    prompt = prompt_of(7, cfg["vocab_size"])
    free = engine.cache.num_free()
    out = engine.generate(prompt, tie_amd.SamplingParams(max_tokens=9))
    assert len(out) == 9 and engine.cache.num_free() == free and not engine.has_work()
    stopper = make_engine(folder, 4, stop_tokens=[out[3]])
    first = out.index(out[3])
    assert stopper.generate(prompt, tie_amd.SamplingParams(max_tokens=9)) == out[:first + 1]   # the stop token is kept
    assert stopper.cache.num_free() == free


def test_chunked_prefill_generates_the_unchunked_tokens(model_folders):
    import tie_amd

    folder, cfg = model_folders["B"]
    prompt = prompt_of(40, cfg["vocab_size"])
    params = tie_amd.SamplingParams(max_tokens=10)
    whole = make_engine(folder, 16, max_seqs=1, max_tokens_per_step=64).generate(prompt, params)
    for kw in (dict(max_tokens_per_step=5), dict(max_tokens_per_step=64, prefill_chunk=13)):
        engine = make_engine(folder, 16, max_seqs=1, **kw)
        assert engine.generate(prompt, params) == whole
        assert engine.stats().steps > 10 and engine.stats().prefill_tokens == 40 and engine.stats().decode_tokens == 9


def test_capacity_rejections_and_clamping(model_folders):
    import tie_amd
    from tie_amd.errors import CapacityError, InvalidArgument

    folder, cfg = model_folders["A"]                      # context 128
    engine = make_engine(folder, 4, kv_blocks=10)         # the pool holds 40 tokens
    with pytest.raises(InvalidArgument, match="at least one prompt token"):
        engine.add_request([])
    with pytest.raises(InvalidArgument, match="not in the vocabulary"):
        engine.add_request([1, cfg["vocab_size"]])
    with pytest.raises(CapacityError, match="the cache of 10 pages"):
        engine.add_request([1] * 40)
    sid = engine.add_request([1] * 30, tie_amd.SamplingParams(max_tokens=100))
    assert engine.sequence(sid).params.max_tokens == 10   # clamped to the room the pool leaves
    while engine.has_work():
        engine.step()
    assert engine.sequence(sid).num_generated == 10 and engine.sequence(sid).finish_reason.value == "length"
    big = make_engine(folder, 4, kv_blocks=64)
    with pytest.raises(CapacityError, match="the model's context holds 128"):
        big.add_request([1] * 128)


def mixed_requests(vocab, sampled):
    import tie_amd

    lens, outs = [3, 17, 9, 30, 1, 12, 25, 6], [10, 4, 12, 8, 6, 9, 5, 11]     # test_engine_batching.cpp:26-41
    reqs = []
    for i, (n, m) in enumerate(zip(lens, outs)):
        prompt = [(t * 7 + i * 13 + 1) % vocab for t in range(n)]
        p = tie_amd.SamplingParams(max_tokens=m)
        if sampled:
            p = tie_amd.SamplingParams(max_tokens=m, temperature=0.8, top_k=10 if i % 2 else 0, seed=100 + i)
        reqs.append((prompt, p))
    return reqs


@pytest.mark.parametrize("sampled", [False, True])
@pytest.mark.parametrize("kv_blocks", [256, 12])          # 12 pages of 4 tokens force preemption
def test_requests_batched_together_generate_what_each_generates_alone(model_folders, sampled, kv_blocks):
    folder, cfg = model_folders["A"]
    reqs = mixed_requests(cfg["vocab_size"], sampled)
    together = make_engine(folder, 4, kv_blocks=kv_blocks, max_seqs=8, max_tokens_per_step=16, policy="fcfs")
    ids = [together.add_request(p, s) for p, s in reqs]
    while together.has_work():
        together.step()
    stats = together.stats()
    if kv_blocks == 12:
        assert stats.preemptions > 0
    assert stats.seqs_scheduled > stats.steps                 # really batched
    assert together.cache.num_free() == kv_blocks
    for sid, (prompt, params) in zip(ids, reqs):
        alone = make_engine(folder, 4, max_seqs=1, max_tokens_per_step=16)
        assert alone.generate(prompt, params) == together.sequence(sid).generated, f"request {sid}"


def test_admission_by_the_whole_pending_input_generates_the_same_tokens_with_fewer_evictions(model_folders):
    """A scarce pool and prompts in portions of 8: by the first portion (the reference's rule) prompts enter that the
    pool cannot hold and are evicted on a later portion; by the whole input they wait. The tokens are the same."""
    folder, cfg = model_folders["A"]
    reqs = mixed_requests(cfg["vocab_size"], False)
    evictions, generated = {}, {}
    for whole in (False, True):
        engine = make_engine(folder, 4, kv_blocks=12, max_seqs=8, max_tokens_per_step=16, prefill_chunk=8,
                             policy="fcfs", admit_whole=whole)
        ids = [engine.add_request(p, s) for p, s in reqs]
        while engine.has_work():
            engine.step()
        assert engine.cache.num_free() == 12
        evictions[whole] = engine.stats().preemptions
        generated[whole] = [engine.sequence(sid).generated for sid in ids]
    assert generated[True] == generated[False]
    assert evictions[True] < evictions[False]


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_a_crowded_engine_finishes_everything_twice_the_same_way(model_folders, model_folders_bf16, dtype):
    """Thirty requests of mixed lengths and sampling through a small pool: chunked prompts, decode steps
    replayed from recorded graphs, preemption and recomputation. Everything finishes with the right
    number of tokens, every page comes back, and a second engine fed the same way produces the same
    tokens (the same batches run the same kernels in the same order: nothing depends on timing)."""
    import random

    import tie_amd

    folder, cfg = (model_folders_bf16 if dtype == "bfloat16" else model_folders)["B"]
    rng = random.Random(12)
    reqs = []
    for i in range(30):
        prompt = [rng.randrange(cfg["vocab_size"]) for _ in range(rng.choice([1, 3, 17, 40, 75]))]
        kind = i % 3
        params = tie_amd.SamplingParams(max_tokens=rng.choice([1, 5, 24]), seed=i,
                                        temperature=0.0 if kind == 0 else 0.8,
                                        top_k=0 if kind < 2 else 10, top_p=1.0 if kind < 2 else 0.9)
        reqs.append((prompt, params))

    def run():
        engine = make_engine(folder, 16, dtype=dtype, kv_blocks=14, max_seqs=6, max_tokens_per_step=48,
                             prefill_chunk=32, policy="fcfs", watermark_blocks=0)
        pending = list(reqs)
        ids = []
        steps = 0
        while pending or engine.has_work():
            for _ in range(2):                                # requests keep arriving while others run
                if pending:
                    ids.append(engine.add_request(*pending.pop(0)))
            engine.step()
            steps += 1
            engine.cache.audit([engine.sequence(i).cache for i in ids if engine.sequence(i).cache is not None])
            assert steps < 3000, "the engine does not finish"
        assert engine.cache.num_free() == 14
        out = [engine.sequence(i).generated for i in ids]
        for (prompt, params), tokens in zip(reqs, out):
            assert len(tokens) == params.max_tokens
            assert all(0 <= t < cfg["vocab_size"] for t in tokens)
        return out, engine.stats()

    first, stats = run()
    assert stats.preemptions > 0 and stats.seqs_scheduled > 2 * stats.steps
    second, _ = run()
    assert first == second
    # And against the plain implementation: every token a greedy request chose is, given the tokens before it,
    # the plain logits' maximum or within the precision's tolerance of it (a near-tie may fall either way).
    weights = load_plain_weights(folder)
    tolerance = tolerances.BFLOAT16["tiny B"] if dtype == "bfloat16" else tolerances.FLOAT32
    checked = 0
    for (prompt, params), tokens in zip(reqs, first):
        if params.temperature != 0.0:
            continue
        logits = plain.forward(weights, cfg, list(prompt) + tokens)
        for k, token in enumerate(tokens):
            row = logits[len(prompt) + k - 1]
            assert float(row.max() - row[token]) <= tolerance * float(row.abs().max()), \
                f"token {k} of a greedy request is not what the plain logits favour"
            checked += 1
    assert checked > 50


def test_a_workload_through_the_bench_runner(model_folders):
    """``tie bench``'s loop over a pool too small for its requests: every request gets its tokens, evictions
    happen, the report's counts are the engine's, and every page and sequence is given back."""
    from tie_amd.bench import assign_arrivals, run_workload, summarize, synthetic_requests

    folder, cfg = model_folders["A"]
    requests = synthetic_requests(14, (3, 30), (2, 9), cfg["vocab_size"], seed=5)
    assign_arrivals(requests, float("inf"), seed=5)
    for late in requests[-3:]:
        late.arrival = 0.01                                  # three arrive while the others run
    engine = make_engine(folder, 4, kv_blocks=14, max_seqs=6, max_tokens_per_step=24, prefill_chunk=8)
    run = run_workload(engine, requests)
    report = summarize(run)
    assert report.requests == 14 and report.prompt_tokens == sum(len(r.prompt) for r in requests)
    assert report.output_tokens == sum(r.max_tokens for r in requests)
    assert report.preemptions > 0 and report.steps == engine.stats().steps and report.mean_seqs_per_step > 1.5
    assert engine.cache.num_free() == 14 and not engine.sequences and not engine.has_work()
    for timing, request in zip(run.requests, requests):
        times = timing.token_times
        assert len(times) == request.max_tokens and times == sorted(times) and times[0] >= timing.arrival
    assert 0 < report.ttft_ms["p50"] <= report.ttft_ms["p99"] <= report.e2e_ms["p99"]
    # the tokens are those each request generates alone
    seen = {}
    engine.on_token = lambda seq_id, token: seen.setdefault(seq_id, []).append(token)
    ids = [engine.add_request(r.prompt, tie_amd_params(r.max_tokens)) for r in requests]
    while engine.has_work():
        engine.step()
    for sid, r in zip(ids, requests):
        alone = make_engine(folder, 4, max_seqs=1, max_tokens_per_step=16)
        assert alone.generate(r.prompt, tie_amd_params(r.max_tokens)) == seen[sid]


def tie_amd_params(max_tokens):
    import tie_amd

    return tie_amd.SamplingParams(max_tokens=max_tokens, temperature=0.0)


def test_a_failing_step_is_rolled_back_and_offered_again(model_folders):
    import tie_amd

    folder, cfg = model_folders["A"]
    reqs = mixed_requests(cfg["vocab_size"], False)
    engine = make_engine(folder, 4, max_seqs=8, max_tokens_per_step=16, policy="fcfs")
    calls = {"n": 0}

    def hook(index, x):
        if index == 1:
            calls["n"] += 1
            if calls["n"] == 3:
                raise RuntimeError("injected failure")

    engine.model.layer_hook = hook
    ids = [engine.add_request(p, s) for p, s in reqs]
    failures = 0
    while engine.has_work():
        try:
            engine.step()
        except RuntimeError:
            failures += 1
    assert failures == 1
    engine.model.layer_hook = None
    for sid, (prompt, params) in zip(ids, reqs):
        alone = make_engine(folder, 4, max_seqs=1, max_tokens_per_step=16)
        assert alone.generate(prompt, params) == engine.sequence(sid).generated


def test_cancel_release_and_callbacks(model_folders):
    import tie_amd
    from tie_amd.errors import InvalidArgument

    folder, cfg = model_folders["A"]
    engine = make_engine(folder, 4, max_seqs=4, max_tokens_per_step=32)
    seen = []
    a = engine.add_request(prompt_of(5, 256), tie_amd.SamplingParams(max_tokens=20))
    b = engine.add_request(prompt_of(6, 256, 1), tie_amd.SamplingParams(max_tokens=5))

    def on_token(seq_id, token):
        seen.append((seq_id, token))
        if seq_id == a and len([s for s in seen if s[0] == a]) == 3:
            engine.cancel(a)                                  # safe from a token callback
        with pytest.raises(InvalidArgument):
            engine.step()                                     # but stepping inside a step is refused

    engine.on_token = on_token
    with pytest.raises(InvalidArgument, match="has not finished"):
        engine.release(a)
    while engine.has_work():
        engine.step()
    assert engine.sequence(a).finish_reason.value == "cancelled" and engine.sequence(a).num_generated == 3
    assert engine.sequence(b).num_generated == 5
    engine.release(a)
    with pytest.raises(InvalidArgument, match="knows no sequence"):
        engine.sequence(a)
    assert engine.cache.num_free() == engine.cache.num_blocks


def test_a_request_whose_sampling_the_kernels_cannot_take_is_refused_when_it_is_added(model_folders, monkeypatch):
    """The drawing kernels take vocabularies up to a size of their own; a request that would need more is
    refused with that size named, before anything runs, and a greedy request goes through."""
    import tie_amd
    from tie_amd import kernels
    from tie_amd.errors import InvalidArgument

    folder, cfg = model_folders["A"]
    engine = make_engine(folder, 4)
    monkeypatch.setattr(kernels, "MAX_FILTERED_VOCAB", cfg["vocab_size"] - 1)
    with pytest.raises(InvalidArgument, match=f"top-k / top-p takes vocabularies of up to {cfg['vocab_size'] - 1}"):
        engine.add_request([1, 2, 3], tie_amd.SamplingParams(temperature=0.7, top_k=5))
    engine.add_request([1, 2, 3], tie_amd.SamplingParams(temperature=0.7, max_tokens=2))      # no filter: the other kernel
    while engine.has_work():
        engine.step()
    monkeypatch.setattr(kernels, "MAX_SAMPLED_VOCAB", cfg["vocab_size"] - 1)
    with pytest.raises(InvalidArgument, match="a temperature takes vocabularies"):
        engine.add_request([1, 2, 3], tie_amd.SamplingParams(temperature=0.7))
    engine.add_request([1, 2, 3], tie_amd.SamplingParams(max_tokens=2))
    while engine.has_work():
        engine.step()


def test_device_sampling_matches_the_host_sampler():
    import numpy as np
    from tie_amd.sampling import DeviceSampler, RandomStream, SamplingParams, sample

    g = torch.Generator().manual_seed(4)
    logits = (torch.randn(6, 1000, generator=g) * 3).cuda()
    logits[0, 17] = logits[0].max() + 1
    logits[0, 400] = logits[0, 17]                            # a tie: the lowest id wins
    logits[5, 3] = float("inf")
    params = [SamplingParams(), SamplingParams(temperature=0.8, seed=1), SamplingParams(temperature=1.5, seed=2),
              SamplingParams(temperature=0.7, top_k=20, top_p=0.8, seed=3), SamplingParams(temperature=1e-40),
              SamplingParams(temperature=1.0, seed=5)]
    sampler = DeviceSampler("cuda:0")
    dev_rngs = [RandomStream(p.seed) for p in params]
    host_rngs = [RandomStream(p.seed) for p in params]
    host = logits.cpu().numpy()
    for _ in range(50):
        got = sampler.sample_rows(logits, params, dev_rngs)
        want = [sample(host[i], params[i], host_rngs[i]) for i in range(6)]
        assert got == want
    assert got[0] == 17 and got[5] == 3
    bad = logits.clone()
    bad[2, 9] = float("nan")
    from tie_amd.errors import InvalidArgument
    with pytest.raises(InvalidArgument, match="NaN"):
        sampler.sample_rows(bad, params, dev_rngs)


def test_steps_queued_before_the_one_before_is_read_draw_the_same_tokens():
    """``launch`` with the ticket of the step before, collected one step late, against the host rule row by row:
    greedy, temperature and top-k / top-p rows side by side, over steps whose logits change, one of them with a
    +inf logit in a drawing row - that row takes no number from its stream, which the next step, already
    queued, can only know on the GPU."""
    from tie_amd.sampling import DeviceSampler, RandomStream, SamplingParams, sample

    g = torch.Generator().manual_seed(12)
    steps = [(torch.randn(5, 3000, generator=g) * 3) for _ in range(12)]
    steps[3][1, 77] = float("inf")           # a temperature row
    steps[4][3, 5] = float("inf")            # a top-k / top-p row, in the step right after
    steps[4][3, 2000] = float("inf")
    steps[8][1, 9] = steps[8][3, 9] = float("inf")
    steps[9][1, 9] = float("inf")            # twice in a row
    params = [SamplingParams(), SamplingParams(temperature=0.9, seed=1), SamplingParams(temperature=0.7, top_k=40, seed=2),
              SamplingParams(temperature=1.3, top_p=0.6, seed=3), SamplingParams(temperature=0.5, top_k=3000, seed=4)]
    host_rngs = [RandomStream(p.seed) for p in params]
    want = [[sample(step[i].numpy(), params[i], host_rngs[i]) for i in range(5)] for step in steps]
    sampler = DeviceSampler("cuda:0")
    rngs = [RandomStream(p.seed) for p in params]
    got, waiting = [], None
    for step in steps:
        ticket = sampler.launch(step.cuda(), params, rngs, waiting)
        if waiting is not None:
            got.append(sampler.collect(waiting))
        waiting = ticket
    got.append(sampler.collect(waiting))
    assert got == want
    assert [r.unit() for r in rngs] == [r.unit() for r in host_rngs]        # the streams stand where the host's do
    # read at once, as a step outside the steady state is
    rngs = [RandomStream(p.seed) for p in params]
    assert [sampler.sample_rows(step.cuda(), params, rngs) for step in steps] == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kv_blocks", [256, 14])
@pytest.mark.parametrize("drawing", [False, True])
def test_steps_launched_ahead_generate_the_same_tokens(model_folders, model_folders_bf16, dtype, kv_blocks, drawing):
    """Requests with the next step queued before the last one's tokens are read, against the same engine
    reading every step at once: equal tokens, through stop tokens (a sequence then ran one token too many,
    which must leave no trace), ends by length, a cancellation and, with 14 pages, evictions. ``drawing``: the
    requests sample, each in its own way (temperature, top-k, top-p, one greedy) from its own stream."""
    import tie_amd

    ways = [dict(temperature=0.8, seed=3), dict(temperature=0.7, top_k=20, top_p=0.8, seed=4), dict(),
            dict(temperature=1.4, top_p=0.9, seed=5), dict(temperature=0.6, top_k=5, seed=6), dict(temperature=1.0, seed=7)]
    if not drawing:
        ways = [dict()] * 6

    folder, cfg = (model_folders_bf16 if dtype == "bfloat16" else model_folders)["A"]
    vocab = cfg["vocab_size"]
    reqs = [([(t * 7 + i * 13 + 1) % vocab for t in range(n)], m)
            for i, (n, m) in enumerate(zip([3, 17, 9, 21, 1, 12], [30, 14, 40, 8, 26, 33]))]

    def run(ahead, stop_tokens=()):
        engine = make_engine(folder, 4, dtype=dtype, kv_blocks=kv_blocks, max_seqs=8, max_tokens_per_step=32,
                             launch_ahead=ahead, stop_tokens=stop_tokens)
        seen = []
        engine.on_token = lambda seq_id, token: seen.append((seq_id, token))
        ids = [engine.add_request(p, tie_amd.SamplingParams(max_tokens=m, **way)) for (p, m), way in zip(reqs, ways)]
        steps = 0
        while engine.has_work():
            engine.step()
            steps += 1
            if steps == 12:
                engine.cancel(ids[2])
            assert steps < 2000
        assert engine.cache.num_free() == kv_blocks and not engine._unread
        out = [engine.sequence(i).generated for i in ids]
        reasons = [engine.sequence(i).finish_reason.value for i in ids]
        for i, tokens in zip(ids, out):
            assert [t for s, t in seen if s == i] == tokens and -1 not in tokens
        return out, reasons, engine

    plain_out, plain_reasons, _ = run(False)
    ahead_out, ahead_reasons, engine = run(True)
    assert engine.steps_launched_ahead > 10
    if kv_blocks == 14:
        assert engine.stats().preemptions > 0, "14 pages were meant to force evictions"
    for i in (0, 1, 3, 4, 5):                                  # (the cancelled one stops wherever it was)
        assert ahead_out[i] == plain_out[i] and ahead_reasons[i] == plain_reasons[i] == "length"
    # a stop token in the middle of some outputs
    stop = plain_out[0][7]
    s_plain, r_plain, _ = run(False, stop_tokens=(stop,))
    s_ahead, r_ahead, engine = run(True, stop_tokens=(stop,))
    assert "stop" in r_plain and engine.steps_launched_ahead > 0
    for i in (0, 1, 3, 4, 5):
        assert s_ahead[i] == s_plain[i] and r_ahead[i] == r_plain[i]
        if r_plain[i] == "stop":
            assert s_plain[i][-1] == stop and stop not in s_plain[i][:-1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_eviction_while_tokens_are_unread_loses_no_request(model_folders, model_folders_bf16, dtype):
    """Four requests decode in step, nobody waits, their tokens are read a step late, and all four need their second
    page in the same step from a pool with one page to spare: requests are evicted with a token still unread, two
    wait afterwards. Everyone finishes with the tokens of the engine that reads every step at once."""
    import tie_amd

    folder, cfg = (model_folders_bf16 if dtype == "bfloat16" else model_folders)["A"]
    vocab = cfg["vocab_size"]
    prompts = [prompt_of(3, vocab, salt) for salt in range(4)]

    def run(ahead):
        engine = make_engine(folder, 4, dtype=dtype, kv_blocks=5, max_seqs=4, max_tokens_per_step=16,
                             launch_ahead=ahead, policy="fcfs")
        ids = [engine.add_request(p, tie_amd.SamplingParams(max_tokens=9)) for p in prompts]
        steps = 0
        while engine.has_work():
            engine.step()
            steps += 1
            assert steps < 500, "a request was lost: the engine never comes to an end"
        assert engine.cache.num_free() == 5
        return [engine.sequence(i).generated for i in ids], engine

    plain_out, _ = run(False)
    ahead_out, engine = run(True)
    assert engine.ahead_replans > 0 and engine.stats().preemptions >= 2 and engine.steps_launched_ahead > 0
    assert ahead_out == plain_out and all(len(out) == 9 for out in ahead_out)
