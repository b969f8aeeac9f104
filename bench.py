"""Decode and prefill throughput of the engine on one MI355X, Qwen3-8B shape, random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --shape 32b                 the same measurements at the Qwen3-32B sizes
    python bench.py --sweep [--shape 32b]       decode at contexts 4096 / 16384 / 32768 x batch 1 / 8 / 32, a line a point
    python bench.py --workload stress           64 requests through the scheduler at the Qwen3-1.7B sizes

Prints ONE JSON line. A "step" is one decode step of the engine (schedule, build the batch, run
the model, sample greedily) at the default batch of 8 with every sequence near the benchmark
context length; ``value`` is decoded tokens a second. The same line carries

* ``prefill``: tokens a second of one 2048-token prompt run as one step, and the fraction of the
  bf16 MFMA peak its flops reach;
* ``roofline``: the bytes a decode step has to read (every weight it uses once, and the cache of
  the live requests) divided by its time, against the HBM peak;
* ``points``: decoded tokens a second at batch 1 and at batch 64, and for each of them (keys
  ``decode_b1_...``) the step time, the bytes read and the same two fractions.

Every decode point times the same ``--steps`` steps. ``ms_per_step`` and ``value`` come from the wall clock
around exactly those steps; ``ms_per_step_median`` is the median of the steps' own times, taken from GPU
events recorded after each. Beside the fractions of the published peaks (HBM 8 TB/s, 2.5 PFLOP/s) stand
``measured_peak`` and ``frac_of_measured``: what a kernel that only reads cold memory, and one that only issues
matrix instructions, reach on this very GPU in this process (``tie_amd.bench.peaks``).

The sizes are those of a Qwen3-8B config.json; weights are random (N(0, 0.02), norm weights
1 + U(-0.1, 0.1)) and token ids are uniform, since neither checkpoints nor datasets exist here.

``--workload stress`` is another measurement with a JSON line of its own: 64 requests at once, prompts of
128 to 2048 tokens, 256 generated tokens each, prompts in portions of 512, a cache of 2 GB - far less than
the requests need together, so sequences are evicted and computed again. It reports what the reference's
bench report holds (``src/bench/report.h:29-36``): tokens a second, steps, mean sequences a step,
preemptions, and percentiles of the time to the first token, between tokens and of whole requests.
"""

import argparse
import json
import sys
import time

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 36, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8,
    "head_dim": 128, "intermediate_size": 12288, "vocab_size": 151936, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "max_position_embeddings": 40960,
}
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
QWEN3_1_7B = dict(QWEN3_8B, num_hidden_layers=28, hidden_size=2048, num_attention_heads=16, intermediate_size=6144,
                  tie_word_embeddings=True)
SHAPES = {"8b": ("Qwen3-8B", QWEN3_8B), "32b": ("Qwen3-32B", QWEN3_32B), "1.7b": ("Qwen3-1.7B", QWEN3_1_7B)}
BLOCK_SIZE = 16
PREFILL_TOKENS = 2048
PEAK_HBM_GBS = 8000.0          # MI355X: 8 TB/s
PEAK_FLOPS = {"bf16": 2.5e15}  # dense MFMA


def log(message):
    print(f"[bench] {message}", file=sys.stderr, flush=True)


def build_model(cfg, seed=0):
    import torch
    from tie_amd.models import expected_tensors_for_config, load_model_from_tensors
    from tie_amd.weights.random_init import random_tensors

    specs = [s for s in expected_tensors_for_config(cfg) if not s.optional]
    tensors = dict(random_tensors(specs, seed, torch.bfloat16, device="cuda"))
    model = load_model_from_tensors(cfg, tensors, "bfloat16", "cuda:0")
    del tensors
    torch.cuda.empty_cache()
    return model


def weight_bytes_per_step(cfg, batch):
    """Bytes of weights one decode step reads: every matrix once, the embedding rows of the batch, the norms."""
    D, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    Q = cfg["num_attention_heads"] * cfg["head_dim"]
    KV = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = (Q + 2 * KV) * D + D * Q + 2 * I * D + D * I
    matrices = (L * per_layer + V * D) * 2
    norms = (L * (2 * D + 2 * cfg["head_dim"]) + D) * 4
    return matrices + norms + batch * D * 2


def kv_bytes_per_token(cfg):
    return 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * cfg["head_dim"] * 2


def prefill_flops(cfg, T, R=1):
    D, I, V, L = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["num_hidden_layers"]
    Q = cfg["num_attention_heads"] * cfg["head_dim"]
    KV = cfg["num_key_value_heads"] * cfg["head_dim"]
    per_layer = (Q + 2 * KV) * D + D * Q + 2 * I * D + D * I
    gemm = 2 * T * L * per_layer + 2 * R * V * D
    attention = 2 * T * T * cfg["head_dim"] * cfg["num_attention_heads"] * L   # causal: QK^T and PV over T^2 / 2 pairs
    return gemm + attention


def measure_stress(model, cfg, args):
    """The scheduler under pressure: returns the report of the run as a dict (and checks every page came back)."""
    from tie_amd.api import create_engine
    from tie_amd.bench import assign_arrivals, report_json, run_workload, summarize, synthetic_requests

    engine = create_engine(model, kv_mem=args.kv_mem, block_size=BLOCK_SIZE, max_seqs=args.requests,
                           max_tokens_per_step=args.portion, prefill_chunk=args.portion, launch_ahead=args.launch_ahead,
                           admit_whole=args.admit_whole)
    from tie_amd.bench.workload import parse_range

    requests = synthetic_requests(args.requests, parse_range("--prompt-len", args.prompt_len),
                                  parse_range("--output-len", args.output_len), cfg["vocab_size"], seed=0)
    assign_arrivals(requests, args.rate, seed=0)
    warm = synthetic_requests(4, (600, 700), (8, 8), cfg["vocab_size"], seed=1)       # compiles nothing, but warms up
    run_workload(engine, warm)
    log(f"stress: {args.requests} requests, {sum(len(r.prompt) for r in requests)} prompt tokens, "
        f"a cache of {engine.cache.num_blocks} pages ({engine.cache.num_blocks * BLOCK_SIZE} tokens)")
    run = run_workload(engine, requests, progress=log)
    assert engine.cache.num_free() == engine.cache.num_blocks, "a page was not given back"
    report = report_json(summarize(run))
    report["kv_blocks"] = engine.cache.num_blocks
    report["graph_replays"] = engine.runner.graph_replays
    report["graphs_recorded"] = len(engine.runner._recorded)
    return report


def measure_long_prompt(model, cfg, args):
    """One prompt of ``--prompt-tokens`` tokens through the engine in portions of ``--portion``, then 16 decoded
    tokens: steps with a prompt portion run eagerly from the host, so this shows what the host costs them."""
    import random

    import torch
    from tie_amd.api import create_engine
    from tie_amd.sampling.params import SamplingParams

    tokens, portion = args.prompt_tokens, args.portion
    blocks = -(-(tokens + 64) // BLOCK_SIZE) + 8
    engine = create_engine(model, kv_blocks=blocks, block_size=BLOCK_SIZE, max_seqs=1, max_tokens_per_step=portion,
                           prefill_chunk=portion, policy="fcfs", watermark_blocks=0, max_seq_len=tokens + 64,
                           launch_ahead=args.launch_ahead)
    rng = random.Random(11)
    best = None
    for i in range(3):                        # the first run warms up
        sid = engine.add_request([rng.randrange(cfg["vocab_size"]) for _ in range(tokens)], SamplingParams(max_tokens=16))
        torch.cuda.synchronize()
        start = time.perf_counter()
        steps = 0
        while engine.sequence(sid).num_generated < 1:
            engine.step()
            steps += 1
        torch.cuda.synchronize()
        prefill_s = time.perf_counter() - start
        while engine.has_work():
            engine.step()
        torch.cuda.synchronize()
        total_s = time.perf_counter() - start
        engine.release(sid)
        log(f"long prompt: {tokens} tokens in {steps} steps of up to {portion}: {prefill_s * 1e3:.1f} ms to the first "
            f"token, {total_s * 1e3:.1f} ms with 16 tokens")
        if i > 0 and (best is None or prefill_s < best["prefill_s"]):
            best = {"prompt_tokens": tokens, "portion": portion, "steps": steps, "prefill_s": prefill_s,
                    "total_s": total_s, "prefill_tok_per_s": tokens / prefill_s}
    return best


def make_engine(model, batch, context, max_tokens_per_step, launch_ahead=True, long_sequences=0, short_context=0):
    from tie_amd.api import create_engine

    blocks = batch * (-(-context // BLOCK_SIZE) + 1) + 8
    if 0 < long_sequences < batch:
        blocks = (long_sequences * (-(-context // BLOCK_SIZE) + 1) +
                  (batch - long_sequences) * (-(-short_context // BLOCK_SIZE) + 1) + 8)
    return create_engine(model, kv_blocks=blocks, block_size=BLOCK_SIZE, max_seqs=max(batch, 1),
                         max_tokens_per_step=max(max_tokens_per_step, batch), policy="fcfs", watermark_blocks=0,
                         max_seq_len=context, launch_ahead=launch_ahead)


def measure_decode(model, cfg, batch, context, steps, warmup, chunk, sampling=None, long_sequences=0,
                   short_context=0):
    """Times ``steps`` decode steps of ``batch`` sequences whose contexts end at (just below) ``context`` tokens;
    with ``long_sequences`` > 0 only that many of them do and the others end at ``short_context``.

    The prompts are prefilled through the engine first (untimed). Sequences that finish their prompt
    early decode while the others still prefill, so every prompt is shortened by the number of steps
    the prefill phase takes: no sequence outgrows ``context`` before the timed steps are over.
    Returns (seconds, mean context length over the timed steps and sequences, graph replays, the median of
    the steps' own times in seconds: a GPU event is recorded behind every step, and in the steady state, where
    the GPU never waits for the host, the time between two of them is one step's).
    """
    import random

    import torch
    from tie_amd.engine.sequence import SeqState
    from tie_amd.sampling.params import SamplingParams

    engine = make_engine(model, batch, context, chunk, long_sequences=long_sequences, short_context=short_context)
    rng = random.Random(batch)
    slack = -(-batch * context // chunk) + batch + 2          # steps the prefill phase may take
    prompt_len = context - (steps + warmup) - slack - 1
    lengths = [prompt_len if long_sequences <= 0 or i < long_sequences else short_context - (context - prompt_len)
               for i in range(batch)]
    assert min(lengths) > 0, "context too short for this many steps"
    ids = [engine.add_request([rng.randrange(cfg["vocab_size"]) for _ in range(lengths[i])],
                              SamplingParams(max_tokens=steps + warmup + slack + 1, seed=i, **(sampling or {})))
           for i in range(batch)]
    started = time.perf_counter()
    last_log = started
    while any(engine.sequence(i).state != SeqState.DECODING for i in ids):
        engine.step()
        if time.perf_counter() - last_log > 20:
            done = sum(engine.sequence(i).state == SeqState.DECODING for i in ids)
            log(f"batch {batch}: prefilling, {done} of {batch} sequences done")
            last_log = time.perf_counter()
    torch.cuda.synchronize()
    log(f"batch {batch}: prefilled {sum(lengths)} tokens in {time.perf_counter() - started:.1f} s "
        f"({engine.stats().steps} steps)")
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    first = sum(engine.sequence(i).num_computed + 1 for i in ids) / batch
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    start = time.perf_counter()
    marks[0].record()
    for k in range(steps):
        engine.step()
        marks[k + 1].record()
    torch.cuda.synchronize()
    seconds = time.perf_counter() - start
    own = sorted(marks[k].elapsed_time(marks[k + 1]) * 1e-3 for k in range(steps))
    median = own[steps // 2] if steps % 2 else (own[steps // 2 - 1] + own[steps // 2]) / 2
    last = sum(engine.sequence(i).num_computed for i in ids) / batch
    assert all(engine.sequence(i).state == SeqState.DECODING for i in ids), "a sequence finished during the timed steps"
    assert max(engine.sequence(i).num_computed for i in ids) <= context
    assert engine.stats().preemptions == 0
    replays = engine.runner.graph_replays
    del engine
    torch.cuda.empty_cache()
    return seconds, (first + last) / 2, replays, median


def measure_prefill(model, cfg, tokens, repeats=3):
    import random

    import torch
    from tie_amd.sampling.params import SamplingParams

    engine = make_engine(model, 1, tokens + 16, tokens, launch_ahead=False)   # the step's token is read inside the step
    rng = random.Random(7)
    best = None
    for i in range(repeats + 1):               # the first run warms up
        prompt = [rng.randrange(cfg["vocab_size"]) for _ in range(tokens)]
        sid = engine.add_request(prompt, SamplingParams(max_tokens=1))
        torch.cuda.synchronize()
        start = time.perf_counter()
        engine.step()                          # the whole prompt in one step, one logits row, one sampled token
        torch.cuda.synchronize()
        seconds = time.perf_counter() - start
        assert engine.sequence(sid).num_generated == 1
        engine.release(sid)
        if i > 0:
            best = seconds if best is None else min(best, seconds)
    del engine
    torch.cuda.empty_cache()
    return best


def main():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=64)
    parser.add_argument("--warmup", type=int, default=8)
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=4096, help="context length the timed decode steps end at")
    parser.add_argument("--layers", type=int, default=0, help="run fewer layers than the shape has (0 = all)")
    parser.add_argument("--shape", choices=sorted(SHAPES), default=None,
                        help="layer sizes: 8b (default), 32b, or 1.7b (the default of --workload stress)")
    parser.add_argument("--workload", choices=["decode", "stress", "long-prompt"], default="decode",
                        help="decode: the headline measurement; stress: many requests through a small cache; "
                             "long-prompt: one long prompt in portions")
    parser.add_argument("--prompt-tokens", type=int, default=8192, help="long-prompt: tokens of the prompt")
    parser.add_argument("--portion", type=int, default=512, help="long-prompt and stress: tokens of a prompt portion (stress: also the token budget of a step)")
    parser.add_argument("--requests", type=int, default=64, help="stress: concurrent requests")
    parser.add_argument("--kv-mem", type=int, default=2 << 30, help="stress: bytes of cache")
    parser.add_argument("--rate", type=float, default=float("inf"), help="stress: requests a second (Poisson arrivals)")
    parser.add_argument("--prompt-len", default="128:2048", help="stress: prompt lengths A:B")
    parser.add_argument("--output-len", default="256", help="stress: generated tokens C or C:D")
    parser.add_argument("--admit-whole", action="store_true",
                        help="stress: a request enters when the pool can hold all of its prompt, not just its first portion")
    parser.add_argument("--launch-ahead", type=int, default=1,
                        help="stress, long-prompt: steps the engine may leave unread behind the one it queues (0: reads every step at once)")
    parser.add_argument("--skip-points", action="store_true", help="skip batch 1, batch 64 and the prefill")
    parser.add_argument("--temperature", type=float, default=0.0, help="decode: sampling temperature (0 = greedy)")
    parser.add_argument("--top-k", type=int, default=0, help="decode: with a temperature, keep the k most likely (0 = all)")
    parser.add_argument("--top-p", type=float, default=1.0, help="decode: with a temperature, nucleus mass (1 = all)")
    parser.add_argument("--long-sequences", type=int, default=0,
                        help="decode: only this many sequences of the batch reach --context, the others --short-context")
    parser.add_argument("--short-context", type=int, default=1024, help="decode: see --long-sequences")
    parser.add_argument("--shares-by-sequence", action="store_true",
                        help="decode: never plan key shares of one length for sequences of very different lengths")
    parser.add_argument("--sweep", action="store_true",
                        help="decode only, one JSON line for every (context, batch) of --sweep-contexts x --sweep-batches")
    parser.add_argument("--sweep-contexts", default="4096,16384,32768")
    parser.add_argument("--sweep-batches", default="1,8,32")
    parser.add_argument("--prefill-only", action="store_true",
                        help="run only the 2048-token prefill (for profiling); prints its figures alone")
    args = parser.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures a single-GPU engine: --gpus {args.gpus} is not supported, run it with --gpus 1")
        return 2

    import torch

    import pathlib
    sys.path.insert(0, str(pathlib.Path(__file__).resolve().parent))
    import tie_amd  # noqa: F401

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 1
    shape_name, shape = SHAPES[args.shape or ("1.7b" if args.workload == "stress" else "8b")]
    cfg = dict(shape)
    layers_of_shape = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    log(f"building {cfg['num_hidden_layers']} layers of the {shape_name} shape with random bf16 weights")
    started = time.perf_counter()
    model = build_model(cfg)
    log(f"model ready in {time.perf_counter() - started:.1f} s")

    if args.workload == "stress":
        report = measure_stress(model, cfg, args)
        print(json.dumps({
            "metric": f"total tok/s, {args.requests} concurrent requests, {shape_name} bf16, {args.kv_mem >> 20} MB of cache",
            "value": round(report["total_tok_per_s"], 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
            "dtype": "bf16", "data": "synthetic",
            "config": {"model": f"{shape_name} shape, random weights", "layers": layers_of_shape,
                       "layers_run": cfg["num_hidden_layers"], "requests": args.requests, "prompt_len": args.prompt_len,
                       "output_len": args.output_len, "prefill_chunk": args.portion, "max_tokens_per_step": args.portion, "kv_bytes": args.kv_mem,
                       "kv_block": BLOCK_SIZE, "policy": "srpt-aging", "admit_whole": int(args.admit_whole), "sampling": "greedy",
                       "launch_ahead": args.launch_ahead},
            "report": report}), flush=True)
        return 0

    if args.workload == "long-prompt":
        report = measure_long_prompt(model, cfg, args)
        print(json.dumps({
            "metric": f"prompt tok/s, one prompt of {args.prompt_tokens} tokens in portions of {args.portion}, {shape_name} bf16",
            "value": round(report["prefill_tok_per_s"], 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
            "dtype": "bf16", "data": "synthetic",
            "config": {"model": f"{shape_name} shape, random weights", "layers": layers_of_shape,
                       "layers_run": cfg["num_hidden_layers"], "prompt_tokens": args.prompt_tokens,
                       "portion": args.portion, "kv_block": BLOCK_SIZE, "launch_ahead": args.launch_ahead},
            "report": report}), flush=True)
        return 0

    if args.prefill_only:
        t = measure_prefill(model, cfg, PREFILL_TOKENS)
        flops = prefill_flops(cfg, PREFILL_TOKENS)
        print(json.dumps({"prefill": {"value": round(PREFILL_TOKENS / t, 1), "tokens": PREFILL_TOKENS,
                                      "ms": round(t * 1e3, 3), "frac": round(flops / t / PEAK_FLOPS["bf16"], 4)},
                          "layers_run": cfg["num_hidden_layers"]}), flush=True)
        return 0

    chunk = 8192
    if args.shares_by_sequence:
        from tie_amd import kernels

        kernels.BALANCED_SHARES_MAX_EQUAL = 0
    sampling = None
    if args.temperature > 0:
        sampling = {"temperature": args.temperature, "top_k": args.top_k, "top_p": args.top_p}
    from tie_amd.bench.peaks import measured_peaks

    peaks = measured_peaks()
    log(f"this GPU: a streaming read reaches {peaks['hbm_read_gbs']:.0f} GB/s, matrix instructions on registers "
        f"{peaks['mfma_bf16_tflops']:.0f} TFLOP/s")

    def decode_point(batch, context=None):
        """One decode measurement: ``--steps`` timed steps at ``batch``; the figures of its roofline."""
        seconds, mean_context, replays, median = measure_decode(model, cfg, batch, context or args.context, args.steps,
                                                                args.warmup, chunk, sampling, args.long_sequences,
                                                                args.short_context)
        ms = seconds / args.steps * 1e3
        step_bytes = weight_bytes_per_step(cfg, batch) + batch * mean_context * kv_bytes_per_token(cfg)
        achieved = step_bytes / (ms * 1e-3) / 1e9
        log(f"decode batch {batch}: {ms:.3f} ms/step (median of the steps {median * 1e3:.3f}), "
            f"{batch * args.steps / seconds:.1f} tok/s, {achieved:.0f} GB/s ({replays} replays)")
        return {"tok_s": batch * args.steps / seconds, "ms": ms, "median_ms": median * 1e3, "gb": step_bytes / 1e9,
                "gbs": achieved, "frac": achieved / PEAK_HBM_GBS, "frac_of_measured": achieved / peaks["hbm_read_gbs"]}

    if args.sweep:
        # One line a point: decode at the contexts and batch sizes named, for tables of other sizes than the headline's.
        for context in [int(c) for c in args.sweep_contexts.split(",")]:
            for batch in [int(b) for b in args.sweep_batches.split(",")]:
                point = decode_point(batch, context)
                print(json.dumps({"metric": f"decode tok/s @ batch {batch}, context {context}, {shape_name} bf16",
                                  "value": round(point["tok_s"], 2), "unit": "tokens/s", "steps": args.steps,
                                  "ms_per_step": round(point["ms"], 4), "ms_per_step_median": round(point["median_ms"], 4),
                                  "config": {"model": f"{shape_name} shape, random weights", "layers": layers_of_shape,
                                             "layers_run": cfg["num_hidden_layers"], "global_batch": batch,
                                             "seq_len": context, "kv_block": BLOCK_SIZE},
                                  "roofline": {"bound": "hbm", "bytes_gb": round(point["gb"], 3),
                                               "achieved": round(point["gbs"], 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                               "frac": round(point["frac"], 4),
                                               "measured_peak": round(peaks["hbm_read_gbs"], 1),
                                               "frac_of_measured": round(point["frac_of_measured"], 4)}}), flush=True)
        return 0

    main_point = decode_point(args.batch)
    result = {
        "metric": f"decode tok/s @ batch {args.batch}, {shape_name} bf16 (plus prefill tok/s @ 2048 and batch 1/64 points)",
        "value": round(main_point["tok_s"], 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(main_point["ms"], 4),
        "ms_per_step_median": round(main_point["median_ms"], 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "model": f"{shape_name} shape, random weights", "layers": layers_of_shape, "layers_run": cfg["num_hidden_layers"],
            "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
            "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": cfg["vocab_size"],
            "global_batch": args.batch, "seq_len": args.context, "long_sequences": args.long_sequences,
            "short_context": args.short_context if args.long_sequences else 0, "kv_block": BLOCK_SIZE, "kv_dtype": "bf16",
            "prefill_tokens": PREFILL_TOKENS, "parallelism": "single GPU",
            "sampling": "greedy" if sampling is None else f"temperature {args.temperature} top_k {args.top_k} top_p {args.top_p}",
        },
        "roofline": {"bound": "hbm", "achieved": round(main_point["gbs"], 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(main_point["frac"], 4), "bytes_gb": round(main_point["gb"], 3),
                     "measured_peak": round(peaks["hbm_read_gbs"], 1),
                     "frac_of_measured": round(main_point["frac_of_measured"], 4)},
    }
    if not args.skip_points:
        t = measure_prefill(model, cfg, PREFILL_TOKENS)
        flops = prefill_flops(cfg, PREFILL_TOKENS)
        result["prefill"] = {"value": round(PREFILL_TOKENS / t, 1), "tokens": PREFILL_TOKENS, "ms": round(t * 1e3, 3),
                             "frac": round(flops / t / PEAK_FLOPS["bf16"], 4),
                             "measured_peak_tflops": round(peaks["mfma_bf16_tflops"], 1),
                             "frac_of_measured": round(flops / t / 1e12 / peaks["mfma_bf16_tflops"], 4)}
        log(f"prefill {PREFILL_TOKENS}: {t * 1e3:.2f} ms, {PREFILL_TOKENS / t:.0f} tok/s, "
            f"{flops / t / 1e12:.1f} TFLOP/s")
        points = {}
        for b in (1, 64):
            point = main_point if b == args.batch else decode_point(b)
            key = f"decode_b{b}"
            points[key] = round(point["tok_s"], 2)            # tokens a second; the rest of the point beside it
            points[key + "_ms"] = round(point["ms"], 4)
            points[key + "_median_ms"] = round(point["median_ms"], 4)
            points[key + "_bytes_gb"] = round(point["gb"], 3)
            points[key + "_gbs"] = round(point["gbs"], 1)
            points[key + "_frac"] = round(point["frac"], 4)
            points[key + "_frac_of_measured"] = round(point["frac_of_measured"], 4)
        result["points"] = points
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
