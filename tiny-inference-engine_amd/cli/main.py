"""``tie``: the command line. ``tie generate`` prints the generated token ids, one line, and a
summary on standard error with the reference's fields (``src/cli/main.cpp:100-109``): load time,
prompt tokens, time to first token, prefill and decode rates, pages used. ``tie bench`` runs a
workload of many requests through the engine and prints the report of ``src/bench/report.cpp:61-88``.
Exit codes as in the reference: 1 for an error of the engine's own kinds, 2 for anything else."""

from __future__ import annotations

import json
import sys
import time
from typing import Sequence

from ..errors import InvalidArgument, TieError
from .args import USAGE, parse_bench_args, parse_generate_args, parse_int


def run_generate(argv: Sequence[str]) -> int:
    opt = parse_generate_args(argv)
    import torch

    from ..api import create_engine
    from ..engine.sequence import SeqState
    from ..errors import KernelUnavailable

    if not torch.cuda.is_available():
        raise KernelUnavailable("no GPU is visible: this engine runs on HIP only")
    load_start = time.perf_counter()
    engine = create_engine(opt.model, dtype=opt.dtype, kv_dtype=opt.kv_dtype, kv_mem=opt.kv_bytes,
                           kv_blocks=opt.kv_blocks, block_size=opt.block_size, max_seqs=opt.max_seqs,
                           max_tokens_per_step=opt.max_tokens_per_step, prefill_chunk=opt.prefill_chunk,
                           policy=opt.policy, aging=opt.aging, admit_whole=opt.admit_whole, stop_tokens=opt.stop_ids)
    load_seconds = time.perf_counter() - load_start

    gen_start = time.perf_counter()
    times = []

    def on_token(seq_id: int, token: int) -> None:
        times.append(time.perf_counter() - gen_start)
        sys.stdout.write(("" if len(times) == 1 else " ") + str(token))
        sys.stdout.flush()

    engine.on_token = on_token
    seq_id = engine.add_request(opt.prompt, opt.sampling)
    try:
        while engine.sequence(seq_id).state != SeqState.FINISHED:
            engine.step()
    finally:
        sys.stdout.write("\n")
        sys.stdout.flush()
    effective = engine.sequence(seq_id).params.max_tokens
    engine.release(seq_id)

    generated = len(times)
    ttft = times[0] if times else 0.0
    prefill_rate = len(opt.prompt) / ttft if ttft > 0 else 0.0
    decode_rate = (generated - 1) / (times[-1] - ttft) if generated > 1 and times[-1] > ttft else 0.0
    cache = engine.cache
    total = len(opt.prompt) + generated
    print(f"\n[tie] hip | load {load_seconds:.2f} s | prompt {len(opt.prompt)} tok | ttft {ttft * 1e3:.0f} ms | "
          f"prefill {prefill_rate:.1f} tok/s | decode {decode_rate:.1f} tok/s | {generated} tok generated | "
          f"kv {cache.blocks_for(total)} blocks for {total} tok, pool {cache.num_blocks} blocks "
          f"({cache.total_bytes() / 2 ** 30:.2f} GiB)", file=sys.stderr)
    if effective < opt.sampling.max_tokens:
        print(f"[tie] note: max_tokens clamped to {effective} by the KV cache / context", file=sys.stderr)
    return 0


def run_bench(argv: Sequence[str]) -> int:
    opt = parse_bench_args(argv)
    import torch

    from ..api import create_engine
    from ..bench import (assign_arrivals, format_report, read_requests_jsonl, report_json, run_workload, summarize,
                         synthetic_requests)
    from ..errors import KernelUnavailable

    if not torch.cuda.is_available():
        raise KernelUnavailable("no GPU is visible: this engine runs on HIP only")
    engine = create_engine(opt.model, dtype=opt.dtype, kv_dtype=opt.kv_dtype, kv_mem=opt.kv_bytes,
                           kv_blocks=opt.kv_blocks, block_size=opt.block_size, max_seqs=opt.max_seqs,
                           max_tokens_per_step=opt.max_tokens_per_step, prefill_chunk=opt.prefill_chunk,
                           policy=opt.policy, aging=opt.aging, admit_whole=opt.admit_whole, launch_ahead=opt.launch_ahead)
    vocab = engine.model.spec.vocab_size
    if opt.synthetic:
        requests = synthetic_requests(opt.synthetic, opt.prompt_len, opt.output_len, vocab, opt.sampling.seed)
    else:
        requests = read_requests_jsonl(opt.prompts, opt.max_tokens, vocab)
    assign_arrivals(requests, opt.rate, opt.sampling.seed)
    run = run_workload(engine, requests, opt.sampling,
                       progress=lambda line: print(f"[tie] {line}", file=sys.stderr, flush=True))
    report = summarize(run)
    if opt.json:
        print(json.dumps(report_json(report)))
    else:
        sys.stdout.write(format_report(report))
    return 0


def run_random_weights(argv: Sequence[str]) -> int:
    from ..config.base import read_config_json
    from ..weights.random_init import write_random_model

    config = out = None
    seed, dtype = 0, "bfloat16"
    i = 0
    while i < len(argv):
        flag = argv[i]
        if i + 1 >= len(argv):
            raise InvalidArgument(f"{flag} needs a value")
        val = argv[i + 1]
        if flag == "--config":
            config = val
        elif flag == "--out":
            out = val
        elif flag == "--seed":
            seed = parse_int(flag, val)
        elif flag == "--dtype":
            dtype = val
        else:
            raise InvalidArgument(f"unknown option '{flag}'")
        i += 2
    if not config or not out:
        raise InvalidArgument("--config and --out are required")
    folder = write_random_model(out, read_config_json(config), seed, dtype)
    print(folder)
    return 0


def main(argv: Sequence[str] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help"):
        (sys.stderr if not argv else sys.stdout).write(USAGE)
        return 1 if not argv else 0
    try:
        if argv[0] == "generate":
            return run_generate(argv[1:])
        if argv[0] == "bench":
            return run_bench(argv[1:])
        if argv[0] == "random-weights":
            return run_random_weights(argv[1:])
        raise InvalidArgument(f"unknown command '{argv[0]}'")
    except TieError as e:
        print(f"tie: error: {e}", file=sys.stderr)
        return 1
    except Exception as e:  # noqa: BLE001
        print(f"tie: internal error: {e}", file=sys.stderr)
        return 2
