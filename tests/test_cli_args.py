"""Command-line parsing (no GPU). Scenarios of the reference's tests/cli/test_args.cpp."""

import subprocess
import sys

import pytest

from conftest import ROOT
from tie_amd.cli.args import parse_bench_args, parse_generate_args, parse_size
from tie_amd.errors import InvalidArgument


def test_defaults_are_the_references():
    o = parse_generate_args(["-m", "dir", "-p", "1,2, 3 4"])
    assert o.model == "dir" and o.prompt == [1, 2, 3, 4]
    assert (o.sampling.temperature, o.sampling.top_k, o.sampling.top_p, o.sampling.seed, o.sampling.max_tokens) == \
        (0.7, 20, 0.8, 0, 256)
    assert o.kv_bytes == 4 << 30 and o.max_seqs == 64 and o.max_tokens_per_step == 512 and o.policy == "srpt-aging"


def test_every_option_is_read():
    o = parse_generate_args(["--model", "m", "--prompt", "7", "--temp", "0", "--top-k", "5", "--top-p", "0.5",
                             "--seed", "9", "--max-tokens", "12", "--kv-mem", "512M", "--stop-ids", "2,3",
                             "--dtype", "float32", "--block-size", "4", "--kv-blocks", "40", "--max-seqs", "8",
                             "--max-tokens-per-step", "64", "--prefill-chunk", "13", "--policy", "fcfs",
                             "--aging", "2", "--device", "hip", "--threads", "4", "--kv-dtype", "float16", "--admit-whole"])
    assert o.kv_dtype == "float16" and parse_generate_args(["-m", "m", "-p", "7"]).kv_dtype is None
    assert o.admit_whole and not parse_generate_args(["-m", "m", "-p", "7"]).admit_whole
    assert o.sampling.temperature == 0.0 and o.sampling.top_k == 5 and o.sampling.top_p == 0.5
    assert o.sampling.seed == 9 and o.sampling.max_tokens == 12 and o.kv_bytes == 512 << 20
    assert o.stop_ids == [2, 3] and o.dtype == "float32" and o.block_size == 4 and o.kv_blocks == 40
    assert (o.max_seqs, o.max_tokens_per_step, o.prefill_chunk, o.policy, o.aging) == (8, 64, 13, "fcfs", 2)


@pytest.mark.parametrize("argv,match", [
    (["-p", "1"], "--model is required"), (["-m", "x"], "--prompt is required"),
    (["-m", "x", "-p", "1", "--bogus"], "unknown option '--bogus'"), (["-m", "x", "-p"], "needs a value"),
    (["-m", "x", "-p", "1", "--temp", "hot"], "finite number"), (["-m", "x", "-p", "1", "--temp", "inf"], "finite number"),
    (["-m", "x", "-p", "1", "--top-k", "2.5"], "integer"), (["-m", "x", "-p", "1", "--top-p", "0"], "top_p"),
    (["-m", "x", "-p", "1", "--max-tokens", "0"], "max_tokens"), (["-m", "x", "-p", "a,b"], "integer"),
    (["-m", "x", "-p", "1", "--kv-mem", "4T"], "--kv-mem"), (["-m", "x", "-p", "1", "--device", "cpu"], "no CPU path"),
    (["-m", "x", "-p", "1", "--chat"], "tokenizer"), (["-m", "x", "-p", "1", "--policy", "lifo"], "lifo"),
    (["-m", "x", "-p", "1", "--kv-dtype", "int8"], "--kv-dtype must be"),
])
def test_bad_arguments_are_refused(argv, match):
    with pytest.raises(InvalidArgument, match=match):
        parse_generate_args(argv)


def test_sizes():
    assert parse_size("4G") == 4 << 30 and parse_size("512m") == 512 << 20 and parse_size("64K") == 65536
    assert parse_size("1000") == 1000
    for bad in ("", "G", "0", "4GB", "-1", "1.5G", "99999999999999999999G"):
        with pytest.raises(InvalidArgument):
            parse_size(bad)


def test_exit_codes_of_the_program():
    run = lambda *a: subprocess.run([sys.executable, str(ROOT / "bin" / "tie"), *a], capture_output=True, text=True)
    r = run()
    assert r.returncode == 1 and "usage: tie generate" in r.stderr
    r = run("--help")
    assert r.returncode == 0 and "usage: tie generate" in r.stdout
    r = run("serve")
    assert r.returncode == 1 and "tie: error: unknown command 'serve'" in r.stderr
    r = run("bench", "-m", "x")
    assert r.returncode == 1 and "tie: error: give exactly one of --prompts or --synthetic" in r.stderr
    r = run("generate", "-m", "/nonexistent", "-p", "1", "--temp", "x")
    assert r.returncode == 1 and "tie: error: --temp expects a finite number" in r.stderr


def test_bench_defaults_and_options():
    """The reference's bench options (src/cli/args.cpp:169-215; tests/cli/test_args.cpp for the scenarios)."""
    import math

    o = parse_bench_args(["-m", "dir", "--synthetic", "8"])
    assert o.synthetic == 8 and o.prompt_len == (512, 1024) and o.output_len == (128, 128) and o.max_tokens == 128
    assert math.isinf(o.rate) and o.sampling.temperature == 0.0 and not o.json
    assert (o.max_seqs, o.max_tokens_per_step, o.policy, o.aging, o.kv_bytes) == (64, 512, "srpt-aging", 16, 4 << 30)
    o = parse_bench_args(["-m", "d", "--prompts", "w.jsonl", "--prompt-len", "3:9", "--output-len", "7", "--rate", "2.5",
                          "--max-tokens", "5", "--json", "--temp", "0.5", "--seed", "4", "--kv-mem", "2G",
                          "--prefill-chunk", "512", "--max-seqs", "16", "--policy", "fcfs"])
    assert o.prompts == "w.jsonl" and o.prompt_len == (3, 9) and o.output_len == (7, 7) and o.rate == 2.5
    assert o.max_tokens == 5 and o.json and o.sampling.temperature == 0.5 and o.sampling.seed == 4
    assert o.kv_bytes == 2 << 30 and o.prefill_chunk == 512 and o.max_seqs == 16 and o.policy == "fcfs"
    assert o.launch_ahead and o.kv_dtype is None
    o = parse_bench_args(["-m", "d", "--synthetic", "2", "--no-launch-ahead", "--kv-dtype", "bf16"])
    assert not o.launch_ahead and o.kv_dtype == "bf16"


@pytest.mark.parametrize("argv,match", [
    (["--synthetic", "4"], "--model is required"), (["-m", "x"], "exactly one of"),
    (["-m", "x", "--synthetic", "4", "--prompts", "f"], "exactly one of"), (["-m", "x", "--synthetic", "0"], "at least 1"),
    (["-m", "x", "--synthetic", "4", "--prompt-len", "9:3"], "1 <= A <= B"),
    (["-m", "x", "--synthetic", "4", "--output-len", "0"], "1 <= A <= B"),
    (["-m", "x", "--synthetic", "4", "--rate", "0"], "positive or inf"),
    (["-m", "x", "--synthetic", "4", "--max-tokens", "0"], "positive"),
    (["-m", "x", "--synthetic", "4", "--max-seqs", "1000"], "max_seqs"),
    (["-m", "x", "--synthetic", "4", "-p", "1"], "unknown option"),
])
def test_bad_bench_arguments_are_refused(argv, match):
    with pytest.raises(InvalidArgument, match=match):
        parse_bench_args(argv)
