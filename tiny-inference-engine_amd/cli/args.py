"""Command-line options of ``tie generate`` and ``tie bench`` in the reference's manner (``src/cli/args.cpp``).

Flags are ``--flag value`` pairs with strict numbers; an unknown flag, a missing value or a
malformed number is an InvalidArgument. Names, meanings and defaults are the reference's where
it has them: ``-m/--model``, ``-p/--prompt``, ``--temp`` (0.7), ``--top-k`` (20), ``--top-p``
(0.8), ``--seed`` (0), ``--kv-mem`` (4G), ``--max-tokens`` (256), ``--device``. This engine has no
tokenizer, so the prompt is a list of token ids and stop tokens are given as ids; ``--chat`` and
``--no-think`` are refused. Options the reference's ``bench`` command names for the serving shape
(``--max-seqs``, ``--max-tokens-per-step``, ``--policy``, ``--aging``) are accepted by ``generate`` as well.

``tie bench`` takes the reference's bench options (``args.cpp:169-215``): ``--synthetic N``,
``--prompt-len A:B`` (512:1024), ``--output-len C:D`` (128), ``--max-tokens`` (128, for workload lines
without one), ``--rate`` (inf), ``--json``, greedy unless ``--temp`` is given; ``--prompts FILE`` reads
token ids (``{"prompt_ids": [...]}`` a line), since prompt text would need a tokenizer.
"""

from __future__ import annotations

import dataclasses
import math
import re
from typing import List, Optional, Sequence, Tuple

from ..errors import InvalidArgument
from ..sampling.params import SamplingParams

USAGE = """usage: tie generate -m <model_dir> -p <token ids> [options]
       tie bench -m <model_dir> (--prompts FILE.jsonl | --synthetic N) [options]
       tie random-weights --config <config.json> --out <model_dir> [--seed S] [--dtype bfloat16|float32]

generate options:
  -m, --model PATH         HuggingFace model directory (config.json + safetensors)
  -p, --prompt IDS         prompt token ids, separated by commas or spaces
  --prompt-file FILE       read the prompt token ids from FILE instead
  --device hip             compute device (default hip; there is no CPU path)
  --dtype D                bfloat16 (default) or float32
  --kv-dtype D             precision of the cached keys and values: that of --dtype by default; float32
                           arithmetic also runs over bfloat16 or float16 pages
  --temp T                 sampling temperature, 0 = greedy (default 0.7)
  --top-k K                keep the K most likely tokens, 0 = off (default 20)
  --top-p P                nucleus sampling threshold (default 0.8)
  --seed S                 sampling seed (default 0)
  --max-tokens N           tokens to generate (default 256)
  --stop-ids IDS           token ids that end generation (the stop token is kept)
  --kv-mem SIZE            KV cache budget, e.g. 4G or 512M (default 4G)
  --kv-blocks N            KV cache size in pages instead of bytes
  --block-size N           tokens per KV page (default 16)
  --max-seqs S             sequences per step (default 64)
  --max-tokens-per-step B  tokens per step (default 512)
  --prefill-chunk C        most prompt tokens of one sequence per step, 0 = budget only (default 0)
  --policy fcfs|srpt-aging admission order (default srpt-aging)
  --aging N                srpt-aging priority gained per step waited, in tokens (default 16)
  --admit-whole            a request enters when the cache can hold all of its pending input, not just its first
                           portion (not in the reference: fewer evictions when the cache is scarce)

bench options (and -m, --device, --dtype, --kv-dtype, --temp (default 0), --top-k, --top-p, --seed, --kv-mem, --kv-blocks,
--block-size, --max-seqs, --max-tokens-per-step, --prefill-chunk, --policy, --aging, --admit-whole as above; --seed also seeds
the synthetic workload and the arrivals):
  --prompts FILE           JSONL, one {"prompt_ids": [...], "max_tokens": N} per line
  --synthetic N            N requests of random tokens
  --prompt-len A:B         synthetic prompt lengths (default 512:1024)
  --output-len C:D         synthetic output lengths (default 128)
  --max-tokens N           output tokens for JSONL lines without max_tokens (default 128)
  --rate R                 requests per second, Poisson arrivals; inf = all at once (default inf)
  --json                   print the report as one JSON object
  --no-launch-ahead        read every step's tokens before the next step is queued: token times are then the
                           moments the tokens exist (by default a decode step is queued before the one before
                           it is read, which is faster and shows every token one step late)
"""


@dataclasses.dataclass
class GenerateOptions:
    model: str = ""
    prompt: List[int] = dataclasses.field(default_factory=list)
    device: str = "hip"
    dtype: str = "bfloat16"
    kv_dtype: Optional[str] = None
    sampling: SamplingParams = dataclasses.field(
        default_factory=lambda: SamplingParams(temperature=0.7, top_k=20, top_p=0.8))
    stop_ids: List[int] = dataclasses.field(default_factory=list)
    kv_bytes: int = 4 << 30
    kv_blocks: Optional[int] = None
    block_size: int = 16
    max_seqs: int = 64
    max_tokens_per_step: int = 512
    prefill_chunk: int = 0
    policy: str = "srpt-aging"
    aging: int = 16
    admit_whole: bool = False


def parse_int(flag: str, text: str) -> int:
    if not re.fullmatch(r"-?\d+", text):
        raise InvalidArgument(f"{flag} expects an integer, got '{text}'")
    return int(text)


def parse_float(flag: str, text: str) -> float:
    try:
        if text != text.strip():
            raise ValueError
        value = float(text)
    except ValueError:
        value = math.nan
    if not math.isfinite(value):
        raise InvalidArgument(f"{flag} expects a finite number, got '{text}'")
    return value


def parse_size(text: str) -> int:
    """"4G", "512M", "64K" or a plain byte count; must be positive (src/cli/args.cpp:105-126)."""
    shift = {"K": 10, "M": 20, "G": 30}.get(text[-1:].upper(), 0)
    digits = text[:-1] if shift else text
    if not digits or not digits.isdigit():
        raise InvalidArgument(f"size '{text}' must be a whole number with an optional K, M or G suffix")
    value = int(digits) << shift
    if value >= 2 ** 64:
        raise InvalidArgument(f"size '{text}' is too large")
    if value == 0:
        raise InvalidArgument(f"size '{text}' must be positive")
    return value


def parse_ids(flag: str, text: str) -> List[int]:
    parts = [p for p in re.split(r"[,\s]+", text.strip()) if p]
    if not parts:
        raise InvalidArgument(f"{flag} expects token ids, got '{text}'")
    return [parse_int(flag, p) for p in parts]


class _Flags:
    """Walks ``--flag value`` pairs."""

    def __init__(self, args: Sequence[str]):
        self.args = list(args)
        self.i = 0
        self.flag = ""

    def __iter__(self):
        while self.i < len(self.args):
            self.flag = self.args[self.i]
            yield self.flag
            self.i += 1

    def value(self) -> str:
        if self.i + 1 >= len(self.args):
            raise InvalidArgument(f"{self.flag} needs a value")
        self.i += 1
        return self.args[self.i]


def _engine_flag(flag: str, flags: _Flags, o) -> bool:
    """Options both commands share: the model, the precision, sampling, the cache and the serving shape."""
    if flag in ("-m", "--model"):
        o.model = flags.value()
    elif flag == "--device":
        o.device = flags.value()
        if o.device not in ("hip", "gpu", "cuda"):
            raise InvalidArgument(f"--device must be hip, got '{o.device}' (this engine has no CPU path)")
    elif flag == "--dtype":
        o.dtype = flags.value()
        if o.dtype not in ("bfloat16", "float32", "bf16", "fp32"):
            raise InvalidArgument(f"--dtype must be bfloat16 or float32, got '{o.dtype}'")
    elif flag == "--kv-dtype":
        o.kv_dtype = flags.value()
        if o.kv_dtype not in ("float32", "fp32", "bfloat16", "bf16", "float16", "fp16"):
            raise InvalidArgument(f"--kv-dtype must be float32, bfloat16 or float16, got '{o.kv_dtype}'")
    elif flag == "--temp":
        o.sampling.temperature = parse_float(flag, flags.value())
    elif flag == "--top-k":
        o.sampling.top_k = parse_int(flag, flags.value())
    elif flag == "--top-p":
        o.sampling.top_p = parse_float(flag, flags.value())
    elif flag == "--seed":
        o.sampling.seed = parse_int(flag, flags.value())
    elif flag == "--kv-mem":
        try:
            o.kv_bytes = parse_size(flags.value())
        except InvalidArgument as e:
            raise InvalidArgument(f"{flag}: {e}") from None
    elif flag == "--kv-blocks":
        o.kv_blocks = parse_int(flag, flags.value())
    elif flag == "--block-size":
        o.block_size = parse_int(flag, flags.value())
    elif flag == "--max-seqs":
        o.max_seqs = parse_int(flag, flags.value())
    elif flag == "--max-tokens-per-step":
        o.max_tokens_per_step = parse_int(flag, flags.value())
    elif flag == "--prefill-chunk":
        o.prefill_chunk = parse_int(flag, flags.value())
    elif flag == "--policy":
        from ..engine.scheduler import parse_policy
        o.policy = parse_policy(flags.value())
    elif flag == "--aging":
        o.aging = parse_int(flag, flags.value())
        if o.aging < 0:
            raise InvalidArgument(f"--aging must be non-negative, got {o.aging}")
    elif flag == "--admit-whole":
        o.admit_whole = True
    elif flag == "--threads":
        parse_int(flag, flags.value())         # CPU threads of the reference's CPU backend: nothing to set here
    else:
        return False
    return True


def parse_generate_args(args: Sequence[str]) -> GenerateOptions:
    o = GenerateOptions()
    flags = _Flags(args)
    for flag in flags:
        if _engine_flag(flag, flags, o):
            continue
        if flag in ("-p", "--prompt"):
            o.prompt = parse_ids(flag, flags.value())
        elif flag == "--prompt-file":
            path = flags.value()
            try:
                with open(path) as f:
                    o.prompt = parse_ids(flag, f.read())
            except OSError as e:
                raise InvalidArgument(f"cannot read {path}: {e.strerror or e}") from None
        elif flag == "--max-tokens":
            o.sampling.max_tokens = parse_int(flag, flags.value())
        elif flag == "--stop-ids":
            o.stop_ids = parse_ids(flag, flags.value())
        elif flag in ("--chat", "--no-think"):
            raise InvalidArgument(f"{flag} needs a tokenizer, which this engine does not have: give token ids")
        else:
            raise InvalidArgument(f"unknown option '{flag}'")
    if not o.model:
        raise InvalidArgument("--model is required")
    if not o.prompt:
        raise InvalidArgument("--prompt is required")
    o.sampling.validate()
    return o


@dataclasses.dataclass
class BenchOptions:
    model: str = ""
    prompts: str = ""                      # JSONL workload of token ids; empty with --synthetic
    synthetic: int = 0                     # number of synthetic requests; 0 with --prompts
    prompt_len: Tuple[int, int] = (512, 1024)
    output_len: Tuple[int, int] = (128, 128)
    max_tokens: int = 128                  # for workload lines without max_tokens
    rate: float = math.inf
    device: str = "hip"
    dtype: str = "bfloat16"
    kv_dtype: Optional[str] = None
    launch_ahead: bool = True
    sampling: SamplingParams = dataclasses.field(default_factory=lambda: SamplingParams(temperature=0.0))
    kv_bytes: int = 4 << 30
    kv_blocks: Optional[int] = None
    block_size: int = 16
    max_seqs: int = 64
    max_tokens_per_step: int = 512
    prefill_chunk: int = 0
    policy: str = "srpt-aging"
    aging: int = 16
    admit_whole: bool = False
    json: bool = False


def parse_bench_args(args: Sequence[str]) -> BenchOptions:
    from ..bench.workload import parse_range
    from ..engine.serving import ServingConfig

    o = BenchOptions()
    flags = _Flags(args)
    for flag in flags:
        if _engine_flag(flag, flags, o):
            continue
        if flag == "--prompts":
            o.prompts = flags.value()
        elif flag == "--synthetic":
            o.synthetic = parse_int(flag, flags.value())
            if o.synthetic < 1:
                raise InvalidArgument(f"--synthetic needs at least 1 request, got {o.synthetic}")
        elif flag == "--prompt-len":
            o.prompt_len = parse_range(flag, flags.value())
        elif flag == "--output-len":
            o.output_len = parse_range(flag, flags.value())
        elif flag == "--max-tokens":
            o.max_tokens = parse_int(flag, flags.value())
            if o.max_tokens < 1:
                raise InvalidArgument(f"--max-tokens must be positive, got {o.max_tokens}")
        elif flag == "--rate":
            text = flags.value()
            o.rate = math.inf if text == "inf" else parse_float(flag, text)
            if not o.rate > 0:
                raise InvalidArgument(f"--rate must be positive or inf, got '{text}'")
        elif flag == "--json":
            o.json = True
        elif flag == "--no-launch-ahead":
            o.launch_ahead = False
        else:
            raise InvalidArgument(f"unknown option '{flag}'")
    if not o.model:
        raise InvalidArgument("--model is required")
    if bool(o.prompts) == bool(o.synthetic):
        raise InvalidArgument("give exactly one of --prompts or --synthetic")
    ServingConfig(o.max_tokens_per_step, o.max_seqs, o.prefill_chunk).validate()
    o.sampling.validate()
    return o
