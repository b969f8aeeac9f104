"""Command-line options of ``tie generate`` in the reference's manner (``src/cli/args.cpp``).

Flags are ``--flag value`` pairs with strict numbers; an unknown flag, a missing value or a
malformed number is an InvalidArgument. Names, meanings and defaults are the reference's where
it has them: ``-m/--model``, ``-p/--prompt``, ``--temp`` (0.7), ``--top-k`` (20), ``--top-p``
(0.8), ``--seed`` (0), ``--kv-mem`` (4G), ``--max-tokens`` (256), ``--device``. This engine has no
tokenizer, so the prompt is a list of token ids and stop tokens are given as ids; ``--chat`` and
``--no-think`` are refused. Options the reference's ``bench`` command names for the serving shape
(``--max-seqs``, ``--max-tokens-per-step``, ``--policy``, ``--aging``) are accepted here as well.
"""

from __future__ import annotations

import dataclasses
import math
import re
from typing import List, Optional, Sequence

from ..errors import InvalidArgument
from ..sampling.params import SamplingParams

USAGE = """usage: tie generate -m <model_dir> -p <token ids> [options]
       tie random-weights --config <config.json> --out <model_dir> [--seed S] [--dtype bfloat16|float32]

generate options:
  -m, --model PATH         HuggingFace model directory (config.json + safetensors)
  -p, --prompt IDS         prompt token ids, separated by commas or spaces
  --prompt-file FILE       read the prompt token ids from FILE instead
  --device hip             compute device (default hip; there is no CPU path)
  --dtype D                bfloat16 (default) or float32
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
"""


@dataclasses.dataclass
class GenerateOptions:
    model: str = ""
    prompt: List[int] = dataclasses.field(default_factory=list)
    device: str = "hip"
    dtype: str = "bfloat16"
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


def parse_generate_args(args: Sequence[str]) -> GenerateOptions:
    o = GenerateOptions()
    i = 0

    def value() -> str:
        nonlocal i
        if i + 1 >= len(args):
            raise InvalidArgument(f"{flag} needs a value")
        i += 1
        return args[i]

    while i < len(args):
        flag = args[i]
        if flag in ("-m", "--model"):
            o.model = value()
        elif flag in ("-p", "--prompt"):
            o.prompt = parse_ids(flag, value())
        elif flag == "--prompt-file":
            path = value()
            try:
                with open(path) as f:
                    o.prompt = parse_ids(flag, f.read())
            except OSError as e:
                raise InvalidArgument(f"cannot read {path}: {e.strerror or e}") from None
        elif flag == "--device":
            o.device = value()
            if o.device not in ("hip", "gpu", "cuda"):
                raise InvalidArgument(f"--device must be hip, got '{o.device}' (this engine has no CPU path)")
        elif flag == "--dtype":
            o.dtype = value()
            if o.dtype not in ("bfloat16", "float32", "bf16", "fp32"):
                raise InvalidArgument(f"--dtype must be bfloat16 or float32, got '{o.dtype}'")
        elif flag == "--temp":
            o.sampling.temperature = parse_float(flag, value())
        elif flag == "--top-k":
            o.sampling.top_k = parse_int(flag, value())
        elif flag == "--top-p":
            o.sampling.top_p = parse_float(flag, value())
        elif flag == "--seed":
            o.sampling.seed = parse_int(flag, value())
        elif flag == "--max-tokens":
            o.sampling.max_tokens = parse_int(flag, value())
        elif flag == "--stop-ids":
            o.stop_ids = parse_ids(flag, value())
        elif flag == "--kv-mem":
            try:
                o.kv_bytes = parse_size(value())
            except InvalidArgument as e:
                raise InvalidArgument(f"{flag}: {e}") from None
        elif flag == "--kv-blocks":
            o.kv_blocks = parse_int(flag, value())
        elif flag == "--block-size":
            o.block_size = parse_int(flag, value())
        elif flag == "--max-seqs":
            o.max_seqs = parse_int(flag, value())
        elif flag == "--max-tokens-per-step":
            o.max_tokens_per_step = parse_int(flag, value())
        elif flag == "--prefill-chunk":
            o.prefill_chunk = parse_int(flag, value())
        elif flag == "--policy":
            from ..engine.scheduler import parse_policy
            o.policy = parse_policy(value())
        elif flag == "--aging":
            o.aging = parse_int(flag, value())
            if o.aging < 0:
                raise InvalidArgument(f"--aging must be non-negative, got {o.aging}")
        elif flag == "--threads":
            parse_int(flag, value())           # CPU threads of the reference's CPU backend: nothing to set here
        elif flag in ("--chat", "--no-think"):
            raise InvalidArgument(f"{flag} needs a tokenizer, which this engine does not have: give token ids")
        else:
            raise InvalidArgument(f"unknown option '{flag}'")
        i += 1
    if not o.model:
        raise InvalidArgument("--model is required")
    if not o.prompt:
        raise InvalidArgument("--prompt is required")
    o.sampling.validate()
    return o
