"""The Python entry point: an engine from a model folder, and one-call generation.

The reference's programmatic interface is its C++ ``Engine`` (``src/engine/engine.h:35-63``:
``add_request``, ``step``, ``has_work``, ``sequence``, ``cancel``, ``release``, ``generate``,
``set_token_callback``, ``stats``); ``create_engine`` wires the same object the way the
reference's command line does (``src/cli/main.cpp:56-68``): weights, a page pool sized by a
memory budget, a scheduler and the engine over them.
"""

from __future__ import annotations

from typing import List, Optional, Sequence

from . import kernels
from .cache.manager import CacheManager
from .engine.engine import Engine
from .engine.scheduler import BatchScheduler, SchedulerConfig
from .engine.serving import ServingConfig
from .models.builder import Model, load_model
from .sampling.params import SamplingParams
from .weights.binder import normalize_mode

DEFAULT_KV_BYTES = 4 << 30  # the reference's default KV budget (src/cli/args.h:24)


def create_engine(model, dtype: str = "bfloat16", kv_mem: Optional[int] = None, kv_blocks: Optional[int] = None,
                  block_size: int = 16, max_seqs: int = 64, max_tokens_per_step: int = 512, prefill_chunk: int = 0,
                  policy: str = "srpt-aging", aging: int = 16, watermark_blocks: int = -1, admit_whole: bool = False,
                  stop_tokens: Sequence[int] = (), max_seq_len: Optional[int] = None,
                  device: str = "cuda:0", use_graphs: Optional[bool] = None, launch_ahead=True,
                  kv_dtype: Optional[str] = None) -> Engine:
    """``model`` is a folder (config.json + safetensors) or a Model that is already loaded.

    ``use_graphs`` False runs every step eagerly; None (the default) records decode-only steps into HIP
    graphs in bfloat16 mode when every part of the model allows it. ``launch_ahead``: steps are queued before
    the tokens of the steps before them are read (``Engine``'s module text says how): True leaves one step
    unread, a number that many, False none; tokens then appear that many ``step()`` calls later. ``kv_dtype``: the precision of the cached keys and values, by
    default that of ``dtype``; float32 arithmetic also runs over a bfloat16 or float16 cache (the reference's
    arrangement, ``src/kv/paged_kv_cache.h:18-25``). A pair no kernel takes is refused here, before anything
    is loaded."""
    mode = model.mode if isinstance(model, Model) else normalize_mode(dtype)
    cache_dtype = kernels.cache_dtype_for(mode, kv_dtype)
    if not isinstance(model, Model):
        model = load_model(model, mode, device)
    if kv_blocks is None and kv_mem is None:
        kv_mem = DEFAULT_KV_BYTES
    context = min(model.spec.max_positions, max_seq_len) if max_seq_len else model.spec.max_positions
    cache = CacheManager(model.cache_plan, block_size=block_size, num_blocks=kv_blocks,
                         budget_bytes=None if kv_blocks is not None else kv_mem, dtype=cache_dtype,
                         device=model.device, max_state_slots=max_seqs, context_hint=context,
                         step_tokens=prefill_chunk or max_tokens_per_step)
    serving = ServingConfig(max_tokens_per_step=max_tokens_per_step, max_seqs=max_seqs, prefill_chunk=prefill_chunk)
    scheduler = BatchScheduler(cache, SchedulerConfig(serving=serving, policy=policy, aging=aging,
                                                      watermark_blocks=watermark_blocks, admit_whole=admit_whole))
    return Engine(model, cache, scheduler, serving, stop_tokens=stop_tokens, max_seq_len=max_seq_len,
                  use_graphs=use_graphs, launch_ahead=launch_ahead)


def generate(model, prompt: Sequence[int], params: Optional[SamplingParams] = None, **engine_options) -> List[int]:
    """Loads ``model``, runs one request to completion and returns the generated token ids."""
    return create_engine(model, **engine_options).generate(prompt, params)
