"""A small, whole inference engine for one GPU (AMD MI355X, gfx950).

Everything between a request's token ids and its next token id: a typed
configuration and a registry of architectures, a strict weight loader, parts
(mixer, feed-forward, norm, position encoding, block) put together by
description, a paged cache manager, one step function for mixed batches, a
continuous-batching scheduler, sampling, and hand-written HIP kernels.
"""

from .errors import (CapacityError, InvalidArgument, KernelUnavailable, LoadError, TieError,
                     UnsupportedError)

__all__ = ["CapacityError", "InvalidArgument", "KernelUnavailable", "LoadError", "TieError", "UnsupportedError"]

from .sampling.params import SamplingParams  # noqa: E402
from .api import create_engine, generate  # noqa: E402
from .engine.engine import Engine  # noqa: E402
from .models.builder import load_model  # noqa: E402
from .weights.random_init import write_random_model  # noqa: E402

__all__ += ["Engine", "SamplingParams", "create_engine", "generate", "load_model", "write_random_model"]
