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
