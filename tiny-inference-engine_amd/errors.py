"""Error taxonomy of the engine.

Four kinds, after the reference's ``src/core/error.h:12-44``: a malformed file,
a well-formed request for something the engine does not handle, a limit that
was exceeded, and an argument that can never be valid. Every message names the
offending value.
"""


class TieError(Exception):
    """Base of every error the engine raises on purpose."""


class LoadError(TieError):
    """A model folder, config.json or safetensors file is malformed or does not fit the model."""


class UnsupportedError(TieError):
    """The input is well formed but asks for something this engine does not run."""


class CapacityError(TieError):
    """A limit (pages, tokens per step, context length, state slots) was exceeded."""


class InvalidArgument(TieError):
    """An argument that no configuration of the engine could accept."""


class KernelUnavailable(TieError):
    """The HIP extension is missing, cannot be built, or no GPU is present."""
