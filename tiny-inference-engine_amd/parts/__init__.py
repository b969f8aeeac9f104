"""The parts models are put together from. Importing the package registers the built-in kinds."""

from .base import (Block, Embedding, FeedForward, Head, Mixer, Norm, PagedBinding, Part, PartSpec, Position,
                   StateBinding,
                   StepContext, TensorSpec, Workspace, build_part, register_part, registered_parts,
                   unregister_part)
from . import attention, block, embedding, feedforward, head, norm, position  # noqa: F401  (registration)
