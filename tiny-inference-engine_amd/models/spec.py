"""The architecture-neutral description of a model: which parts, in which order.

An architecture's spec builder turns its typed configuration into a ModelSpec;
everything below the builder (weight loading, cache sizing, the step function,
random initialisation) reads only the spec. A part is named by the key under
which its class is registered and carries its sizes and constants as
parameters, so one model can mix different mixers and feed-forwards layer by
layer. The order in which layers run is data as well: ``order`` may name a
layer twice, and a call may read the cache another call writes.
"""

from __future__ import annotations

import dataclasses
from typing import Mapping, Optional, Tuple

from ..parts.base import PartSpec


@dataclasses.dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (block) of a mixer, a feed-forward and their norms.

    Either part may be None: a layer of a mixer alone or of a feed-forward alone, for architectures that
    interleave them otherwise than in pairs, or whose layers would need two mixers with caches of their own
    (two entries of the run order, the second without a feed-forward). The arrangement says what it needs.
    """

    block: PartSpec
    mixer: Optional[PartSpec]
    feed_forward: Optional[PartSpec]
    norms: Mapping[str, PartSpec] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelSpec.layers``. ``cache`` names the cache slot the
    call's mixer uses; by default every call owns a slot of its own (its index
    in the order). A call with ``reads_cache_of`` set to an earlier position in
    the order uses that call's slot read-only: it writes no keys or values.
    """

    layer: int
    reads_cache_of: Optional[int] = None


@dataclasses.dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[LayerCall, ...]
    head: PartSpec

    def validate(self) -> None:
        from ..errors import InvalidArgument

        if not self.layers or not self.order:
            raise InvalidArgument("a model needs at least one layer and one entry in its run order")
        for position, call in enumerate(self.order):
            if not 0 <= call.layer < len(self.layers):
                raise InvalidArgument(f"run order entry {position} names layer {call.layer}; there are {len(self.layers)}")
            if call.reads_cache_of is not None:
                src = call.reads_cache_of
                if not 0 <= src < position:
                    raise InvalidArgument(
                        f"run order entry {position} reads the cache of entry {src}, which does not run before it")
                if self.order[src].reads_cache_of is not None:
                    raise InvalidArgument(
                        f"run order entry {position} reads the cache of entry {src}, which owns no cache itself")
