"""What a mixer needs from the cache, and how a model's needs are grouped.

A mixer declares one need (or none): paged keys and values, all of them or a
window of them, or a state of fixed size per request. Run-order entries with
equal needs share a *group*: one page pool, one block table per request and one
tensor whose leading dimension counts the entries (planes) of the group. The
reference has a single group - every layer is full attention with the same head
geometry (``src/kv/paged_kv_cache.h:27-30``) - and no fixed-size state at all.
"""

from __future__ import annotations

import dataclasses
import functools
from typing import List, Optional, Sequence, Tuple, Union

from ..errors import InvalidArgument


@dataclasses.dataclass(frozen=True)
class PagedKV:
    """Keys and values of every cached position, in pages.

    ``window`` = None keeps all positions; ``window`` = w means a query at
    position p reads keys p-w+1 .. p, so pages wholly before that range can be
    given back while the request still runs.
    """

    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None

    def __post_init__(self):
        if self.num_kv_heads <= 0 or self.head_dim <= 0:
            raise InvalidArgument("a paged cache needs positive num_kv_heads and head_dim")
        if self.window is not None and self.window <= 0:
            raise InvalidArgument(f"an attention window must be positive, got {self.window}")


@dataclasses.dataclass(frozen=True)
class FixedState:
    """A state of fixed shape per request (per run-order entry), kept in a slot."""

    shape: Tuple[int, ...]
    dtype: str = "float32"

    def __post_init__(self):
        if any(d <= 0 for d in self.shape):
            raise InvalidArgument(f"a state needs positive dimensions, got {self.shape}")


CacheNeed = Union[PagedKV, FixedState]


@dataclasses.dataclass(frozen=True)
class CacheGroup:
    need: CacheNeed
    num_planes: int


@dataclasses.dataclass(frozen=True)
class CallCache:
    """Where one run-order entry finds its cache: a plane of a group, written or only read."""

    group: int
    plane: int
    writes: bool


@dataclasses.dataclass(frozen=True)
class CachePlan:
    groups: Tuple[CacheGroup, ...]
    calls: Tuple[Optional[CallCache], ...]

    @functools.cached_property
    def paged_groups(self) -> List[int]:
        return [i for i, g in enumerate(self.groups) if isinstance(g.need, PagedKV)]

    @functools.cached_property
    def state_groups(self) -> List[int]:
        return [i for i, g in enumerate(self.groups) if isinstance(g.need, FixedState)]


def plan_cache(needs: Sequence[Optional[CacheNeed]], reads_cache_of: Sequence[Optional[int]]) -> CachePlan:
    """Groups the needs of the run-order entries.

    ``needs[i]`` is what entry i's mixer needs (None for a mixer without cache);
    ``reads_cache_of[i]`` is an earlier entry whose plane entry i reads instead
    of owning one, and whose need must equal its own.
    """
    if len(needs) != len(reads_cache_of):
        raise InvalidArgument("plan_cache: one need and one sharing entry per run-order entry")
    group_of = {}
    planes: List[int] = []
    calls: List[Optional[CallCache]] = []
    for i, need in enumerate(needs):
        src = reads_cache_of[i]
        if need is None:
            if src is not None:
                raise InvalidArgument(f"run order entry {i} reads a cache but its mixer needs none")
            calls.append(None)
            continue
        if src is not None:
            owner = calls[src] if 0 <= src < i else None
            if owner is None or not owner.writes:
                raise InvalidArgument(f"run order entry {i} reads the cache of entry {src}, which owns none")
            if needs[src] != need:
                raise InvalidArgument(
                    f"run order entry {i} needs {need} but reads the cache of entry {src}, which holds {needs[src]}")
            calls.append(CallCache(owner.group, owner.plane, False))
            continue
        if need not in group_of:
            group_of[need] = len(planes)
            planes.append(0)
        g = group_of[need]
        calls.append(CallCache(g, planes[g], True))
        planes[g] += 1
    ordered = sorted(group_of.items(), key=lambda kv: kv[1])
    groups = tuple(CacheGroup(need, planes[g]) for need, g in ordered)
    return CachePlan(groups, tuple(calls))
