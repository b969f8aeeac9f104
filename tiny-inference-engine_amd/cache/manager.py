"""The cache manager: pages of keys and values, block tables, state slots.

One page holds ``block_size`` consecutive positions of K and V for every plane
(run-order entry) and every KV head of its group, so one page id addresses the
same slots in all planes of the group - the reference's layout
(``src/kv/paged_kv_cache.h:27-30``, ``paged_kv_cache.cpp:91-99``) with a group
dimension added. Per group the device tensor is

    [planes][2 (K, V)][num_blocks][num_kv_heads][block_size * head_dim]

where a key page holds one row per position (``[block_size][head_dim]``) and a
value page is transposed (``[head_dim][block_size]``, one row per dimension):
the matrix cores consume keys along head_dim and values along positions, and
each gets its operand in contiguous 16-byte pieces this way.

A request holds one block table per paged group: position j lives in page
``table[j // block_size]`` at offset ``j % block_size``. Tables grow
all-or-nothing (``reserve``), shrink on a failed step (``truncate``), lose their
leading pages once a window has passed them (``trim``) and are given back whole
when the request ends or is preempted (``release``). Pages are never cleared:
attention reads only positions below the context length it is given.

Requests of models with fixed-size state also hold one state slot, an index
into ``[planes][max_state_slots][*shape]`` tensors; a slot is cleared when it is
assigned. A model without such state (Qwen3) has no state groups: the pool of
slots exists and hands out indices, but no memory stands behind them.
"""

from __future__ import annotations

import math
from typing import Dict, Iterable, List, Optional

import torch

from ..errors import CapacityError, InvalidArgument
from .block_pool import BlockPool
from .spec import CachePlan, FixedState, PagedKV

# What the kernels read and write; which of them goes with which compute mode is the kernels' to say
# (``kernels.cache_dtype_for``).
_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}
_INT32_MAX = 2 ** 31 - 1
FREED = -1  # table entry of a page that a window has passed and that was given back


class RequestCache:
    """What one request holds in the cache: a block table per group and a state slot."""

    __slots__ = ("tables", "trimmed", "state_slot", "version", "rows")

    def __init__(self, num_groups: int):
        self.tables: List[List[int]] = [[] for _ in range(num_groups)]
        self.trimmed: List[int] = [0] * num_groups
        self.state_slot: int = -1
        self.version: int = 0                     # grows whenever a table changes
        self.rows: List[object] = [None] * num_groups   # a step builder's memo of each table as an array row

    def num_held(self) -> int:
        return sum(1 for table in self.tables for b in table if b != FREED)

    def holds_pages(self) -> bool:
        return any(b != FREED for table in self.tables for b in table)


class CacheManager:
    def __init__(self, plan: CachePlan, block_size: int = 16, num_blocks: Optional[int] = None,
                 budget_bytes: Optional[int] = None, dtype: str = "bfloat16", device=None,
                 max_state_slots: int = 64, context_hint: Optional[int] = None, step_tokens: int = 0):
        """``num_blocks`` pages in every paged group, or as many as ``budget_bytes`` pay for.

        A budget covers everything the cache holds: the state slots of fixed-size groups first, then pages.
        With ``context_hint`` (the context length requests are expected to reach) a group with a window gets
        only the share of pages its requests can hold at a time - the window, one step's new tokens
        (``step_tokens``) and two pages of slack, out of ``context_hint`` - and the groups that keep every key
        get the rest; without it every paged group gets the same number of pages.
        """
        if block_size <= 0:
            raise InvalidArgument(f"block_size must be positive, got {block_size}")
        if dtype not in _DTYPES:
            raise InvalidArgument(f"KV cache dtype must be one of {', '.join(_DTYPES)}, got '{dtype}'")
        if (num_blocks is None) == (budget_bytes is None):
            raise InvalidArgument("give exactly one of num_blocks and budget_bytes")
        if max_state_slots <= 0:
            raise InvalidArgument(f"max_state_slots must be positive, got {max_state_slots}")
        self.plan = plan
        self.block_size = block_size
        self.dtype = dtype
        self.device = device
        self.max_state_slots = max_state_slots
        elem = torch.empty((), dtype=_DTYPES[dtype]).element_size()
        self.page_bytes: Dict[int, int] = {
            g: 2 * plan.groups[g].num_planes * plan.groups[g].need.num_kv_heads * block_size *
            plan.groups[g].need.head_dim * elem for g in plan.paged_groups}
        self.bytes_per_block = sum(self.page_bytes.values())      # one page of every paged group
        self.state_bytes = 0
        for g in plan.state_groups:
            need = plan.groups[g].need
            if need.dtype not in _STATE_DTYPES:
                raise InvalidArgument(f"state dtype must be one of {', '.join(_STATE_DTYPES)}, got '{need.dtype}'")
            count = 1
            for d in need.shape:
                count *= d
            self.state_bytes += (plan.groups[g].num_planes * max_state_slots * count *
                                 torch.empty((), dtype=_STATE_DTYPES[need.dtype]).element_size())
        cap = _INT32_MAX // block_size                            # slots (page * block_size + offset) must fit in int32
        share = {g: 1.0 for g in plan.paged_groups}
        if num_blocks is None:
            if context_hint is not None and context_hint > 0:
                for g in plan.paged_groups:
                    window = plan.groups[g].need.window
                    if window is not None:
                        share[g] = min(1.0, (window + step_tokens + 2 * block_size) / context_hint)
            left = budget_bytes - self.state_bytes
            if not plan.paged_groups:
                num_blocks = 1
            else:
                per_full_page = sum(share[g] * self.page_bytes[g] for g in plan.paged_groups)
                num_blocks = int(left // per_full_page) if left > 0 else 0
                if num_blocks == 0:
                    raise CapacityError(
                        f"a cache budget of {budget_bytes} bytes does not pay for the {self.state_bytes} bytes of "
                        f"state slots and one {self.bytes_per_block}-byte page of every group")
        if num_blocks <= 0:
            raise InvalidArgument(f"the cache needs at least one block, got {num_blocks}")
        self.num_blocks = min(num_blocks, cap)                    # pages of the groups that keep every key
        self.pool_blocks: Dict[int, int] = {
            g: max(1, min(self.num_blocks, math.ceil(share[g] * self.num_blocks - 1e-9))) for g in plan.paged_groups}

        self.pools: Dict[int, BlockPool] = {g: BlockPool(self.pool_blocks[g]) for g in plan.paged_groups}
        self.has_windows = any(plan.groups[g].need.window is not None for g in plan.paged_groups)
        self._free_state_slots: List[int] = list(range(max_state_slots - 1, -1, -1))
        self._state_slot_used = [False] * max_state_slots
        self.kv: Dict[int, torch.Tensor] = {}
        self.state: Dict[int, torch.Tensor] = {}
        if device is not None:
            for g, group in enumerate(plan.groups):
                need = group.need
                if isinstance(need, PagedKV):
                    self.kv[g] = torch.zeros(
                        (group.num_planes, 2, self.pool_blocks[g], need.num_kv_heads, block_size, need.head_dim),
                        dtype=_DTYPES[dtype], device=device)
                else:
                    self.state[g] = torch.zeros((group.num_planes, max_state_slots) + tuple(need.shape),
                                                dtype=_STATE_DTYPES[need.dtype], device=device)

    def total_bytes(self) -> int:
        """What the cache holds in all: every group's pages and the state slots."""
        return sum(self.pool_blocks[g] * self.page_bytes[g] for g in self.pool_blocks) + self.state_bytes

    def all_free(self) -> bool:
        """Whether every page of every group and every state slot is back."""
        return all(pool.num_free == pool.num_blocks for pool in self.pools.values()) and \
            len(self._free_state_slots) == self.max_state_slots

    # ----------------------------------------------------------------- sizes
    def blocks_for(self, tokens: int) -> int:
        return (tokens + self.block_size - 1) // self.block_size

    def num_free(self, group: Optional[int] = None) -> int:
        """Free pages of one group, or the fewest over all paged groups."""
        if group is not None:
            return self.pools[group].num_free
        if not self.pools:
            return self.num_blocks
        return min(p.num_free for p in self.pools.values())

    def has_free_pages(self, count: int) -> bool:
        """Whether every paged group has ``count`` free pages."""
        return all(pool.num_free >= count for pool in self.pools.values())

    def holds_pages(self, req: "RequestCache") -> bool:
        """Whether giving back what ``req`` holds would free at least one page of some group."""
        return req.holds_pages()

    @property
    def num_free_state_slots(self) -> int:
        return len(self._free_state_slots)

    @property
    def capacity_tokens(self) -> int:
        """The most tokens one request can hold: the pages of the smallest group that keeps every key (a
        group with a window gives pages back as a request grows and sets no such limit)."""
        full = [self.pool_blocks[g] for g in self.pools if self.plan.groups[g].need.window is None]
        return (min(full) if full else self.num_blocks) * self.block_size if self.pools else _INT32_MAX

    # -------------------------------------------------------------- requests
    def new_request(self) -> RequestCache:
        return RequestCache(len(self.plan.groups))

    def _needs_state_slot(self) -> bool:
        return bool(self.plan.state_groups)

    def fit(self, req: RequestCache, computed: int, want: int) -> int:
        """The most of ``want`` further tokens the request can run with its pages plus the free ones.

        Between steps a table covers exactly the computed tokens, so the room of a
        group is (pages in the table + free pages) * block_size - computed
        (``src/engine/batch_scheduler.cpp:44-48``); the smallest room over the groups counts.
        """
        if self._needs_state_slot() and req.state_slot < 0 and not self._free_state_slots:
            return 0
        room = want
        for g, pool in self.pools.items():
            room = min(room, (len(req.tables[g]) + pool.num_free) * self.block_size - computed)
        return max(0, min(room, want))

    def can_admit(self, tokens: int, keep_free: int) -> bool:
        """Whether a request without pages can take ``tokens`` and leave ``keep_free`` pages free in every group."""
        if self._needs_state_slot() and not self._free_state_slots:
            return False
        need = self.blocks_for(tokens)
        return all(pool.num_free - need >= keep_free for pool in self.pools.values())

    def reserve(self, req: RequestCache, new_len: int) -> bool:
        """Grows every table of ``req`` to cover ``new_len`` tokens, all or nothing.

        Returns False, changing nothing, when a pool lacks the pages or no state
        slot is free (``src/kv/paged_kv_cache.cpp:41-49``). Never shrinks.
        """
        if new_len < 0:
            raise InvalidArgument(f"cannot reserve KV blocks for {new_len} tokens")
        want = self.blocks_for(new_len)
        for g, pool in self.pools.items():
            if want - len(req.tables[g]) > pool.num_free:
                return False
        if self._needs_state_slot() and req.state_slot < 0:
            if not self._free_state_slots:
                return False
            slot = self._free_state_slots.pop()
            self._state_slot_used[slot] = True
            req.state_slot = slot
            for tensor in self.state.values():
                tensor[:, slot].zero_()
        for g, pool in self.pools.items():
            table = req.tables[g]
            if len(table) < want:
                req.version += 1
            while len(table) < want:
                table.append(pool.allocate())
        return True

    def slots(self, req: RequestCache, group: int, old_len: int, new_len: int) -> List[int]:
        """Cache slots (page * block_size + offset) of positions [old_len, new_len); never allocates."""
        if old_len < 0 or new_len < old_len:
            raise InvalidArgument(f"bad token range [{old_len}, {new_len})")
        table = req.tables[group]
        bs = self.block_size
        if self.blocks_for(new_len) > len(table):
            raise InvalidArgument(f"block table of {len(table)} blocks cannot hold {new_len} tokens")
        out = []
        for pos in range(old_len, new_len):
            page = table[pos // bs]
            if page == FREED:
                raise InvalidArgument(f"position {pos} lies in a page that was already given back")
            out.append(page * bs + pos % bs)
        return out

    def truncate(self, req: RequestCache, length: int) -> None:
        """Gives back the pages beyond those ``length`` tokens need (a failed step's reservation)."""
        if length < 0:
            raise InvalidArgument(f"cannot truncate a block table to {length} tokens")
        keep = self.blocks_for(length)
        req.version += 1
        for g, pool in self.pools.items():
            table = req.tables[g]
            while len(table) > keep:
                page = table.pop()
                if page != FREED:
                    pool.release(page)
            req.trimmed[g] = min(req.trimmed[g], len(table))
        if length == 0:
            self._release_state_slot(req)

    def trim(self, req: RequestCache, computed: int) -> int:
        """Gives back pages of windowed groups that no later query can read; returns how many.

        The next query sits at position ``computed`` or later and reads keys from
        ``computed - window + 1`` on, so pages wholly below that are free to go.
        Their table entries stay (as FREED) so that positions keep their index.
        """
        freed = 0
        if not self.has_windows:
            return freed
        for g, pool in self.pools.items():
            window = self.plan.groups[g].need.window
            if window is None:
                continue
            first_page = max(0, computed - window + 1) // self.block_size
            table = req.tables[g]
            first_page = min(first_page, len(table))
            for i in range(req.trimmed[g], first_page):
                if table[i] != FREED:
                    pool.release(table[i])
                    table[i] = FREED
                    freed += 1
                    req.version += 1
            req.trimmed[g] = max(req.trimmed[g], first_page)
        return freed

    def _release_state_slot(self, req: RequestCache) -> None:
        if req.state_slot >= 0:
            if not self._state_slot_used[req.state_slot]:
                raise InvalidArgument(f"state slot {req.state_slot} released while already free")
            self._state_slot_used[req.state_slot] = False
            self._free_state_slots.append(req.state_slot)
            req.state_slot = -1

    def release(self, req: RequestCache) -> None:
        """Gives back everything the request holds (it ended, was cancelled or is preempted)."""
        req.version += 1
        for g, pool in self.pools.items():
            for page in req.tables[g]:
                if page != FREED:
                    pool.release(page)
            req.tables[g].clear()
            req.trimmed[g] = 0
        self._release_state_slot(req)

    # --------------------------------------------------------------- storage
    def kv_planes(self, group: int, plane: int):
        """K and V of one plane: ``[num_blocks, num_kv_heads, block_size, head_dim]`` and, transposed
        inside the page, ``[num_blocks, num_kv_heads, head_dim, block_size]``."""
        tensor = self.kv[group]
        nb, kvh, bs, dh = tensor.shape[2:]
        return tensor[plane, 0], tensor[plane, 1].view(nb, kvh, dh, bs)

    def state_plane(self, group: int, plane: int) -> torch.Tensor:
        """The states of one plane: ``[max_state_slots, *shape]``."""
        return self.state[group][plane]

    # ----------------------------------------------------------------- audit
    def audit(self, requests: Iterable[RequestCache]) -> None:
        """Checks that no page is lost, held twice or free while held. Raises AssertionError."""
        requests = list(requests)
        for g, pool in self.pools.items():
            held = [b for r in requests for b in r.tables[g] if b != FREED]
            assert len(held) == len(set(held)), f"group {g}: a page is held twice: {sorted(held)}"
            for b in held:
                assert pool.ref_count(b) == 1, f"group {g}: page {b} is held but has count {pool.ref_count(b)}"
            assert len(held) + pool.num_free == pool.num_blocks, (
                f"group {g}: {len(held)} held + {pool.num_free} free != {pool.num_blocks} pages")
        slots = [r.state_slot for r in requests if r.state_slot >= 0]
        assert len(slots) == len(set(slots)), f"a state slot is held twice: {sorted(slots)}"
        assert len(slots) + len(self._free_state_slots) == self.max_state_slots or not self._needs_state_slot(), \
            "a state slot was lost"
