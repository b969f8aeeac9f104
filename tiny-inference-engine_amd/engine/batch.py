"""One step's batch: flat, unpadded runs of tokens, one run per request.

An entry is (a request's cache holdings, how many of its tokens are already
cached, its next tokens, the rows among them whose logits are wanted). The runs
may be whole prompts, portions of prompts cut anywhere, or single decoded
tokens, freely mixed. ``build`` lays out the arrays the kernels read, as the
reference's engine does (``src/engine/engine.cpp:104-135``):

    tokens[T] positions[T] seq_of_row[T] query_start[S+1] context_lens[S]
    state_slots[S] logit_rows[R] token_sources[T]   and per paged cache group:
    slot_mapping[T] block_tables[S, max_blocks_per_seq]

``context_lens`` counts the cached tokens AFTER this step; the query at row t of
sequence s sits at position ``context_lens[s] - n_new[s] + (t - query_start[s])``.
All arrays travel to the device in one copy from one pinned staging buffer.
"""

from __future__ import annotations

import dataclasses
import itertools
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .. import kernels
from ..cache.manager import CacheManager, RequestCache
from ..errors import CapacityError, InvalidArgument


@dataclasses.dataclass
class StepEntry:
    cache: RequestCache
    start: int                       # tokens of the request already in the cache
    tokens: Sequence[int]            # its next tokens, run in this step
    want: Sequence[int] = ()         # places among ``tokens`` whose logits are wanted
    token_from: int = -1             # >= 0: the entry's one token is not known to the host; it is this entry of
                                     # the tokens an earlier step's sampling left on the device (ModelRunner.step)


class GroupStep:
    """This step's view of one paged cache group."""

    def __init__(self, slot_mapping, block_tables):
        self.slot_mapping = slot_mapping     # int32 [T]
        self.block_tables = block_tables     # int32 [S, max_blocks_per_seq]
        self.extra: Dict[str, torch.Tensor] = {}
        # a step of single tokens over sequences of very different lengths: (shares, their length in tiles of 32
        # keys as one int32 on the device) for the decode attention kernel; None: the rule by the step's size
        self.key_shares = None


class StepBatch:
    """The arrays of one step, on the device, plus the host-side numbers parts plan with."""

    def __init__(self):
        self.num_tokens = 0
        self.num_seqs = 0
        self.num_logit_rows = 0
        self.tokens = self.positions = self.seq_of_row = self.token_sources = None
        self.takes_device_tokens = False      # some row's token comes from an earlier step's sampling output
        self.query_start = self.context_lens = self.state_slots = self.logit_rows = None
        self.groups: Dict[int, GroupStep] = {}
        # host copies for planning
        self.host_new_tokens: List[int] = []
        self.host_context_lens: List[int] = []
        self.host_state_slots: List[int] = []
        self.max_context = 0
        self.plan_context = 0      # the context length kernels size their grids for (>= max_context)
        self.share_key = ()        # the shares planned per cache group, where a recorded step depends on them
        self.max_new_tokens = 0
        self.all_decode = False
        self.memo: Dict = {}       # per-step values kernels derive once and share between layers


def _align(n: int, to: int = 4) -> int:
    return (n + to - 1) // to * to


class BatchBuilder:
    """Builds StepBatches into reusable staging memory."""

    def __init__(self, cache: CacheManager, vocab_size: int, max_blocks_per_seq: int, device):
        if max_blocks_per_seq <= 0:
            raise InvalidArgument(f"max_blocks_per_seq must be positive, got {max_blocks_per_seq}")
        self.cache = cache
        self.vocab_size = vocab_size
        self.max_blocks_per_seq = max_blocks_per_seq
        self.device = torch.device(device)
        self._host: Optional[torch.Tensor] = None
        self._dev: Optional[torch.Tensor] = None
        self._copied = None  # event: the last copy out of the staging buffer has finished

    def _buffers(self, count: int):
        if self._host is None or self._host.numel() < count:
            size = max(count * 2, 4096)
            pin = self.device.type == "cuda"
            self._host = torch.empty(size, dtype=torch.int32, pin_memory=pin)
            self._dev = torch.empty(size, dtype=torch.int32, device=self.device)
            self._copied = None
        elif self._copied is not None:
            self._copied.synchronize()
        return self._host, self._dev

    @property
    def staging_ptr(self) -> int:
        """Address of the device-side staging buffer; a recorded step is bound to it."""
        return 0 if self._dev is None else self._dev.data_ptr()

    @staticmethod
    def _table_row(cache, g: int, MB: int) -> np.ndarray:
        """A request's block table of group ``g`` as a row of ``MB`` page numbers: 0 where the table has ended,
        FREED where a window has passed. Kept on the request between steps, rebuilt only when the table changed."""
        memo = cache.rows[g]
        if memo is None or memo[0] != cache.version or memo[1].shape[0] != MB:
            arr = np.zeros(MB, dtype=np.int32)
            table = cache.tables[g][:MB]
            if table:
                arr[:len(table)] = table
            memo = cache.rows[g] = (cache.version, arr)
        return memo[1]

    def _check(self, entries: Sequence[StepEntry]):
        """Refuses what must never reach a kernel; returns (rows, wanted rows, whether every entry is one token)."""
        MB = self.max_blocks_per_seq
        groups = self.cache.plan.paged_groups
        needs_slot = bool(self.cache.plan.state_groups)
        seen = set()
        T = R = 0
        for e in entries:
            n = len(e.tokens)
            if n < 1:
                raise InvalidArgument("an entry of a step needs at least one token")
            key = id(e.cache)
            if key in seen:
                raise InvalidArgument("a request appears twice in one step")
            seen.add(key)
            if e.start < 0:
                raise InvalidArgument(f"an entry starts at position {e.start}")
            if e.token_from >= 0 and n != 1:
                raise InvalidArgument(f"an entry takes its token from the device and brings {n} tokens, not one")
            for w in e.want:
                if not 0 <= w < n:
                    raise InvalidArgument(f"wanted place {w} lies outside the entry's {n} tokens")
            need = self.cache.blocks_for(e.start + n)
            if need > MB:
                raise CapacityError(
                    f"{e.start + n} tokens need {need} KV blocks but a block-table row holds {MB}")
            for g in groups:
                if len(e.cache.tables[g]) < need:
                    raise InvalidArgument(
                        f"a request has {len(e.cache.tables[g])} KV blocks reserved; {e.start + n} tokens need {need}")
            if needs_slot and e.cache.state_slot < 0:
                raise InvalidArgument("a request of a model with per-request state has no state slot")
            T += n
            R += len(e.want)
        return T, R, T == len(entries)

    def _bad_token(self, ids) -> InvalidArgument:
        bad = next(int(t) for t in ids if not 0 <= int(t) < self.vocab_size)
        return InvalidArgument(f"token id {bad} outside vocabulary of {self.vocab_size}")

    def _fill_decode(self, entries, view, batch: StepBatch) -> None:
        """Every entry brings one token: the arrays are filled as whole vectors, not entry by entry."""
        S = len(entries)
        bs, MB = self.cache.block_size, self.max_blocks_per_seq
        starts = np.fromiter((e.start for e in entries), dtype=np.int32, count=S)
        ids = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=S)
        if ids.min() < 0 or ids.max() >= self.vocab_size:
            raise self._bad_token(ids)
        order = np.arange(S + 1, dtype=np.int32)
        view("tokens")[:] = ids
        view("token_sources")[:] = np.fromiter((e.token_from for e in entries), dtype=np.int32, count=S)
        view("positions")[:] = starts
        view("seq_of_row")[:] = order[:S]
        view("query_start")[:] = order
        view("context_lens")[:] = starts + 1
        slots = [e.cache.state_slot for e in entries]
        view("state_slots")[:] = np.maximum(np.asarray(slots, dtype=np.int32), 0)
        view("logit_rows")[:] = [s for s, e in enumerate(entries) for _ in e.want]     # wanted places are all 0
        page_of_start = starts // bs
        for g in self.cache.plan.paged_groups:
            tables = view(("tables", g)).reshape(S, MB)
            for s, e in enumerate(entries):
                tables[s] = self._table_row(e.cache, g, MB)
            pages = tables[order[:S], page_of_start]
            if pages.min() < 0:
                s = int(np.argmin(pages))
                raise InvalidArgument(f"position {int(starts[s])} lies in a page that was already given back")
            view(("slots", g))[:] = pages * bs + starts % bs
            np.maximum(tables, 0, out=tables)        # FREED (-1) -> 0: the kernels never read those entries
        batch.host_new_tokens = [1] * S
        batch.host_context_lens = (starts + 1).tolist()
        batch.host_state_slots = slots

    def _fill_general(self, entries, view, batch: StepBatch) -> None:
        """Entries of any length: the rows of all of them are laid out as whole vectors (a step of many decoded
        tokens beside a few prompts costs the host little more than a step of decoded tokens alone)."""
        bs, MB = self.cache.block_size, self.max_blocks_per_seq
        S = len(entries)
        counts = np.fromiter((len(e.tokens) for e in entries), dtype=np.int32, count=S)
        starts = np.fromiter((e.start for e in entries), dtype=np.int32, count=S)
        first_row = np.zeros(S + 1, dtype=np.int32)
        np.cumsum(counts, out=first_row[1:])
        T = int(first_row[-1])
        ids = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int64, count=T)
        if ids.min() < 0 or ids.max() >= self.vocab_size:
            raise self._bad_token(ids)
        seq = np.repeat(np.arange(S, dtype=np.int32), counts)
        where = starts[seq] + (np.arange(T, dtype=np.int32) - first_row[seq])
        view("tokens")[:] = ids
        view("token_sources")[:] = np.repeat(np.fromiter((e.token_from for e in entries), dtype=np.int32, count=S), counts)
        view("positions")[:] = where
        view("seq_of_row")[:] = seq
        view("query_start")[:] = first_row
        view("context_lens")[:] = starts + counts
        slots = [e.cache.state_slot for e in entries]
        view("state_slots")[:] = np.maximum(np.asarray(slots, dtype=np.int32), 0)
        view("logit_rows")[:] = [int(first_row[s]) + w for s, e in enumerate(entries) for w in e.want]
        page_of_row = where // bs
        for g in self.cache.plan.paged_groups:
            tables = view(("tables", g)).reshape(S, MB)
            for s, e in enumerate(entries):
                tables[s] = self._table_row(e.cache, g, MB)
            pages = tables[seq, page_of_row]
            if pages.min() < 0:
                gone = int(where[int(np.argmin(pages))])
                raise InvalidArgument(f"position {gone} lies in a page that was already given back")
            view(("slots", g))[:] = pages * bs + where % bs
            np.maximum(tables, 0, out=tables)        # FREED (-1) -> 0: the kernels never read those entries
        batch.host_new_tokens = counts.tolist()
        batch.host_context_lens = (starts + counts).tolist()
        batch.host_state_slots = slots

    def build(self, entries: Sequence[StepEntry]) -> StepBatch:
        if not entries:
            raise InvalidArgument("a step needs at least one entry")
        MB = self.max_blocks_per_seq
        S = len(entries)
        T, R, all_single = self._check(entries)
        groups = self.cache.plan.paged_groups
        layout = {}
        offset = 0
        for name, count in (("tokens", T), ("positions", T), ("seq_of_row", T), ("query_start", S + 1),
                            ("context_lens", S), ("state_slots", S), ("logit_rows", R), ("token_sources", T)):
            layout[name] = (offset, count)
            offset += _align(count)
        for g in groups:
            layout[("slots", g)] = (offset, T)
            offset += _align(T)
            layout[("tables", g)] = (offset, S * MB)
            offset += _align(S * MB)
            layout[("share_tiles", g)] = (offset, 1)
            offset += _align(1)
        host_t, dev_t = self._buffers(offset)
        host = host_t.numpy()

        def view(key):
            o, c = layout[key]
            return host[o:o + c]

        batch = StepBatch()
        if all_single:
            self._fill_decode(entries, view, batch)
        else:
            self._fill_general(entries, view, batch)

        batch.max_context = max(batch.host_context_lens)
        batch.plan_context = 1024                 # contexts are planned for in buckets: 1024, 2048, 4096, ...
        while batch.plan_context < batch.max_context:
            batch.plan_context *= 2
        shares = {}
        for g in groups:
            need = self.cache.plan.groups[g].need
            shares[g] = (kernels.decode_share_plan(batch.host_context_lens, need.num_kv_heads, batch.plan_context,
                                                   self.cache.block_size, need.window) if all_single else (0, 0))
            view(("share_tiles", g))[0] = shares[g][1]

        dev_t[:offset].copy_(host_t[:offset], non_blocking=True)
        if self.device.type == "cuda":
            self._copied = torch.cuda.Event()
            self._copied.record()

        def dev(key, shape=None):
            o, c = layout[key]
            t = dev_t[o:o + c]
            return t.view(*shape) if shape else t

        batch.num_tokens, batch.num_seqs, batch.num_logit_rows = T, S, R
        batch.tokens, batch.positions, batch.seq_of_row = dev("tokens"), dev("positions"), dev("seq_of_row")
        batch.query_start, batch.context_lens = dev("query_start"), dev("context_lens")
        batch.state_slots, batch.logit_rows = dev("state_slots"), dev("logit_rows")
        batch.token_sources = dev("token_sources")
        batch.takes_device_tokens = any(e.token_from >= 0 for e in entries)
        for g in groups:
            batch.groups[g] = GroupStep(dev(("slots", g)), dev(("tables", g), (S, MB)))
            if shares[g][1] > 0:
                batch.groups[g].key_shares = (shares[g][0], dev(("share_tiles", g)))
        batch.share_key = tuple(shares[g][0] if shares[g][1] > 0 else 0 for g in groups)
        batch.max_new_tokens = max(batch.host_new_tokens)
        batch.all_decode = batch.max_new_tokens == 1
        return batch
