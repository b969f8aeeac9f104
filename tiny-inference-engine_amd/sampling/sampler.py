"""Drawing the next token from a row of logits.

The rules are the reference's (``src/sampling/sampler.cpp:18-81``):

* empty logits, any NaN, or all -inf: InvalidArgument;
* temperature 0, or one whose reciprocal is not finite: the first maximum (ties go to the lowest id);
* a +inf logit is certain: the lowest such id, without touching the random stream;
* otherwise ``(logit - max) * (1 / temperature)`` - shifted before scaling so a tiny temperature can
  neither overflow nor turn every logit into -inf -, the ``top_k`` most likely kept (value
  descending, id ascending), unnormalised softmax weights with a float32 exp and a double sum, the
  smallest prefix whose weight reaches ``top_p * total`` kept, one uniform draw in [0, total) and a
  walk over the kept candidates.

``sample`` works on the host from a float32 row: it is the rule written out, for single rows and for checking.
``DeviceSampler`` handles whole steps on the GPU: greedy rows, plain temperature rows and rows with top-k or
top-p each have a kernel; only the token ids come back, and the uniform numbers still come from each request's
own stream. The top-k / top-p kernel sums its weights as integers in units of 2^-44 of the largest, where
``sample`` sums in double precision: the two differ only for a draw within 1e-8 of a boundary.
"""

from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

from ..errors import InvalidArgument
from .params import SamplingParams
from .rng import RandomStream


def sample(logits: np.ndarray, params: SamplingParams, rng: RandomStream) -> int:
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    n = logits.shape[0]
    if n == 0:
        raise InvalidArgument("cannot sample from empty logits")
    nan = np.isnan(logits)
    if nan.any():
        raise InvalidArgument(f"logit {int(np.argmax(nan))} is NaN")
    arg = int(np.argmax(logits))                      # first maximum: ties go to the lowest id
    max_raw = logits[arg]
    if max_raw == -np.inf:
        raise InvalidArgument("all logits are -inf")
    if params.greedy or max_raw == np.inf:
        return arg
    with np.errstate(over="ignore", invalid="ignore"):
        inv_t = np.float32(1.0) / np.float32(params.temperature)
        scaled = (logits - max_raw) * inv_t           # float32; the maximum maps to 0, the rest to [-inf, 0]

    ids = None                                        # None: all candidates in index order
    if 0 < params.top_k < n:
        k = params.top_k
        kth = np.partition(scaled, n - k)[n - k]      # value of the k-th most likely
        above = np.flatnonzero(scaled > kth)
        ties = np.flatnonzero(scaled == kth)[:k - above.size]
        ids = np.concatenate([above, ties])
        ids = ids[np.lexsort((ids, -scaled[ids]))]    # value descending, id ascending
    elif params.top_p < 1.0:
        ids = np.lexsort((np.arange(n), -scaled))
    cand = scaled if ids is None else scaled[ids]
    with np.errstate(invalid="ignore"):
        weights = np.exp(cand - cand.max(), dtype=np.float32)
    cumulative = np.cumsum(weights, dtype=np.float64)
    keep = cand.shape[0]
    total = float(cumulative[-1])
    if params.top_p < 1.0:
        keep = int(np.searchsorted(cumulative, float(np.float32(params.top_p)) * total, side="left")) + 1
        keep = min(keep, cand.shape[0])
        total = float(cumulative[keep - 1])
    r = rng.uniform(0.0, total)
    pick = int(np.searchsorted(cumulative[:keep], r, side="right"))   # first i with r - cumulative[i] < 0
    pick = min(pick, keep - 1)
    return int(pick if ids is None else ids[pick])


class GreedyTicket:
    """Rows whose argmax has been asked of the GPU and not yet read: see ``DeviceSampler.launch_greedy``."""

    __slots__ = ("rows", "device_tokens", "host", "event")

    def __init__(self, rows, device_tokens, host, event):
        self.rows = rows
        self.device_tokens = device_tokens     # int32 [rows] on the device: the chosen tokens, in row order
        self.host = host                       # pinned int32 [2 * rows]: tokens, then the maxima's bits
        self.event = event


class DeviceSampler:
    """Samples the rows of one step's logits, on the GPU where the parameters allow it.

    The results come back through pinned host buffers that live as long as the sampler: a step of greedy
    rows is one kernel, one copy of ``2 R`` words and one wait. ``launch_greedy`` / ``collect`` split that
    into asking and reading, so that a caller may queue the next step (whose tokens it takes from
    ``ticket.device_tokens``) before it reads this one's; two sets of buffers alternate for that."""

    GREEDY, PLAIN, FILTERED = 0, 1, 2      # argmax kernel / temperature kernel / top-k and top-p kernel

    def __init__(self, device):
        self.device = torch.device(device)
        self._rows = 0
        self._sets = []
        self._turn = 0

    def _buffers(self, rows: int):
        """Device words and pinned host words: 3 R of results (argmax, maxima, draws), then 6 R of parameters."""
        if rows > self._rows:
            self._rows = max(64, 2 * rows)
            self._sets = [(torch.empty(9 * self._rows, dtype=torch.int32, device=self.device),
                           torch.empty(9 * self._rows, dtype=torch.int32, pin_memory=self.device.type == "cuda"))
                          for _ in range(2)]
        self._turn ^= 1
        return self._sets[self._turn]

    def _fetch(self, dev: torch.Tensor, host: torch.Tensor, count: int) -> np.ndarray:
        host[:count].copy_(dev[:count], non_blocking=True)
        if self.device.type == "cuda":
            torch.cuda.current_stream(self.device).synchronize()
        return host.numpy()[:count]

    # ------------------------------------------------------------- greedy rows, asked for and read apart
    def launch_greedy(self, logits: torch.Tensor) -> GreedyTicket:
        """Queues the argmax of every row and the copy of the results to the host; returns at once."""
        from .. import kernels

        R = logits.shape[0]
        dev, host = self._buffers(R)
        kernels.argmax_rows(logits, dev[:R], dev[R:2 * R].view(torch.float32))
        host[:2 * R].copy_(dev[:2 * R], non_blocking=True)
        event = None
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
        return GreedyTicket(R, dev[:R], host, event)

    def collect(self, ticket: GreedyTicket) -> List[int]:
        """Waits for a ticket's results; the tokens of its rows (ties went to the lowest id)."""
        if ticket.event is not None:
            ticket.event.synchronize()
        R = ticket.rows
        fetched = ticket.host.numpy()[:2 * R]
        best, top = fetched[:R], fetched[R:].view(np.float32)
        if (best < 0).any():
            raise InvalidArgument(f"a logit of row {int(np.flatnonzero(best < 0)[0])} is NaN")
        if (top == -np.inf).any():
            raise InvalidArgument(f"all logits of row {int(np.flatnonzero(top == -np.inf)[0])} are -inf")
        return best.tolist()

    # ------------------------------------------------------------------------------------ any rows, at once
    def sample_rows(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                    rngs: Sequence[RandomStream]) -> List[int]:
        from .. import kernels

        R = logits.shape[0]
        if R != len(params) or R != len(rngs):
            raise InvalidArgument("one set of sampling parameters and one random stream per row")
        V = logits.shape[1]
        # Without a filter the reference walks the candidates in index order, with one in the order of likelihood
        # (src/sampling/sampler.cpp:41-54): the same uniform number picks different tokens, so each has its kernel.
        kinds = np.fromiter((self.GREEDY if p.greedy else (self.FILTERED if 0 < p.top_k < V or p.top_p < 1.0 else self.PLAIN)
                             for p in params), dtype=np.int8, count=R)
        if not kinds.any():
            return self.collect(self.launch_greedy(logits))
        # The argmax kernel works on all rows: it answers the greedy rows, finds NaN and all -inf rows, and a
        # +inf logit, which is certain and consumes no random number. Index and maximum lie side by side, so one
        # copy brings both.
        dev, host = self._buffers(R)
        kernels.argmax_rows(logits, dev[:R], dev[R:2 * R].view(torch.float32))
        fetched = self._fetch(dev, host, 2 * R)
        best, top = fetched[:R], fetched[R:].view(np.float32)
        if (best < 0).any():
            raise InvalidArgument(f"a logit of row {int(np.flatnonzero(best < 0)[0])} is NaN")
        if (top == -np.inf).any():
            raise InvalidArgument(f"all logits of row {int(np.flatnonzero(top == -np.inf)[0])} are -inf")
        out = best.astype(np.int64)
        plain = np.flatnonzero((kinds == self.PLAIN) & (top != np.inf))
        filtered = np.flatnonzero((kinds == self.FILTERED) & (top != np.inf))
        if not plain.size and not filtered.size:
            return out.tolist()
        # The parameters of the drawing rows go up in one copy: 1 / temperature, top_p, top_k, the numbers of the
        # drawing rows, those with a filter first (one word a row each), one uniform number a row (two words).
        P = R + (R & 1)                                    # the float64 numbers start on 8 bytes
        at = 3 * self._rows
        words = host[at:at + 6 * P].numpy()
        inv_t, top_p = words[:R].view(np.float32), words[P:P + R].view(np.float32)
        top_k, rows, uniform = words[2 * P:2 * P + R], words[3 * P:3 * P + R], words[4 * P:6 * P].view(np.float64)[:R]
        inv_t[:], top_p[:], top_k[:], uniform[:] = 1.0, 1.0, 0, 0.0
        for i in np.concatenate([plain, filtered]):
            inv_t[i] = np.float32(1.0) / np.float32(params[i].temperature)
            uniform[i] = rngs[i].unit()
        for i in filtered:
            top_p[i], top_k[i] = params[i].top_p, min(params[i].top_k, V)
        rows[:filtered.size] = filtered
        rows[filtered.size:filtered.size + plain.size] = plain
        up = dev[at:at + 6 * P]
        up.copy_(host[at:at + 6 * P], non_blocking=True)
        d_inv_t, d_uniform = up[:R].view(torch.float32), up[4 * P:6 * P].view(torch.float64)[:R]
        drawn = dev[2 * R:3 * R]
        maxima = dev[R:2 * R].view(torch.float32)
        if plain.size:
            kernels.sample_rows(logits, d_inv_t, d_uniform, drawn,
                                up[3 * P + filtered.size:3 * P + filtered.size + plain.size], maxima)
        if filtered.size:
            kernels.sample_rows_filtered(logits, d_inv_t, d_uniform, up[2 * P:2 * P + R], up[P:P + R].view(torch.float32),
                                         drawn, up[3 * P:3 * P + filtered.size], maxima)
        got = self._fetch(dev[2 * R:], host[2 * R:], R)
        out[plain] = got[plain]
        out[filtered] = got[filtered]
        return out.tolist()
