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

from typing import List, Optional, Sequence

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


class Ticket:
    """Rows whose tokens have been asked of the GPU and not yet read: see ``DeviceSampler.launch``."""

    __slots__ = ("rows", "device_tokens", "host", "event", "drew_none", "drawing", "rngs")

    def __init__(self, rows, device_tokens, host, event, drew_none=None, drawing=(), rngs=()):
        self.rows = rows
        self.device_tokens = device_tokens     # int32 [rows] on the device: the chosen tokens, in row order
        self.host = host                       # pinned int32 [2 * rows]: tokens, then the maxima's bits
        self.event = event
        self.drew_none = drew_none             # int32 [rows] on the device: 1 where a drawing row took no number
        self.drawing = drawing                 # the rows that draw, and their streams: a number is taken from a
        self.rngs = rngs                       # stream when the row is known to have used one


class DeviceSampler:
    """Samples the rows of one step's logits on the GPU.

    The results come back through pinned host buffers that live as long as the sampler: a step is the argmax
    kernel over all rows (the greedy rows' answer, the maxima for the others, and what finds a NaN or a row of
    -inf), a drawing kernel for the rows with a temperature and one for those with top-k or top-p, which put
    their tokens where the argmax stood, one copy of ``2 R`` words and one wait. ``launch`` / ``collect`` split
    that into asking and reading, so that a caller may queue the next step (whose tokens it takes from
    ``ticket.device_tokens``) before it reads this one's; sets of buffers take turns for that (two, or as many as
    ``keep_apart`` says).

    A row's uniform number is the next of its request's stream, but a row with a +inf logit takes none, and
    whether that happened in a step not yet read is known on the GPU only. A step queued behind such a step
    (``previous``) therefore carries two numbers a row, the stream's next and the one after, and the kernel takes
    the one that fits what the step before did; the streams move on when a step is read."""

    GREEDY, PLAIN, FILTERED = 0, 1, 2      # argmax kernel / temperature kernel / top-k and top-p kernel
    RESULTS, PARAMETERS = 3, 8             # words a row: tokens, maxima, marks / what the drawing kernels take

    def __init__(self, device):
        self.device = torch.device(device)
        self._rows = 0
        self._sets = []
        self._turn = 0
        self._num_sets = 2

    def keep_apart(self, tickets: int) -> None:
        """How many tickets may be outstanding or in the making at a time: each has a set of buffers of its own."""
        if tickets > self._num_sets:
            self._num_sets = tickets
            self._rows = 0                 # the next launch makes the sets anew (outstanding tickets keep theirs)

    def _buffers(self, rows: int):
        if rows > self._rows:
            self._rows = max(64, 2 * rows)
            words = (self.RESULTS + self.PARAMETERS) * self._rows
            self._sets = [(torch.empty(words, dtype=torch.int32, device=self.device),
                           torch.empty(words, dtype=torch.int32, pin_memory=self.device.type == "cuda"))
                          for _ in range(self._num_sets)]
        self._turn = (self._turn + 1) % self._num_sets
        return self._sets[self._turn]

    # ------------------------------------------------------------------------- asked for and read apart
    def launch_greedy(self, logits: torch.Tensor) -> Ticket:
        """Queues the argmax of every row and the copy of the results to the host; returns at once."""
        from .. import kernels

        R = logits.shape[0]
        dev, host = self._buffers(R)
        kernels.argmax_rows(logits, dev[:R], dev[R:2 * R].view(torch.float32))
        return self._ticket(dev, host, R)

    def _ticket(self, dev, host, R, drew_none=None, drawing=(), rngs=()) -> Ticket:
        host[:2 * R].copy_(dev[:2 * R], non_blocking=True)
        event = None
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
        return Ticket(R, dev[:R], host, event, drew_none, drawing, rngs)

    def launch(self, logits: torch.Tensor, params: Sequence[SamplingParams], rngs: Sequence[RandomStream],
               previous: Optional[Ticket] = None) -> Ticket:
        """Queues the choice of a token for every row; returns at once. ``previous``: the ticket of the step
        before, of the same requests in the same rows, if it has not been collected yet."""
        from .. import kernels

        R, V = logits.shape
        if R != len(params) or R != len(rngs):
            raise InvalidArgument("one set of sampling parameters and one random stream per row")
        if previous is not None and previous.rows != R:
            raise InvalidArgument(f"the step before had {previous.rows} rows, this one has {R}")
        # Without a filter the reference walks the candidates in index order, with one in the order of likelihood
        # (src/sampling/sampler.cpp:41-54): the same uniform number picks different tokens, so each has its kernel.
        kinds = np.fromiter((self.GREEDY if p.greedy else (self.FILTERED if 0 < p.top_k < V or p.top_p < 1.0 else self.PLAIN)
                             for p in params), dtype=np.int8, count=R)
        dev, host = self._buffers(R)
        maxima = dev[R:2 * R].view(torch.float32)
        kernels.argmax_rows(logits, dev[:R], maxima)
        filtered, plain = np.flatnonzero(kinds == self.FILTERED), np.flatnonzero(kinds == self.PLAIN)
        if not filtered.size and not plain.size:
            return self._ticket(dev, host, R)
        # The parameters go up in one copy, a word a row each: 1 / temperature, top_p, top_k, the numbers of the
        # drawing rows (those with a filter first), and two words a row for each of the two uniform numbers.
        P = R + (R & 1)                                    # the float64 numbers start on 8 bytes
        at = self.RESULTS * self._rows
        words = host[at:at + self.PARAMETERS * P].numpy()
        inv_t, top_p = words[:R].view(np.float32), words[P:P + R].view(np.float32)
        top_k, rows = words[2 * P:2 * P + R], words[3 * P:3 * P + R]
        uniform, other = words[4 * P:6 * P].view(np.float64)[:R], words[6 * P:8 * P].view(np.float64)[:R]
        inv_t[:], top_p[:], top_k[:], uniform[:], other[:] = 1.0, 1.0, 0, 0.0, 0.0
        drawing = np.concatenate([filtered, plain])
        if previous is not None and not np.array_equal(previous.drawing, drawing):
            raise InvalidArgument("the step before did not draw for the same rows")
        ahead = 0 if previous is None else 1               # numbers of the stream that the step before may have used
        for i in drawing:
            inv_t[i] = np.float32(1.0) / np.float32(params[i].temperature)
            uniform[i] = rngs[i].peek_unit(ahead)
            other[i] = rngs[i].peek_unit(0)
        for i in filtered:
            top_p[i], top_k[i] = params[i].top_p, min(params[i].top_k, V)
        rows[:drawing.size] = drawing
        up = dev[at:at + self.PARAMETERS * P]
        up.copy_(host[at:at + self.PARAMETERS * P], non_blocking=True)
        d_inv_t = up[:R].view(torch.float32)
        d_uniform, d_other = up[4 * P:6 * P].view(torch.float64)[:R], up[6 * P:8 * P].view(torch.float64)[:R]
        drew_none = dev[2 * R:3 * R]
        take_other = None if previous is None else previous.drew_none
        if take_other is None:
            d_other = None
        if filtered.size:
            kernels.sample_rows_filtered(logits, d_inv_t, d_uniform, up[2 * P:2 * P + R], up[P:P + R].view(torch.float32),
                                         dev[:R], up[3 * P:3 * P + filtered.size], maxima, d_other, take_other, drew_none)
        if plain.size:
            kernels.sample_rows(logits, d_inv_t, d_uniform, dev[:R], up[3 * P + filtered.size:3 * P + drawing.size], maxima,
                                d_other, take_other, drew_none)
        return self._ticket(dev, host, R, drew_none, drawing, [rngs[i] for i in drawing])

    def collect(self, ticket: Ticket) -> List[int]:
        """Waits for a ticket's results; the tokens of its rows. Moves the streams of the rows that drew."""
        if ticket.event is not None:
            ticket.event.synchronize()
        R = ticket.rows
        fetched = ticket.host.numpy()[:2 * R]
        best, top = fetched[:R], fetched[R:].view(np.float32)
        if (best < 0).any():
            raise InvalidArgument(f"a logit of row {int(np.flatnonzero(best < 0)[0])} is NaN")
        if (top == -np.inf).any():
            raise InvalidArgument(f"all logits of row {int(np.flatnonzero(top == -np.inf)[0])} are -inf")
        for i, rng in zip(ticket.drawing, ticket.rngs):
            if top[i] != np.inf:               # a +inf logit is certain and takes no random number
                rng.skip()
        return best.tolist()

    # ------------------------------------------------------------------------------------ any rows, at once
    def sample_rows(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                    rngs: Sequence[RandomStream]) -> List[int]:
        if all(p.greedy for p in params):
            return self.collect(self.launch_greedy(logits))
        return self.collect(self.launch(logits, params, rngs))
