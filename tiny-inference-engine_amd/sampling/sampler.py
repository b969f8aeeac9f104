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

``sample`` works on the host from a float32 row. ``DeviceSampler`` handles whole steps: greedy rows
and plain temperature rows are drawn by GPU kernels (only the token ids come back, and the uniform
numbers still come from each request's own stream); rows with top-k or top-p go through ``sample``.
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


class DeviceSampler:
    """Samples the rows of one step's logits, on the GPU where the parameters allow it."""

    def __init__(self, device):
        self.device = device

    def sample_rows(self, logits: torch.Tensor, params: Sequence[SamplingParams],
                    rngs: Sequence[RandomStream]) -> List[int]:
        from .. import kernels

        R = logits.shape[0]
        if R != len(params) or R != len(rngs):
            raise InvalidArgument("one set of sampling parameters and one random stream per row")
        out = [0] * R
        greedy_rows = [i for i, p in enumerate(params) if p.greedy]
        plain_rows = [i for i, p in enumerate(params) if not p.greedy and p.top_k == 0 and p.top_p >= 1.0]
        host_rows = [i for i in range(R) if i not in set(greedy_rows) and i not in set(plain_rows)]
        # Kernels work on all rows at once; each kind's result is read where it applies.
        host_argmax = host_max = None
        if greedy_rows or plain_rows:
            # index and maximum side by side in one buffer: one copy to the host, one wait for the GPU
            both = torch.empty(2 * R, dtype=torch.int32, device=logits.device)
            kernels.argmax_rows(logits, both[:R], both[R:].view(torch.float32))
            host = both.cpu().numpy()
            host_argmax = host[:R]
            host_max = host[R:].view(np.float32)
            for i in greedy_rows + plain_rows:
                if host_argmax[i] < 0:
                    raise InvalidArgument(f"a logit of row {i} is NaN")
                if host_max[i] == -np.inf:
                    raise InvalidArgument(f"all logits of row {i} are -inf")
            for i in greedy_rows:
                out[i] = int(host_argmax[i])
        # A +inf logit is certain and does not consume a random number; the other rows draw one each.
        drawing = [i for i in plain_rows if host_max[i] != np.inf]
        for i in plain_rows:
            out[i] = int(host_argmax[i])
        if drawing:
            inv_t = np.ones(R, dtype=np.float32)
            uniform = np.zeros(R, dtype=np.float64)
            for i in drawing:
                inv_t[i] = np.float32(1.0) / np.float32(params[i].temperature)
                uniform[i] = rngs[i].unit()
            drawn = torch.empty(R, dtype=torch.int32, device=logits.device)
            kernels.sample_rows(logits, torch.from_numpy(inv_t).to(logits.device),
                                torch.from_numpy(uniform).to(logits.device), drawn)
            host_drawn = drawn.cpu().numpy()
            for i in drawing:
                out[i] = int(host_drawn[i])
        for i in host_rows:
            out[i] = sample(logits[i].cpu().numpy(), params[i], rngs[i])
        return out
