"""The random stream of a request: a 64-bit Mersenne Twister seeded with the request's seed.

The reference gives every sequence a ``std::mt19937_64`` (``src/engine/sequence.h:23``,
seeded at ``src/engine/engine.cpp:58``) and draws one
``uniform_real_distribution<double>(0, total)`` per sampled token
(``src/sampling/sampler.cpp:75``). The generator below implements the published
MT19937-64 recurrence (Matsumoto and Nishimura) so that a seed means the same
stream here; ``uniform`` maps one 64-bit output to [low, high) the way the
standard distribution does for a 64-bit engine.
"""

from __future__ import annotations

import math

_N, _M = 312, 156
_UPPER, _LOWER = 0xFFFFFFFF80000000, 0x000000007FFFFFFF
_MATRIX = 0xB5026F5AA96619E9
_MASK64 = 0xFFFFFFFFFFFFFFFF
_TWO64 = float(2 ** 64)


class RandomStream:
    __slots__ = ("_state", "_next", "_seen")

    def __init__(self, seed: int = 0):
        state = [seed & _MASK64]
        for i in range(1, _N):
            prev = state[-1]
            state.append((6364136223846793005 * (prev ^ (prev >> 62)) + i) & _MASK64)
        self._state = state
        self._next = _N
        self._seen = []            # outputs looked at with ``peek_unit`` and not taken yet, the next one first

    def _refill(self) -> None:
        s = self._state
        for i in range(_N):
            y = (s[i] & _UPPER) | (s[i + 1 - _N if i + 1 >= _N else i + 1] & _LOWER)
            v = s[i + _M - _N if i + _M >= _N else i + _M] ^ (y >> 1)
            if y & 1:
                v ^= _MATRIX
            s[i] = v
        self._next = 0

    def next_u64(self) -> int:
        if self._seen:
            return self._seen.pop(0)
        return self._generate()

    def _generate(self) -> int:
        if self._next >= _N:
            self._refill()
        y = self._state[self._next]
        self._next += 1
        y ^= (y >> 29) & 0x5555555555555555
        y ^= (y << 17) & 0x71D67FFFEDA60000
        y ^= (y << 37) & 0xFFF7EEE000000000
        y ^= y >> 43
        return y & _MASK64

    def unit(self) -> float:
        """A double in [0, 1): one output scaled by 2^-64, clamped below 1."""
        return self._as_unit(self.next_u64())

    @staticmethod
    def _as_unit(output: int) -> float:
        u = output / _TWO64
        return u if u < 1.0 else math.nextafter(1.0, 0.0)

    def peek_unit(self, ahead: int = 0) -> float:
        """What the ``ahead + 1``-th call of ``unit`` from now will return; takes nothing from the stream."""
        while len(self._seen) <= ahead:
            self._seen.append(self._generate())
        return self._as_unit(self._seen[ahead])

    def skip(self, count: int = 1) -> None:
        """Takes ``count`` outputs from the stream, unseen."""
        for _ in range(count):
            self.next_u64()

    def uniform(self, low: float, high: float) -> float:
        return self.unit() * (high - low) + low
