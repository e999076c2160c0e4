"""The 64-bit Mersenne Twister and the uniform double drawn from it.

The reference gives every request its own ``std::mt19937_64`` so that a seed
produces the same tokens alone or in a batch (engine/include/llm/scheduler.h:103)
and draws ``std::uniform_real_distribution<double>(0, 1)`` from it
(engine/src/sampler.cpp:49-54).  This is the same generator (Matsumoto and
Nishimura's MT19937-64 with the standard parameters) and the same mapping to a
double: one 64-bit draw divided by 2^64, rounded to nearest, and the largest
double below 1 if that rounds up to 1.
"""
from __future__ import annotations

import math

_NN, _MM = 312, 156
_MATRIX_A = 0xB5026F5AA96619E9
_UPPER, _LOWER = 0xFFFFFFFF80000000, 0x7FFFFFFF
_MASK = 0xFFFFFFFFFFFFFFFF


class MT19937_64:
    def __init__(self, seed: int = 5489):
        self._mt = [0] * _NN
        self._mt[0] = seed & _MASK
        for i in range(1, _NN):
            prev = self._mt[i - 1]
            self._mt[i] = (6364136223846793005 * (prev ^ (prev >> 62)) + i) & _MASK
        self._index = _NN

    def _twist(self) -> None:
        mt = self._mt
        for i in range(_NN):
            x = (mt[i] & _UPPER) | (mt[(i + 1) % _NN] & _LOWER)
            mt[i] = mt[(i + _MM) % _NN] ^ (x >> 1) ^ (_MATRIX_A if x & 1 else 0)
        self._index = 0

    def next_u64(self) -> int:
        if self._index >= _NN:
            self._twist()
        x = self._mt[self._index]
        self._index += 1
        x ^= (x >> 29) & 0x5555555555555555
        x ^= (x << 17) & 0x71D67FFFEDA60000
        x ^= (x << 37) & 0xFFF7EEE000000000
        x ^= x >> 43
        return x & _MASK

    def uniform(self) -> float:
        """A double in [0, 1)."""
        u = self.next_u64() / 18446744073709551616   # exact quotient, rounded once
        return math.nextafter(1.0, 0.0) if u >= 1.0 else u
