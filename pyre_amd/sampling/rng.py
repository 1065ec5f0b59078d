"""A counter-based stream of uniform numbers: the number for (seed, request,
token index) is a pure function of the three, so a request draws the same
numbers whatever else is in its batch and whenever it is scheduled."""

from __future__ import annotations

_MASK = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed: int, request: int, index: int) -> float:
    """A float32-exact number in [0, 1): 24 bits of a hash of the key."""
    h = _splitmix64(seed & _MASK)
    h = _splitmix64(h ^ (request & _MASK))
    h = _splitmix64(h ^ (index & _MASK))
    return (h >> 40) / float(1 << 24)
