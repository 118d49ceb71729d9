"""Counter-based uniform numbers: u = f(seed, counter), no state to carry."""

from __future__ import annotations

_MASK = (1 << 64) - 1


def _mix(x: int) -> int:
    """One round of the splitmix64 finaliser."""
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed: int, counter: int) -> float:
    """A number in [0, 1) with 24 random bits (exact in float32), fixed by (seed, counter)."""
    value = _mix(_mix(seed & _MASK) ^ ((counter * 0xD1B54A32D192ED03) & _MASK))
    return (value >> 40) / float(1 << 24)
