"""Integer helpers (reference: spio/util/math.py:6-21)."""

from math import gcd


def divup(n: int, d: int) -> int:
    """Ceiling of n / d for positive d."""
    return -(-n // d)


def next_relative_prime(a: int, b: int) -> int:
    """Smallest r >= a with gcd(r, b) == 1.

    Used to pick LDS strides that do not alias banks.
    """
    r = a
    limit = a + max(b, 1)
    while r <= limit:
        if gcd(r, b) == 1:
            return r
        r += 1
    raise AssertionError(f"no number coprime to {b} in [{a}, {limit}]")
