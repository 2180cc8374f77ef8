"""Choice of the Hadamard routine for a width (reference: quantize/hadamard_helpers.py)."""
from __future__ import annotations

import math

from .. import ops


def is_pow2(n: int) -> bool:
    return n > 0 and n & (n - 1) == 0


def next_power_of_two(x: int) -> int:
    return 1 if x == 0 else 2 ** (x - 1).bit_length()


def prev_power_of_two(x: int) -> int:
    return 0 if x < 1 else 2 ** (x.bit_length() - 1)


def get_had_fn(dim: int):
    """(transform, base N, scale): widths 40*2^k, 28*2^k, 20*2^k, 12*2^k pick the
    composite variants, every other width must be a power of two
    (hadamard_helpers.py:18-36)."""
    scale = 1.0 / math.sqrt(dim)
    for base in (40, 28, 20, 12):
        if dim % base == 0 and is_pow2(dim // base):
            return ops.composite_hadamard_variant(base), base, scale
    assert is_pow2(dim), f"Invalid dim: {dim}. dim must be a power of 2."
    return ops.fast_hadamard_transform, 2, scale


def had_transform(w):
    """Rotates the last axis of a weight; returns a new tensor (hadamard_helpers.py:39-48)."""
    shape = w.shape
    fn, _, scale = get_had_fn(shape[-1])
    return fn(w.reshape(-1, shape[-1]), scale).reshape(shape)
