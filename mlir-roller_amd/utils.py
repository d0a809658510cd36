"""Integer helpers of the rTile policy.

Same names, arguments and results as /root/reference/src/utils.py (get_all_factors :6-17,
factorize :20-31, coalesced_factor :34-40, coalesced_tensor_shape :44-57, get_block_dims :60-69);
written independently with plain integer arithmetic (the reference goes through numpy floats).
"""

from __future__ import annotations

import math
from typing import List, Sequence


def get_all_factors(n: int) -> List[int]:
    """All positive divisors of ``n`` in ascending order."""
    if n < 1:
        raise ValueError(f"get_all_factors needs a positive integer, got {n}")
    low, high = [], []
    for d in range(1, math.isqrt(n) + 1):
        if n % d == 0:
            low.append(d)
            if d != n // d:
                high.append(n // d)
    return low + high[::-1]


def factorize(n: int) -> List[int]:
    """Prime factors of ``n`` with multiplicity, ascending (``factorize(12) == [2, 2, 3]``)."""
    primes: List[int] = []
    p = 2
    while n > 1:
        while n % p == 0:
            primes.append(p)
            n //= p
        p += 1
    return primes


def coalesced_factor(subtensor: Sequence[int], tensor: Sequence[int]) -> int:
    """Length, in elements, of the longest contiguous run that a row-major ``subtensor`` of
    ``tensor`` occupies: trailing dimensions multiply in for as long as the sub-tensor spans the
    full extent; the first dimension that does not (or the outermost one) ends the run."""
    run = 1
    for sub_extent, full_extent in zip(reversed(subtensor), reversed(tensor)):
        run *= sub_extent
        if sub_extent != full_extent:
            break
    return run


def coalesced_tensor_shape(subtensor: Sequence[int], tensor: Sequence[int], transaction_size: int) -> int:
    """Elements actually moved when ``subtensor`` is fetched in transactions of
    ``transaction_size`` elements: runs shorter than a transaction are rounded up to one."""
    elements = math.prod(subtensor)
    if elements == 0:
        return 0
    run = coalesced_factor(subtensor, tensor)
    return transaction_size * elements // min(transaction_size, run)


def get_block_dims(block_tile: Sequence[int], reg_tile: Sequence[int]) -> List[int]:
    """Thread-block extents ``[x, y, z]`` for a block tile split into per-thread tiles.  Tile
    vectors are ``[m, n, k]`` with x running along n, hence the swap of the first two entries;
    a zero on either side means "not tiled" and yields 1."""
    dims = [b // r if b != 0 and r != 0 else 1 for b, r in zip(block_tile, reg_tile)]
    dims[0], dims[1] = dims[1], dims[0]
    return dims
