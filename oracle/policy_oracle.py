"""Oracle of the reference's rTile policy -- TEST INFRASTRUCTURE, not product code.

A second, deliberately plain restatement of /root/reference/src/analyze.py + utils.py + arch.py
(functions over dicts and tuples, brute-force divisor search, no classes), used by the tests to
cross-check ``mlir_roller_amd.analyze`` on its ``CUDA()`` device model over many shapes.  It
shares no code with the product.  Itself it is pinned by tests/golden/policy_a100.json (vectors
written by the reference's own code) and by hand-derived known answers (tests/test_policy.py).

Only ``tests/`` may import this module.
"""

from __future__ import annotations

import math
from itertools import product
from typing import Dict, List, Optional

# The reference's A100 description (arch.py:41-61).
A100 = {
    "reg_cap": 65536, "smem_cap": 64 * 1024, "cores": 108, "warp": 32, "partitions": 4,
    "max_smem": 2 * 64 * 1024, "write_txn_bytes": 32, "read_txn_bytes": 128, "smem_bw": 12080,
}
EL_BYTES = 4  # fp32: (32 + 7) // 8, analyze.py:39-41


def divisors(n: int) -> List[int]:
    """utils.py:6-17 by trial division."""
    return [d for d in range(1, n + 1) if n % d == 0]


def divisors_upto(n: int, limit: int) -> List[int]:
    return [d for d in range(1, min(n, limit) + 1) if n % d == 0]


def run_length(sub: List[int], full: List[int]) -> int:
    """utils.py:34-40, recursive as written there."""
    if sub[-1] != full[-1] or len(sub) == 1:
        return sub[-1]
    return sub[-1] * run_length(sub[:-1], full[:-1])


def moved_elements(sub: List[int], full: List[int], txn: int) -> int:
    """utils.py:44-57."""
    count = math.prod(sub)
    return 0 if count == 0 else txn * count // min(txn, run_length(sub, full))


def tile_traffic(m: int, n: int, M: int, N: int, K: int, dev=A100) -> int:
    """analyze.py:62-81: operand panels [m,K] of [M,K] and [n,K] of [N,K], output [m,n] of [M,N]."""
    rte, wte = dev["read_txn_bytes"] // EL_BYTES, dev["write_txn_bytes"] // EL_BYTES
    elems = moved_elements([m, K], [M, K], rte) + moved_elements([n, K], [N, K], rte)
    elems += moved_elements([m, n], [M, N], wte)
    return elems * EL_BYTES


def analyse_tile(m: int, n: int, rstep: int, M: int, N: int, K: int, dev=A100) -> Optional[Dict]:
    """analyze.py:125-168; None where the reference marks the tile invalid."""
    smem = rstep * (m + n) * EL_BYTES
    if smem > dev["smem_cap"]:
        return None
    regs = int(2 * m * n * EL_BYTES / 32)
    if regs > dev["reg_cap"]:
        return None
    grid = math.ceil(M / m) * math.ceil(N / n)
    per_core = min(dev["max_smem"] // max(smem, 1), dev["reg_cap"] // max(regs, 1), dev["partitions"])
    return {
        "block_tile": [m, n], "thread_tile": [], "rstep": rstep, "traffic": tile_traffic(m, n, M, N, K, dev),
        "smem_cost": smem, "block_per_SM": per_core, "grid_size": grid,
        "num_wave": math.ceil(grid / (per_core * dev["cores"])),
    }


def reduce_steps(K: int) -> List[int]:
    """analyze.py:203-215."""
    d = divisors(K)
    if len(d) == 2 and K > 64:
        d = [1]
        while d[-1] * 2 < K:
            d.append(d[-1] * 2)
    return d


def base_reduce_step(M: int, N: int, K: int, dev=A100) -> int:
    """analyze.py:217-221 with tile [1, 1]: each operand tile [1, s] is scored by
    2ab/(a^2+b^2) of its contiguous run against the read transaction; the first maximum wins."""
    rte = dev["read_txn_bytes"] // EL_BYTES
    best, best_score = None, -1.0
    for s in reduce_steps(K):
        score = 0.0
        for spatial in (M, N):
            run = run_length([1, s], [spatial, K])
            score += (2 * run * rte) / (run * run + rte * rte)
        if score > best_score:
            best, best_score = s, score
    return best


def tile_sizes(extent: int) -> List[int]:
    """analyze.py:226-239 with init tile 1."""
    return sorted(set(divisors(extent)) | {s for s in (2, 4, 8, 16, 32) if 1 < s < extent})


def ranked_tiles(M: int, N: int, K: int, dev=A100) -> List[Dict]:
    """analyze.py:223-255: product order (m outer), valid only, stable sort by (traffic+1)*waves."""
    rstep = base_reduce_step(M, N, K, dev)
    tiles = [t for m, n in product(tile_sizes(M), tile_sizes(N))
             if (t := analyse_tile(m, n, rstep, M, N, K, dev)) is not None]
    return sorted(tiles, key=lambda t: (t["traffic"] + 1) * t["num_wave"])


def grow_reduce_step(tile: Dict, M: int, N: int, K: int, dev=A100) -> None:
    """analyze.py:257-277."""
    m, n = tile["block_tile"]
    limit = min(dev["max_smem"] // tile["block_per_SM"], dev["smem_cap"])
    steps = [s for s in reduce_steps(K) if s % tile["rstep"] == 0 and s * (m + n) * EL_BYTES <= limit]
    if not steps:
        steps = [tile["rstep"]]
    best, best_score = None, -1
    for s in steps:
        score = run_length([m, s], [M, K]) + run_length([n, s], [N, K])
        if score > best_score:
            best, best_score = s, score
    tile["rstep"] = best
    tile["smem_cost"] = best * (m + n) * EL_BYTES


def block_sizes(m: int, n: int, dev=A100) -> List[int]:
    """analyze.py:279-308."""
    def score(t):
        warps = (t + dev["warp"] - 1) // dev["warp"]
        return (max(warps / dev["partitions"], dev["partitions"] / warps), (warps * dev["warp"] - t) / t)
    return sorted(divisors_upto(m * n, 1024), key=score)


def thread_tile(m: int, n: int, threads: int, K: int, dev=A100) -> Optional[List[int]]:
    """analyze.py:329-365."""
    area = (m * n) // threads
    pairs = [[area // i, i] for i in range(1, int(math.sqrt(area)) + 1) if area % i == 0]
    best = sorted(pairs, key=lambda p: p[0] * K / dev["smem_bw"] + p[1] * K / dev["smem_bw"])[0]
    if int(best[0] * best[1] * EL_BYTES / 4) >= 256:
        return None
    return best


def hints(M: int, N: int, K: int, topk: int = 10, dev=A100) -> List[Dict]:
    """analyze.py:367-381 (emit_config) with assign_thread_tile(td, 2) of :310-327 inlined:
    at most two block sizes per tile, and the first untileable block size ends that tile."""
    out: List[Dict] = []
    for tile in ranked_tiles(M, N, K, dev):
        grow_reduce_step(tile, M, N, K, dev)
        taken = 0
        for threads in block_sizes(*tile["block_tile"], dev):
            tt = thread_tile(*tile["block_tile"], threads, K, dev)
            if tt is None:
                break
            out.append({**tile, "block_tile": list(tile["block_tile"]), "thread_tile": tt})
            taken += 1
            if len(out) >= topk:
                return out
            if taken == 2:
                break
    return out
