"""Writes tests/golden/policy_a100.json: input/output vectors of the reference's rTile policy.

Run once, in the build container, where /root/reference is mounted:

    python tests/golden/make_policy_golden.py

The reference's pure-Python policy (/root/reference/src/analyze.py, arch.py, utils.py) is
imported -- not copied -- and evaluated on its own ``CUDA()`` device model for the shapes the
benchmark uses.  What is recorded is data only: for every shape the complete ordered top-20 hint
list (block tile, thread tile, reduce step and every analysis field), the head of the ranked
block-tile list, the ordered block-size recommendation for a few tiles, and the integer helpers
on a set of arguments.  Hand-derived known answers cover only the head of these lists; the
complete order depends on stable-sort ties and float tie-breaks that only the reference itself
can fix, which is why these vectors exist.

``humanize`` (used by the reference solely inside ``TileDict.__repr__``, analyze.py:110-118) is
not installed here; an empty placeholder module satisfies the import and is never called.
Nothing under tests/ or the package imports this script or the reference at test time: the
tests read the JSON.
"""

from __future__ import annotations

import itertools
import json
import sys
import types
from pathlib import Path

REFERENCE_SRC = Path("/root/reference/src")
OUT = Path(__file__).resolve().parent / "policy_a100.json"

README_SHAPES = [
    (2048, 2048, 2048), (2048, 2048, 8192), (2048, 4096, 2048), (2048, 4096, 4096),
    (2048, 8192, 2048), (2048, 8192, 4096), (2048, 8192, 8192), (4096, 2048, 2048),
    (4096, 4096, 8192), (4096, 8192, 2048), (4096, 8192, 4096), (8192, 2048, 8192),
    (8192, 4096, 2048), (8192, 4096, 4096),
]
EXTRA_SHAPES = [(3000, 5000, 1536), (4096, 4096, 4096), (8192, 8192, 8192), (1024, 768, 512),
                (96, 80, 48), (127, 131, 67)]


TILE_FIELDS = ["block_m", "block_n", "thread_m", "thread_n", "rstep", "traffic", "smem_cost",
               "block_per_SM", "num_wave", "grid_size"]


def tile_record(td) -> list:
    """One TileDict as a row; column names are in ``TILE_FIELDS`` (thread tile 0, 0 = unset)."""
    thread = list(td.thread_tile) or [0, 0]
    return [int(v) for v in (*td.block_tile, *thread, td.rstep, td.traffic, td.smem_cost,
                             td.block_per_SM, td.num_wave, td.grid_size)]


def main() -> None:
    sys.modules.setdefault("humanize", types.ModuleType("humanize"))
    sys.path.insert(0, str(REFERENCE_SRC))
    import analyze as ref_analyze  # noqa: E402
    import arch as ref_arch  # noqa: E402
    import utils as ref_utils  # noqa: E402

    golden = {"source": "NaOHCC/mlir-roller src/analyze.py on CUDA() (A100 model)", "tile_fields": TILE_FIELDS, "shapes": [], "utils": {}}

    for m, n, k in README_SHAPES + EXTRA_SHAPES:
        config = ref_analyze.MatmulConfig(M=m, N=n, K=k, el_bits=32)
        arch = ref_arch.CUDA()
        policy = ref_analyze.Policy(config, arch)
        base_rstep = policy._assign_reduce_step()
        ranked = policy.get_block_tiles_candidates([1, 1], base_rstep)
        hints = ref_analyze.get_roller_hints(config, ref_arch.CUDA(), topk=20)
        block_sizes = {}
        for tile in ([128, 128], [64, 64], [64, 256], [32, 96]):
            td = ref_analyze.TileDict.from_block_tile(tile, base_rstep, config, arch)
            if td.valid:
                block_sizes["x".join(map(str, tile))] = [int(b) for b in policy.recommend_block_size(td)]
        golden["shapes"].append({
            "M": m, "N": n, "K": k,
            "base_rstep": int(base_rstep),
            "reduce_step_candidates": [int(s) for s in policy.get_reduce_step_candidates(k)],
            "n_valid_block_tiles": len(ranked),
            "ranked_block_tiles": [tile_record(td) for td in ranked[:40]],
            "block_sizes": block_sizes,
            "hints": [tile_record(td) for td in hints],
        })

    u = golden["utils"]
    ns = [1, 2, 3, 4, 12, 36, 64, 97, 128, 360, 1536, 2048, 3000, 4096, 5000, 8192, 16384, 65536]
    u["get_all_factors"] = {str(x): ref_utils.get_all_factors(x) for x in ns}
    u["factorize"] = {str(x): ref_utils.factorize(x) for x in ns}
    cases = []
    fulls = [[2048, 2048], [3000, 1536], [8, 8], [5000, 3000]]
    for full in fulls:
        for sub in itertools.product([1, 4, 8, 128, full[0]], [1, 4, 32, full[1]]):
            sub = [min(sub[0], full[0]), min(sub[1], full[1])]
            for txn in (8, 32):
                cases.append({"sub": sub, "full": full, "txn": txn,
                              "factor": int(ref_utils.coalesced_factor(sub, full)),
                              "shape": int(ref_utils.coalesced_tensor_shape(sub, full, txn))})
    u["coalesced"] = cases
    u["get_block_dims"] = [
        {"block": b, "reg": r, "dims": ref_utils.get_block_dims(list(b), list(r))}
        for b, r in ([[128, 128, 0], [16, 8, 0]], [[64, 256, 0], [16, 8, 0]], [[64, 64, 0], [8, 8, 0]],
                     [[32, 96, 16], [4, 0, 2]])
    ]
    traffic = []
    for (m, n, k), tile in itertools.product([(2048, 2048, 2048), (4096, 8192, 4096), (3000, 5000, 1536)],
                                             [[128, 128], [64, 4], [1, 1], [256, 64], [2048, 2048], [8, 5000]]):
        config = ref_analyze.MatmulConfig(M=m, N=n, K=k, el_bits=32)
        traffic.append({"M": m, "N": n, "K": k, "tile": tile,
                        "bytes": int(ref_analyze.compute_memory_traffic(tile, config, ref_arch.CUDA()))})
    u["compute_memory_traffic"] = traffic

    OUT.write_text(json.dumps(golden, separators=(",", ":")).replace('{"M"', '\n{"M"') + "\n")
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes)")


if __name__ == "__main__":
    main()
