"""Writes tests/golden/gemm_exact_cases.json: small integer-valued GEMM problems with their exact
products, computed here with Python integers (a triple loop, no numpy arithmetic).  The reference
holds no vectors for its GEMM payload (/root/reference/src/roller.py:50-62 is checked against
``dA @ dB`` at run time only, :552), so these are first-principles known answers: every value is an
integer far below 2^24, hence exactly representable in float32 and independent of summation order.

    python tests/golden/make_gemm_golden.py
"""

import json
import random
from pathlib import Path

CASES = [("tiny", 3, 4, 2, 9), ("ragged", 37, 53, 29, 9), ("one_row", 1, 70, 33, 5), ("one_col", 65, 1, 40, 5),
         ("k1", 20, 24, 1, 9), ("tile_edge", 66, 68, 20, 7), ("vec4", 32, 48, 24, 9)]


def main() -> None:
    rng = random.Random(20240611)
    out = []
    for name, m, n, k, amp in CASES:
        a = [[rng.randint(-amp, amp) for _ in range(k)] for _ in range(m)]
        b = [[rng.randint(-amp, amp) for _ in range(n)] for _ in range(k)]
        c = [[sum(a[i][p] * b[p][j] for p in range(k)) for j in range(n)] for i in range(m)]
        assert max(abs(v) for row in c for v in row) < 2 ** 24
        out.append({"name": name, "M": m, "N": n, "K": k, "A": a, "B": b, "C": c})
    path = Path(__file__).resolve().parent / "gemm_exact_cases.json"
    path.write_text(json.dumps(out, separators=(",", ":")))
    print(f"{path}: {len(out)} cases, {path.stat().st_size} bytes")


if __name__ == "__main__":
    main()
