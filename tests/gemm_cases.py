"""Seeded random problems for the GPU parity tests: shape, pipeline depth, operand layout,
accumulate mode and which of the policy's first two hints to take.  Kept apart from the tests so
that the build step can compile the same kernel configurations ahead of time."""

import numpy as np

# vectors, slivers and a very long K, as (M, N, K)
EXTREME_SHAPES = [(1, 1, 1), (1, 7, 3), (100000, 8, 64), (8, 100000, 64), (64, 64, 100000), (65536, 128, 128),
                  (3, 50000, 5), (50000, 3, 5), (257, 255, 1023), (4096, 4, 4096), (4, 4096, 4096), (1, 4096, 4096),
                  (4096, 1, 4096)]


def seeded_policy_cases(arch, count: int = 40, seed: int = 20240607):
    """Yields ``(case, matmul_config, hint, depth, trans_b, accumulate)``; ragged and tiny
    shapes, K and N odd or multiples of 4, a quarter of them tile-aligned."""
    from mlir_roller_amd.analyze import MatmulConfig, get_roller_hints

    rng = np.random.default_rng(seed)
    for case in range(count):
        M, N, K = int(rng.integers(1, 700)), int(rng.integers(1, 700)), int(rng.integers(1, 600))
        if rng.random() < 0.5:
            N, K = max(4, N // 4 * 4), max(4, K // 4 * 4)                       # eligible for 128-bit accesses
        if rng.random() < 0.25:
            M, N, K = -(-M // 64) * 64, -(-N // 64) * 64, -(-K // 32) * 32      # often tile-aligned
        depth, trans_b, accumulate = int(rng.integers(1, 4)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        config = MatmulConfig(M, N, K, 32)
        hints = get_roller_hints(config, arch, topk=2)
        if not hints:
            raise AssertionError(f"no hints for {(M, N, K)}")
        yield case, config, hints[int(rng.integers(0, len(hints)))], depth, trans_b, accumulate
