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


TEMPLATE_SEEDS = (20250101, 11)


def seeded_template_cases(count: int = 72, seed: int = TEMPLATE_SEEDS[0]):
    """Yields ``(case, GemmConfig, (M, N, K))``: random points of the kernel template's own
    parameter space -- not what the policy would pick -- with a problem size to match: both matrix
    instructions, 1 to 8 waves, 1 to 7 column blocks per wave, K steps of 1 to 8 fragment rounds,
    every pipeline depth, layout, edge mode, access width, remap mode and padding the library
    accepts.  Only configurations that ``rl_gemm_config_check`` accepts are kept."""
    from mlir_roller_amd import hip
    from mlir_roller_amd.hip import GemmConfig

    rng = np.random.default_rng(seed)
    pick = lambda options: options[int(rng.integers(0, len(options)))]
    case = 0
    while case < count:
        mi = pick([16, 32])
        tm, tn = int(rng.integers(1, 5)), int(rng.integers(1, 8))
        waves_m, waves_n = pick([1, 1, 2, 4]), pick([1, 2, 2, 4])
        acc_regs = tm * tn * (16 if mi == 32 else 4)
        if tm * tn > 32 or waves_m * waves_n > 8 or acc_regs > (128 if waves_m * waves_n > 4 else 256):
            continue
        wm, wn = tm * mi, tn * mi
        bm, bn = wm * waves_m, wn * waves_n
        if bm > 384 or bn > 448:
            continue
        bk = (4 * 64 // mi) * pick([1, 1, 2, 2, 3, 4, 8])
        vec, trans_b, accum = pick([4, 4, 1]), pick([0, 0, 1]), pick([0, 0, 1])
        stages = pick([1, 2, 3, 3, 4, 4, 5, 5])
        threads = 64 * waves_m * waves_n
        a_units, b_units = bm * bk // 4, bk * bn // 4
        can_direct = stages >= 3 and vec == 4 and bk & (bk - 1) == 0 and a_units % 64 == 0 and b_units % 64 == 0
        direct = int(can_direct and rng.random() < 0.8)
        if stages > 3 and not (direct and a_units % threads == 0 and b_units % threads == 0):
            stages = 3
        pad_a = 0 if direct else pick([0, 4])
        pad_b = 0 if direct else pick([0, 0, 4])
        swz, group = pick([0, 1, 2, 3, 3]), pick([1, 3, 8])
        M, N, K = int(rng.integers(1, 3 * bm)), int(rng.integers(1, 3 * bn)), int(rng.integers(1, 5 * bk + 1))
        if rng.random() < 0.3:
            M, N, K = -(-M // bm) * bm, -(-N // bn) * bn, -(-K // bk) * bk           # sometimes whole tiles
        elif rng.random() < 0.4:
            K = -(-K // bk) * bk                                                      # only M and N ragged
        if vec == 4:
            N, K = max(4, N // 4 * 4), max(4, K // 4 * 4)
        aligned_mn, aligned_k = M % bm == 0 and N % bn == 0, K % bk == 0
        edge = 1 if not aligned_k else (2 if not aligned_mn else pick([0, 0, 1, 2]))
        cfg = GemmConfig(bm, bn, bk, wm, wn, mi, stages, pad_a, pad_b, vec, edge, swz, group, accum, direct, trans_b)
        try:
            hip.config_check(cfg)
        except hip.HipError:
            continue
        yield case, cfg, (M, N, K)
        case += 1


STREAMK_SEED = 20250911


def seeded_streamk_cases(count: int = 48, seed: int = STREAMK_SEED):
    """Yields ``(case, GemmConfig, (M, N, K))``: the draw of ``seeded_template_cases`` (another seed)
    moved onto the stream-K form of the kernel -- the pipelined loop on two buffers, 1, 2 or 4
    workgroups per CU -- with K lengthened to 3-40 K steps, so that tiles are split from two to
    dozens of ways.  Only configurations that ``rl_gemm_config_check`` accepts are kept."""
    import dataclasses

    from mlir_roller_amd import hip

    rng = np.random.default_rng(seed + 1)
    case = 0
    for _, cfg, (M, N, K) in seeded_template_cases(count=4 * count, seed=seed):
        if case == count:
            break
        sk = dataclasses.replace(cfg, stages=3, streamk=int(rng.choice([1, 2, 2, 4])))
        steps = int(rng.integers(3, 41))
        K = (steps - 1) * cfg.bk + (K - 1) % cfg.bk + 1          # the drawn remainder of the last K step is kept
        if cfg.vec == 4:
            K = max(4, K // 4 * 4)
        if cfg.edge != 1 and K % cfg.bk:
            K = -(-K // cfg.bk) * cfg.bk
        try:
            hip.config_check(sk)
        except hip.HipError:
            continue
        yield case, sk, (M, N, K)
        case += 1



DWORD_DIRECT_SEED = 20251125


def seeded_dword_direct_cases(count: int = 40, seed: int = DWORD_DIRECT_SEED):
    """Yields ``(case, GemmConfig, (M, N, K))``: the draw of ``seeded_template_cases`` (another seed)
    moved onto the direct-to-LDS loads of dword-aligned rows -- vec=1 with direct=1, which means the
    pipelined loop on two buffers, all three extents tested, no padding -- a third of them as stream-K.
    N and K are drawn again, odd ones included; K runs from less than one K step (the tile K ends in
    is the first) over exactly two (no tile is cut short) to a dozen.  Only configurations that
    ``rl_gemm_config_check`` accepts are kept."""
    import dataclasses

    from mlir_roller_amd import hip

    rng = np.random.default_rng(seed + 1)
    case = 0
    for _, cfg, (M, _, _) in seeded_template_cases(count=6 * count, seed=seed):
        if case == count:
            break
        dw = dataclasses.replace(cfg, vec=1, direct=1, stages=3, edge=1, pad_a=0, pad_b=0,
                                 streamk=int(rng.choice([0, 0, 1, 2])))
        N = int(rng.integers(1, 3 * cfg.bn))
        K = int(rng.choice([rng.integers(1, cfg.bk + 1), 2 * cfg.bk, 3 * cfg.bk - 1, rng.integers(1, 12 * cfg.bk)]))
        try:
            hip.config_check(dw)
        except hip.HipError:
            continue
        yield case, dw, (M, N, K)
        case += 1
