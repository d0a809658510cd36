"""The stream-K work split, checked by brute force on the host.

``rl_gemm_streamk_segments`` runs, for one workgroup index, the very code the kernel's workgroups run
(csrc/gemm_sk_decode.inc is compiled into the library and into every stream-K kernel).  Walking all
workgroups of a launch must hand out every K step of every tile exactly once: the full rounds of
tiles whole, one tile per workgroup and round (neighbouring tiles at the same time), the rest in pieces
that belong to consecutive workgroups in K order, each in a workspace slot of its own -- which is what
makes the sum of a split tile independent of which workgroup finishes last."""

import random

import pytest

from mlir_roller_amd import hip
from mlir_roller_amd.hip import GemmConfig


@pytest.fixture(scope="module")
def lib():
    if not hip.LIB_PATH.exists():
        hip.build_library()
    return hip.lib()


def sk_config(bm, bn, bk, wm, wn, mi, edge, streamk=2, group=8, swz=3):
    return GemmConfig(bm, bn, bk, wm, wn, mi, 3, 0, 0, 4, edge, swz, group, 0, 1, 0, streamk)


CASES = [
    # (config, (M, N, K), compute units)
    (sk_config(96, 160, 32, 48, 80, 16, 2), (3000, 5000, 1536), 256),
    (sk_config(96, 160, 32, 48, 80, 16, 2, streamk=1), (3000, 5000, 1536), 256),
    (sk_config(128, 128, 32, 64, 64, 16, 0), (2048, 2048, 2048), 256),
    (sk_config(128, 128, 32, 64, 64, 16, 0), (1536, 1536, 1536), 256),       # 144 tiles on 512 workgroups
    (sk_config(128, 128, 32, 64, 64, 16, 2), (1000, 1000, 1024), 256),
    (sk_config(64, 64, 32, 32, 32, 16, 1), (1000, 1000, 1000), 256),
    (sk_config(64, 320, 32, 16, 320, 16, 2, streamk=1), (3000, 5000, 1536), 256),
    (sk_config(256, 256, 32, 128, 128, 32, 2, streamk=1), (3000, 5000, 1536), 256),
    (sk_config(128, 128, 32, 64, 64, 16, 1), (130, 130, 40), 256),           # fewer units than workgroups
    (sk_config(32, 32, 16, 32, 32, 16, 1, streamk=8), (37, 53, 29), 256),
    (sk_config(128, 64, 32, 64, 32, 16, 2, group=3), (1100, 900, 512), 7),   # odd CU count, short last panel
    (sk_config(128, 64, 32, 64, 32, 16, 2, swz=1), (1100, 900, 512), 304),
    (sk_config(96, 96, 32, 48, 48, 16, 2), (96 * 5 + 1, 96 * 7 + 95, 32 * 9), 16),
    (sk_config(128, 96, 32, 64, 48, 16, 1), (4095, 4097, 4093), 256),        # 1376 tiles on 512 workgroups: two rounds whole, 352 tiles shared
    (sk_config(64, 160, 32, 32, 80, 16, 0), (8192, 8192, 8192), 256),        # 6656 tiles = 13 rounds, nothing shared
    (sk_config(64, 64, 32, 32, 32, 16, 1, streamk=1), (1000, 1000, 1000), 60),   # 256 tiles on 60: four rounds whole, 16 tiles shared
]


def all_segments(cfg, shape, cus):
    sched = hip.streamk_schedule(cfg, *shape, compute_units=cus)
    return sched, [hip.streamk_segments(cfg, *shape, wg, compute_units=cus) for wg in range(sched.grid)]


@pytest.mark.parametrize("cfg,shape,cus", CASES, ids=lambda v: v.tag() if isinstance(v, GemmConfig) else str(v))
def test_every_k_step_of_every_tile_is_handed_out_once(lib, cfg, shape, cus):
    M, N, K = shape
    sched, per_wg = all_segments(cfg, shape, cus)
    nbm, nbn, kt = -(-M // cfg.bm), -(-N // cfg.bn), -(-K // cfg.bk)
    assert (sched.tile_rows, sched.tile_cols, sched.k_steps, sched.tiles, sched.units) == (nbm, nbn, kt, nbm * nbn, nbm * nbn * kt)
    assert sched.grid == min(cus * cfg.streamk, sched.units)
    # the full rounds of the grid are worked whole -- all but one if the tiles left over are fewer than a
    # quarter of the grid (or have fewer K steps than there are workgroups)
    rounds, left = divmod(sched.tiles, sched.grid)
    assert sched.whole_tiles == sched.grid * (rounds - 1 if rounds and left and (4 * left < sched.grid or left * kt < sched.grid) else rounds)
    covered, tile_number, pieces_of = {}, {}, {}
    for wg, segs in enumerate(per_wg):
        assert segs, f"workgroup {wg} has no work"            # the decoding of pieces relies on it
        # its share of the tiles that are shared out comes first, then its whole tiles: tile round * grid + wg
        shared = [s for s in segs if s.tile >= sched.whole_tiles]
        assert [s.tile for s in segs[:len(shared)]] == [s.tile for s in shared]
        assert [(s.tile, s.k_begin, s.k_end, s.pieces) for s in segs[len(shared):]] == \
            [(t, 0, kt, 1) for t in range(wg, sched.whole_tiles, sched.grid)]
        assert bool(shared) == (sched.whole_tiles < sched.tiles)
        for i, s in enumerate(segs):
            assert 0 <= s.tile_m < nbm and 0 <= s.tile_n < nbn and 0 <= s.k_begin < s.k_end <= kt
            assert tile_number.setdefault((s.tile_m, s.tile_n), s.tile) == s.tile and 0 <= s.tile < sched.tiles
            for k in range(s.k_begin, s.k_end):
                assert (s.tile_m, s.tile_n, k) not in covered
                covered[(s.tile_m, s.tile_n, k)] = wg
            pieces_of.setdefault((s.tile_m, s.tile_n), []).append((wg, i, len(shared), s))
    assert len(covered) == nbm * nbn * kt                       # nothing left out ...
    assert sum(s.k_end - s.k_begin for segs in per_wg for s in segs) == nbm * nbn * kt   # ... and nothing twice
    assert len(set(tile_number.values())) == nbm * nbn          # one arrival counter per tile
    used_slots = set()
    for (tm, tn), plist in pieces_of.items():
        plist.sort(key=lambda e: e[3].k_begin)
        first_wg = plist[0][0]
        assert plist[0][3].k_begin == 0 and plist[-1][3].k_end == kt
        for j, (wg, i, n, s) in enumerate(plist):
            assert wg == first_wg + j                           # consecutive workgroups, in K order
            assert s.pieces == len(plist) and s.first_workgroup == first_wg
            if j:
                assert s.k_begin == plist[j - 1][3].k_end
            if len(plist) == 1:
                assert s.slot == -1
            else:
                # the slot the reader computes for piece j: 2*first+1 for the first, 2*(first+j) after it
                assert s.slot == (2 * first_wg + 1 if j == 0 else 2 * (first_wg + j))
                assert s.slot not in used_slots and 0 <= s.slot < 2 * sched.grid
                used_slots.add(s.slot)
                # a piece that starts inside a tile is its workgroup's first segment; one that starts a
                # tile and does not finish it is the last of its share
                assert (i == 0) if s.k_begin else (i == n - 1)
    assert sched.workspace_bytes == sched.counter_bytes + 2 * sched.grid * cfg.bm * cfg.bn * 4
    assert sched.counter_bytes >= 4 * sched.tiles and sched.counter_bytes % 256 == 0


@pytest.mark.parametrize("cfg,shape,cus", CASES, ids=lambda v: v.tag() if isinstance(v, GemmConfig) else str(v))
def test_shares_are_equal_to_within_one_k_step(lib, cfg, shape, cus):
    sched, per_wg = all_segments(cfg, shape, cus)
    shares = [sum(s.k_end - s.k_begin for s in segs) for segs in per_wg]
    assert sum(shares) == sched.units and max(shares) - min(shares) <= 1


def test_tiles_are_walked_in_panels(lib):
    # panel of 3 tile rows over a 9 x 15 tile grid: consecutive tiles go down a panel's column first
    cfg = sk_config(128, 64, 32, 64, 32, 16, 2, group=3)
    where = {}
    for wg in range(hip.streamk_schedule(cfg, 1100, 900, 512, 7).grid):
        for s in hip.streamk_segments(cfg, 1100, 900, 512, wg, 7):
            assert where.setdefault(s.tile, (s.tile_m, s.tile_n)) == (s.tile_m, s.tile_n)
    order = [where[t] for t in range(len(where))]
    assert order[:7] == [(0, 0), (1, 0), (2, 0), (0, 1), (1, 1), (2, 1), (0, 2)] and order[45] == (3, 0) and len(order) == 9 * 15


def test_random_problems(lib):
    rng = random.Random(7)
    tiles = [(128, 128, 64, 64, 16), (64, 128, 32, 64, 16), (256, 128, 128, 64, 32), (96, 160, 48, 80, 16), (32, 64, 32, 32, 16)]
    for _ in range(25):
        bm, bn, wm, wn, mi = rng.choice(tiles)
        shape = (rng.randint(1, 1500), rng.randint(1, 1500), rng.randint(1, 700))
        cfg = sk_config(bm, bn, 32, wm, wn, mi, 1, streamk=rng.choice([1, 2, 4]), group=rng.choice([1, 4, 8]))
        cus = rng.choice([1, 8, 60, 256])
        test_every_k_step_of_every_tile_is_handed_out_once(None, cfg, shape, cus)
        test_shares_are_equal_to_within_one_k_step(None, cfg, shape, cus)


def test_rejects_what_it_cannot_split(lib):
    cfg = sk_config(128, 128, 32, 64, 64, 16, 1)
    with pytest.raises(hip.HipError):
        hip.streamk_schedule(cfg, 0, 128, 128)
    with pytest.raises(hip.HipError):
        hip.streamk_schedule(GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 0), 128, 128, 128)   # not stream-K
    with pytest.raises(hip.HipError):
        hip.config_check(GemmConfig(128, 128, 32, 64, 64, 16, 2, 4, 0, 4, 1, 3, 8, 0, 0, 0, 2))   # needs the pipelined loop
