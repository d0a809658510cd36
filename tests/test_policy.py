"""Host policy: mlir_roller_amd.{utils,arch,analyze}.

Three layers of evidence that the product policy means what the reference's means:
  1. golden vectors written by the reference's own code on its A100 model
     (tests/golden/policy_a100.json): complete ordered top-20 hint lists for M0..M13 and six more
     shapes, ranked block tiles, block-size orders, and the integer helpers;
  2. known answers derived by hand from the reference's source (closed forms, first hint);
  3. an independent plain restatement (oracle/policy_oracle.py), itself pinned by (1), compared
     with the product on shapes the fixture does not hold.
Then the MI355X model: MFMA-aligned tiles, wave tiles, resource limits, ranking sanity.
"""

import itertools
import math
import random

import pytest

from mlir_roller_amd import analyze, utils
from mlir_roller_amd.analyze import MatmulConfig, Policy, TileDict, get_roller_hints
from mlir_roller_amd.arch import CUDA, MI355X, TileDevice
from mlir_roller_amd.roller import hint_to_gemm_config
from oracle import policy_oracle as po


def row(td):
    thread = list(td.thread_tile) or [0, 0]
    return [*td.block_tile, *thread, td.rstep, td.traffic, td.smem_cost, td.block_per_SM, td.num_wave, td.grid_size]


def orow(d):
    thread = list(d["thread_tile"]) or [0, 0]
    return [*d["block_tile"], *thread, d["rstep"], d["traffic"], d["smem_cost"], d["block_per_SM"], d["num_wave"], d["grid_size"]]


# ---- 1. golden vectors from the reference ----------------------------------------------------

def test_integer_helpers_match_reference_vectors(golden_policy):
    u = golden_policy["utils"]
    for n, expect in u["get_all_factors"].items():
        assert utils.get_all_factors(int(n)) == expect
        assert po.divisors(int(n)) == expect
    for n, expect in u["factorize"].items():
        assert utils.factorize(int(n)) == expect
    for case in u["coalesced"]:
        assert utils.coalesced_factor(case["sub"], case["full"]) == case["factor"]
        assert utils.coalesced_tensor_shape(case["sub"], case["full"], case["txn"]) == case["shape"]
        assert po.run_length(case["sub"], case["full"]) == case["factor"]
        assert po.moved_elements(case["sub"], case["full"], case["txn"]) == case["shape"]
    for case in u["get_block_dims"]:
        assert utils.get_block_dims(case["block"], case["reg"]) == case["dims"]
    for case in u["compute_memory_traffic"]:
        cfg = MatmulConfig(case["M"], case["N"], case["K"], 32)
        assert analyze.compute_memory_traffic(case["tile"], cfg, CUDA()) == case["bytes"]
        assert po.tile_traffic(*case["tile"], case["M"], case["N"], case["K"]) == case["bytes"]


def test_product_policy_reproduces_reference_hints(golden_policy):
    assert len(golden_policy["shapes"]) == 20
    for sh in golden_policy["shapes"]:
        cfg = MatmulConfig(sh["M"], sh["N"], sh["K"], 32)
        policy = Policy(cfg, CUDA())
        assert policy._assign_reduce_step() == sh["base_rstep"]
        assert policy.get_reduce_step_candidates(sh["K"]) == sh["reduce_step_candidates"]
        ranked = policy.get_block_tiles_candidates([1, 1], sh["base_rstep"])
        assert len(ranked) == sh["n_valid_block_tiles"]
        assert [row(t) for t in ranked[:40]] == sh["ranked_block_tiles"]
        for name, order in sh["block_sizes"].items():
            tile = [int(v) for v in name.split("x")]
            td = TileDict.from_block_tile(tile, sh["base_rstep"], cfg, CUDA())
            assert policy.recommend_block_size(td) == order
        hints = get_roller_hints(cfg, CUDA(), topk=20)
        assert [row(h) for h in hints] == sh["hints"], (sh["M"], sh["N"], sh["K"])


def test_policy_oracle_reproduces_reference_hints(golden_policy):
    for sh in golden_policy["shapes"]:
        M, N, K = sh["M"], sh["N"], sh["K"]
        assert po.base_reduce_step(M, N, K) == sh["base_rstep"]
        ranked = po.ranked_tiles(M, N, K)
        assert len(ranked) == sh["n_valid_block_tiles"]
        assert [orow(t) for t in ranked[:40]] == sh["ranked_block_tiles"]
        assert [orow(h) for h in po.hints(M, N, K, 20)] == sh["hints"]
        for name, order in sh["block_sizes"].items():
            assert po.block_sizes(*[int(v) for v in name.split("x")]) == order


# ---- 2. hand-derived known answers ---------------------------------------------------------------

def test_closed_form_traffic():
    # n >= 8 write-transaction elements: 4 * (K*(m+n) + m*n)
    for (M, N, K), (m, n) in itertools.product([(2048, 2048, 2048), (4096, 8192, 4096)], [(128, 128), (64, 256), (32, 8)]):
        cfg = MatmulConfig(M, N, K, 32)
        assert analyze.compute_memory_traffic([m, n], cfg, CUDA()) == 4 * (K * (m + n) + m * n)
    # narrower than a write transaction: each row of the tile costs a whole transaction (8 elems)
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    assert analyze.compute_memory_traffic([64, 4], cfg, CUDA()) == 4 * (2048 * 68 + 8 * 64)


def test_hand_derived_tile_analysis_a100():
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    expect = {
        (128, 128): (2162688, 32768, 4, 256, 1),
        (64, 256): (2686976, 40960, 3, 256, 1),
        (64, 64): (1064960, 16384, 4, 1024, 3),
        (64, 128): (1605632, 24576, 4, 512, 2),
        (128, 256): (3276800, 49152, 2, 128, 1),
        (256, 256): (4456448, 65536, 2, 64, 1),
    }
    for tile, (traffic, smem, bps, grid, waves) in expect.items():
        td = TileDict.from_block_tile(list(tile), 32, cfg, CUDA())
        assert td.valid
        assert (td.traffic, td.smem_cost, td.block_per_SM, td.grid_size, td.num_wave) == (traffic, smem, bps, grid, waves)
    assert not TileDict.from_block_tile([512, 1], 32, cfg, CUDA()).valid  # 128 * 513 bytes > 64 KiB
    big = TileDict.from_block_tile([4096, 8192], 1, MatmulConfig(8192, 8192, 64, 32), CUDA())
    assert not big.valid and big.traffic == -1  # register estimate over the cap, analysis left unset


def test_first_hint_a100_is_the_documented_one():
    for shape in [(2048, 2048, 2048), (2048, 2048, 8192), (4096, 8192, 4096)]:
        h = get_roller_hints(MatmulConfig(*shape, 32), CUDA(), topk=1)[0]
        assert (h.block_tile, h.thread_tile, h.rstep, h.smem_cost, h.block_per_SM) == ([128, 128], [16, 8], 32, 32768, 4)
        assert utils.get_block_dims(h.block_tile + [0], h.thread_tile + [0]) == [16, 8, 1]


def test_reduce_step_expansion_and_thread_tiles_a100():
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    policy = Policy(cfg, CUDA())
    td = TileDict.from_block_tile([64, 64], 32, cfg, CUDA())
    policy._expand_reduce_axis(td)
    assert (td.rstep, td.smem_cost) == (64, 32768) and td.block_per_SM == 4  # occupancy not recomputed
    td = TileDict.from_block_tile([128, 128], 32, cfg, CUDA())
    policy._expand_reduce_axis(td)
    assert td.rstep == 32
    # [128,128]: 128 threads -> [16,8]; next block size 64 -> [16,16] needs 256 regs -> sequence ends
    assert [t.thread_tile for t in policy.assign_thread_tile(td, 2)] == [[16, 8]]
    assert policy.recommend_block_size(td)[:5] == [128, 64, 256, 32, 512]
    assert policy.recommend_block_size(td)[-1] == 1024


def test_large_prime_reduce_axis_uses_powers_of_two():
    policy = Policy(MatmulConfig(64, 64, 127, 32), CUDA())
    assert policy.get_reduce_step_candidates(127) == [1, 2, 4, 8, 16, 32, 64]
    assert policy.get_reduce_step_candidates(61) == [1, 61]  # small prime: divisors kept


def test_tiledict_hash_repr_and_clone():
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    h = get_roller_hints(cfg, CUDA(), topk=2)
    assert hash(h[0]) == hash(tuple(h[0].block_tile + h[0].thread_tile))
    assert len({h[0]: 1, h[1]: 2}) == 2
    text = repr(h[0])
    assert "block_tile=[128, 128]" in text and "2.1 MiB" in text and "32.0 KiB" in text
    twin = h[0].clone()
    twin.block_tile[0] = 1
    assert h[0].block_tile[0] == 128


# ---- 3. product vs independent restatement on further shapes -----------------------------------

def test_product_equals_restatement_on_random_shapes():
    rng = random.Random(7)
    dims = [48, 64, 96, 100, 127, 192, 250, 256, 384, 500, 512, 640, 1000, 1024, 1536, 3000]
    for _ in range(25):
        M, N, K = rng.choice(dims), rng.choice(dims), rng.choice(dims)
        got = [row(h) for h in get_roller_hints(MatmulConfig(M, N, K, 32), CUDA(), topk=12)]
        assert got == [orow(h) for h in po.hints(M, N, K, 12)], (M, N, K)


def test_invariants_of_emitted_hints_a100():
    for shape in [(2048, 4096, 2048), (3000, 5000, 1536), (1000, 640, 384)]:
        cfg = MatmulConfig(*shape, 32)
        arch = CUDA()
        policy = Policy(cfg, arch)
        base = policy._assign_reduce_step()
        ranked = policy.get_block_tiles_candidates([1, 1], base)
        prios = [(t.traffic + 1) * t.num_wave for t in ranked]
        assert prios == sorted(prios)
        for h in get_roller_hints(cfg, arch, topk=20):
            m, n = h.block_tile
            tm, tn = h.thread_tile
            assert h.smem_cost == h.rstep * (m + n) * 4 <= arch.smem_cap
            assert cfg.K % h.rstep == 0 and h.rstep % base == 0
            assert (m * n) % (tm * tn) == 0 and tm >= tn and tm * tn < 256
            assert h.grid_size == math.ceil(cfg.M / m) * math.ceil(cfg.N / n)


# ---- MI355X model -------------------------------------------------------------------------------------

def test_mi355x_model_numbers():
    a = MI355X()
    assert (a.compute_max_core, a.warp_size, a.sm_partition, a.xcd_count) == (256, 64, 4, 8)
    assert a.reg_cap == 131072 and a.lds_bytes == 160 * 1024
    assert a.smem_cap == a.max_smem_usage == 80 * 1024  # per pipeline stage under double buffering
    assert a.get_avaliable_tensorintrin_shapes() == [(32, 32, 2), (16, 16, 4)]
    # 256 CUs * 4 SIMDs * 64 FLOP/clk * 2.4 GHz
    assert a.peak_matrix_tflops == pytest.approx(256 * 4 * 64 * 2.4e9 / 1e12, rel=1e-3)
    with pytest.raises(NotImplementedError):
        CUDA().get_avaliable_tensorintrin_shapes()
    assert TileDevice().reg_estimate_divisor == 32 and TileDevice().thread_reg_limit == 256


class _Props:
    compute_units = 128
    lds_bytes_per_block = 65536
    clock_khz = 2000000
    l2_bytes = 1 << 20


def test_mi355x_from_device_overrides():
    a = MI355X.from_device(_Props())
    assert a.compute_max_core == 128 and a.smem_cap == 32768 and a.clock_mhz == 2000
    assert a.peak_matrix_tflops == pytest.approx(128 * 256 * 2.0e9 / 1e12)


SHAPES_MI = [(2048, 2048, 2048), (2048, 2048, 8192), (4096, 8192, 4096), (8192, 4096, 2048), (3000, 5000, 1536), (200, 300, 72)]


@pytest.mark.parametrize("shape", SHAPES_MI)
def test_mi355x_hints_are_launchable_kernel_configs(shape):
    cfg = MatmulConfig(*shape, 32)
    arch = MI355X()
    hints = get_roller_hints(cfg, arch, topk=20)
    assert 1 <= len(hints) <= 20
    for h in hints:
        m, n = h.block_tile
        wm, wn = h.wave_tile
        mi = h.mfma
        assert mi in (32, 16) and m % wm == 0 and n % wn == 0 and wm % mi == 0 and wn % mi == 0
        assert (wm // mi) * (wn // mi) <= 32                        # MFMA blocks one wave keeps in registers
        assert h.threads == 64 * (m // wm) * (n // wn) <= 1024
        assert h.rstep % (4 * 64 // mi) == 0
        # thread tile = wave tile seen per lane; launch geometry formula of the reference still holds
        assert h.thread_tile == [wm // 8, wn // 8]
        dims = utils.get_block_dims(h.block_tile + [0], h.thread_tile + [0])
        assert dims[0] * dims[1] == h.threads
        assert h.thread_tile[0] * h.thread_tile[1] <= 256          # accumulators per lane
        swizzled = (cfg.K % 4 == 0 and cfg.N % 4 == 0 and h.rstep & (h.rstep - 1) == 0
                    and (m * h.rstep) % 256 == 0 and (h.rstep * n) % 256 == 0)
        padded = not swizzled and (h.rstep // 4) % 2 == 0                             # padding only where it makes the row an odd number of 16-byte units
        assert h.smem_cost == (h.rstep * (m + n) + (4 * m if padded else 0)) * 4   # one stage; padded rows off the direct path
        assert 2 * h.smem_cost <= arch.lds_bytes                    # double-buffered tile fits a CU
        g = hint_to_gemm_config(cfg, h, 3)
        assert g.lds_bytes == 2 * h.smem_cost and g.direct == int(swizzled)
        assert h.grid_size == math.ceil(cfg.M / m) * math.ceil(cfg.N / n)


def test_mi355x_ranking_prefers_tiles_that_fill_the_chip():
    policy = Policy(MatmulConfig(2048, 2048, 2048, 32), MI355X())
    by_tile = {tuple(t.block_tile): policy.estimate_seconds(t) for t in policy.get_block_tiles_candidates([1, 1], 32)}
    # 256x256 leaves three quarters of the CUs idle on a 2048^2 output; 128x128 gives one tile per CU
    assert by_tile[(128, 128)] < by_tile[(256, 128)] < by_tile[(256, 256)]
    big = Policy(MatmulConfig(8192, 8192, 8192, 32), MI355X())
    by_tile = {tuple(t.block_tile): big.estimate_seconds(t) for t in big.get_block_tiles_candidates([1, 1], 32)}
    assert by_tile[(256, 256)] < by_tile[(32, 32)]
    ranked = big.get_block_tiles_candidates([1, 1], 32)
    est = [big.estimate_seconds(t) for t in ranked]
    assert est == sorted(est)


def test_mi355x_ragged_problem_gets_ladder_tiles():
    policy = Policy(MatmulConfig(3000, 5000, 1536, 32), MI355X())
    tiles = {tuple(t.block_tile) for t in policy.get_block_tiles_candidates([1, 1], 32)}
    assert (128, 128) in tiles and (256, 256) in tiles     # neither divides 3000 or 5000
    assert all(m % 16 == 0 and n % 16 == 0 for m, n in tiles)
    assert all(s % 16 == 0 for s in policy.get_reduce_step_candidates(1536))
    odd = Policy(MatmulConfig(37, 53, 29, 32), MI355X())
    assert odd._assign_reduce_step() % 16 == 0
    assert get_roller_hints(MatmulConfig(37, 53, 29, 32), MI355X(), topk=4)


def test_split_block_over_waves():
    a = MI355X()
    assert analyze.split_block_over_waves([128, 128], 4, 32, a) == ([64, 64], 32)
    assert analyze.split_block_over_waves([256, 256], 4, 32, a) == ([128, 128], 32)
    assert analyze.split_block_over_waves([128, 128], 2, 32, a) == ([64, 128], 32)
    assert analyze.split_block_over_waves([16, 64], 1, 16, a) == ([16, 64], 16)   # only the 16x16x4 shape fits
    assert analyze.split_block_over_waves([48, 48], 1, 32, a) == ([48, 48], 16)   # 3 column blocks: dword reads of B
    assert analyze.split_block_over_waves([192, 320], 4, 32, a) == ([96, 160], 32)   # 3 x 5 blocks of 32x32
    assert analyze.split_block_over_waves([256, 256], 1, 32, a) is None           # 64 blocks: more than a wave keeps in registers
    assert analyze.split_block_over_waves([64, 64], 4, 8, a) == ([32, 32], 32)   # k step 8 rules out 16x16x4 only


def test_mi355x_block_sizes_aim_for_one_wave_per_simd():
    cfg = MatmulConfig(4096, 8192, 4096, 32)
    policy = Policy(cfg, MI355X())
    td = TileDict.from_block_tile([256, 256], 32, cfg, MI355X())
    assert policy.recommend_block_size(td)[:3] == [256, 512, 1024]      # 4 waves, then 8 and 16: whole waves on every SIMD first
    assert policy.score_block_size(192) > policy.score_block_size(512)  # three waves leave a SIMD idle
    assert Policy(cfg, CUDA()).recommend_block_size(TileDict.from_block_tile([128, 128], 32, cfg, CUDA()))[0] == 128
    hints = get_roller_hints(cfg, MI355X(), topk=4)
    # one hint per block tile, at one wave per SIMD, with the 16x16x4 instruction where it fits.  First the
    # tile of which two fit a CU at once (each hides the other's barriers, fill and drain), then its
    # neighbours of the same kind, then the one-per-CU 256 x 256 tile with the 32x32x2 instruction or the
    # next smaller tile (their estimates are 0.1 % apart and change places from one refit of the sweep to
    # the next; the sweep has them 0.5 % apart, the smaller tile ahead)
    listed = [(h.block_tile, h.wave_tile, h.threads, h.mfma, h.stream_k) for h in hints]
    assert listed[:3] == [([128, 128], [64, 64], 256, 16, 0), ([64, 256], [64, 64], 256, 16, 0), ([256, 64], [64, 64], 256, 16, 0)]
    assert listed[3] in (([256, 256], [128, 128], 256, 32, 0), ([64, 128], [32, 64], 256, 16, 0))
    assert len({tuple(h.block_tile) for h in hints}) == 4
    # the second block size of a tile is still there for callers that complete tiles themselves
    td = policy.get_block_tiles_candidates([1, 1], 32)[0]
    assert [(h.wave_tile, h.threads) for h in policy.assign_thread_tile(td, 2)] == [([64, 64], 256), ([32, 64], 512)]
    # 256x256 (one per CU) is out for 16x16x4: at four waves 128x128 would be 64 blocks, more than the
    # kernel keeps in registers, and at eight waves 4 x 8 blocks of 16x16 need more fragment registers
    # than half a SIMD's file leaves
    big = next(t for t in policy.get_block_tiles_candidates([1, 1], 32) if t.block_tile == [256, 256])
    assert [(h.wave_tile, h.threads, h.mfma) for h in policy.assign_thread_tile(big, 2)] == [([128, 128], 256, 32), ([64, 128], 512, 32)]
    assert analyze.split_block_over_waves([256, 256], 4, 32, MI355X(), shapes=[(16, 16, 4)]) is None
    assert analyze.split_block_over_waves([256, 128], 4, 32, MI355X(), shapes=[(16, 16, 4)]) == ([64, 128], 16)   # 4 x 8 = 32 blocks


def test_mi355x_register_budget_drops_splits_that_would_spill():
    arch = MI355X()
    for shape in SHAPES_MI + [(8192, 8192, 8192)]:
        for h in get_roller_hints(MatmulConfig(*shape, 32), arch, topk=40):
            waves_per_simd = -(-(h.threads // 64) // arch.sm_partition)
            acc = h.thread_tile[0] * h.thread_tile[1]
            frags = 2 * 4 * (h.wave_tile[0] // h.mfma + h.wave_tile[1] // h.mfma)
            assert acc + frags + Policy.REG_OVERHEAD <= arch.regs_per_lane // waves_per_simd, h
    cfg = MatmulConfig(8192, 8192, 8192, 32)
    policy = Policy(cfg, arch)
    assert not TileDict.from_block_tile([512, 256], 16, cfg, arch).valid   # 131072 accumulators fill the CU's registers
    td = TileDict.from_block_tile([256, 256], 32, cfg, arch)
    assert [(h.threads, h.mfma) for h in policy._assign_wave_tiles(td, 256)] == [(256, 32)]
    # eight waves share a SIMD in pairs: 128 accumulators + 48 fragment registers + 50 fit 256,
    # 128 + 96 + 50 (16x16x4: 4 x 8 blocks) do not -- that kernel spills
    assert [(h.threads, h.mfma) for h in policy._assign_wave_tiles(td, 512)] == [(512, 32)]
    assert policy._assign_wave_tiles(td, 1024) == []                               # 64 + 96 > 128
    assert policy._assign_wave_tiles(td, 96) == []                                 # not a whole number of waves


def test_mi355x_reduce_step_stays_short_unless_the_device_model_says_grow():
    import dataclasses
    arch = MI355X()
    assert not arch.grow_reduce_step and CUDA().grow_reduce_step
    # the committed model: every hint keeps the 32-wide step (whole 128-byte lines, smallest stages)
    for shape in SHAPES_MI:
        assert {h.rstep for h in get_roller_hints(MatmulConfig(*shape, 32), arch, topk=8)} == {32}, shape
    small = [h for h in get_roller_hints(MatmulConfig(2048, 2048, 2048, 32), arch, topk=8) if h.block_tile == [128, 128]][0]
    assert (small.rstep, small.smem_cost, small.block_per_SM) == (32, 32768, 2)
    # with growth switched on (the reference's rule) the step takes the share of LDS a block really has:
    # 2048^2 output, 128x128 tiles: 256 blocks on 256 CUs -> one block per CU -> the whole 80 KB stage budget
    grow = dataclasses.replace(arch, grow_reduce_step=True)
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    td = TileDict.from_block_tile([128, 128], 32, cfg, grow)
    Policy(cfg, grow)._expand_reduce_axis(td)
    assert (td.rstep, td.smem_cost) == (64, 65536)
    # 4096x8192 output with the same tile: 8 blocks per CU, two resident -> 40 KB each -> step stays 32
    cfg = MatmulConfig(4096, 8192, 4096, 32)
    td = TileDict.from_block_tile([128, 128], 32, cfg, grow)
    Policy(cfg, grow)._expand_reduce_axis(td)
    assert td.rstep == 32


def test_mi355x_top_hints_compile_without_spills_or_scratch():
    """The register model against the real compiler: the first eight hints of every benchmark shape
    (and of two ragged ones) become kernels that spill nothing and use no scratch memory."""
    from mlir_roller_amd import hip
    from mlir_roller_amd.benchmark import README_SHAPES
    seen = {}
    for shape in list(README_SHAPES) + [(3000, 5000, 1536), (200, 300, 72), (2560, 2560, 2560), (1920, 2880, 2048),
                                        (4095, 4097, 4093), (2049, 2047, 2051)]:
        cfg = MatmulConfig(*shape, 32)
        for h in get_roller_hints(cfg, MI355X(), topk=8):
            seen.setdefault(hint_to_gemm_config(cfg, h, 3), (shape, h))
    assert len(seen) >= 20
    for g, (shape, h) in seen.items():
        res = hip.code_object_resources(hip.compile_config(g))
        assert res["vgpr_spills"] == 0 and res["scratch_bytes"] == 0, (shape, g.tag(), res)
        # scalar registers that overflow are parked in vector-register lanes, not in memory.  Only two kinds
        # of kernel get there, and within bounds: the one-wave tiles of tiny ragged problems (dozens of
        # per-load predicates) and the stream-K kernels (the split's parameters stay live across the
        # segments of a workgroup; their K loop itself carries no such traffic, which a GPU timing shows)
        # -- and the kernels for dword-aligned rows (the step that K ends in works its offsets out again)
        assert res["sgpr_spills"] == 0 or (res["sgpr_spills"] <= 64 and (g.threads == 64 or g.streamk)) \
            or (res["sgpr_spills"] <= 160 and g.vec == 1), (shape, g.tag(), res)
        assert 0 < res["vgprs"] <= 512 // max(1, g.threads // 256), (g.tag(), res)
        # a stream-K grid is sized for that many workgroups per CU: they have to fit the register file together
        if g.streamk and g.threads >= 256:
            assert res["vgprs"] <= 512 // (g.streamk * (g.threads // 256)), (shape, g.tag(), res)


def test_mi355x_small_wave_tiles_list_the_long_k_instruction_first():
    arch = MI355X()
    def first(shape):
        policy = Policy(MatmulConfig(*shape, 32), arch)
        td = policy.get_block_tiles_candidates([1, 1], 32)[0]
        return list(policy.assign_thread_tile(td, 2))
    a, b = first((2048, 2048, 2048))                       # 64x128 over four, then eight waves
    assert (a.block_tile, a.wave_tile, a.mfma, b.wave_tile, b.mfma) == ([64, 128], [32, 64], 16, [32, 32], 16)
    a, b = first((4096, 8192, 4096))                       # 128x128 over four, then eight waves
    assert (a.block_tile, a.wave_tile, a.mfma, b.wave_tile, b.mfma) == ([128, 128], [64, 64], 16, [32, 64], 16)
    both = Policy(MatmulConfig(2048, 4096, 2048, 32), arch)._assign_wave_tiles(
        TileDict.from_block_tile([128, 256], 32, MatmulConfig(2048, 4096, 2048, 32), arch), 256)
    assert [(t.wave_tile, t.mfma) for t in both] == [([64, 128], 16), ([64, 128], 32)]   # up to 64x128: long k first


def test_committed_ranking_constants_equal_a_refit_of_the_committed_sweep():
    """The MI355X ranking model is reproducible from the tree: refitting the committed sweep gives
    the constants that ``arch.MI355X`` carries, and replaying the policy on that sweep finds a kernel
    within one percent of the fastest measured one among its first four hints (two percent with its
    first hint alone) on every benchmark shape."""
    from mlir_roller_amd import calibrate
    data = calibrate.load()
    records = data["records"]
    assert len(records) >= 500 and len({tuple(r["shape"]) for r in records}) >= 15
    arch = MI355X()
    fit = calibrate.fit(records)
    assert tuple(fit["mfma_efficiency"]) == tuple(arch.mfma_efficiency), fit
    assert fit["co_resident_gain"] == arch.co_resident_gain, fit
    assert fit["rms_residual"] < 0.02 and fit["points"] >= 100
    assert calibrate.fit_waves_per_simd(records)["waves_per_partition"] == arch.waves_per_partition
    assert calibrate.fit_long_k_mfma(records)["long_k_mfma_up_to"] == arch.long_k_mfma_up_to
    stream_k = calibrate.fit_stream_k(records)
    assert stream_k["stream_k_loss"] == arch.stream_k_loss and stream_k["pairs"] >= 100, stream_k
    pieces = calibrate.fit_stream_k_pieces(records)
    assert pieces["stream_k_piece_bandwidth"] == arch.stream_k_piece_bandwidth and pieces["points"] >= 50, pieces
    small = calibrate.fit_small_tiles(records)
    assert small["small_tile_slope"] == arch.small_tile_slope and small["points"] >= 10, small
    from mlir_roller_amd.benchmark import README_SHAPES
    rows = {tuple(r["shape"]): r for r in calibrate.check(records, topk=4)}
    for shape in list(README_SHAPES) + [(3000, 5000, 1536)]:
        row = rows[shape]
        assert row["unmeasured_in_topk"] == 0 and row["topk_over_fastest"] <= 1.01, row
        assert row["top1_over_fastest"] <= 1.02, row
    # off the benchmark table -- cubes from 512 to 2560, a problem of one and a half rounds of tiles, problems
    # with a long K and few tiles (where a stream-K kernel is twice as fast as any whole-tile kernel):
    # the first four hints hold a kernel within 1 % of the fastest measured.  Three outliers are known: the
    # smallest cube, a 3.7 us kernel whose leaders differ by less than the launch-to-launch spread, the tall
    # and skinny 65536 x 128 x 128 (four K steps per tile), whose fastest kernels have eight waves, and
    # 1920 x 2880 x 2048 (one and a half rounds), where the estimates of the first eight stream-K kernels lie
    # within 0.6 % of one another and their times within 5 %
    off_table = [s for s in rows if s not in README_SHAPES and s != (3000, 5000, 1536)]
    assert {(4096, 64, 4096), (64, 4096, 4096), (384, 512, 256), (256, 256, 256), (65536, 128, 128)} <= set(off_table)
    for shape in off_table:
        limit = {(256, 256, 256): 1.05, (65536, 128, 128): 1.05, (1920, 2880, 2048): 1.03}.get(shape, 1.01)
        assert rows[shape]["unmeasured_in_topk"] == 0 and rows[shape]["topk_over_fastest"] <= limit, rows[shape]
    # a stream-K kernel leads where K is long and the tiles are few, and there the first hint is the fastest or
    # its mirror image (32 x 64 and 64 x 32 tiles: the same estimate, times within 2 %)
    for shape in [(4096, 64, 4096), (64, 4096, 4096)]:
        assert stream_k["best_plain_over_best_stream_k"]["x".join(map(str, shape))] > 1.8
        assert rows[shape]["top1_over_fastest"] <= 1.02, rows[shape]


def test_first_four_hints_on_dword_aligned_shapes_hold_a_kernel_close_to_the_fastest():
    """Shapes whose K or N is not a multiple of 4 (rows that are only dword-aligned) have a data set of
    their own, measured like the sweep (``calibrate measure --shapes ... --out``): seven shapes from
    1001 x 999 x 1003 to 8191 x 8193 x 8189, 96 kernels each in both forms.  No constant is fitted to it;
    it checks that the model that was fitted to aligned shapes still orders these: whole tiles of 64 x 96,
    four to a CU, are among the three fastest kernels on four of them (the loads of misaligned rows touch two cache
    lines where aligned ones touch one, and more resident workgroups hide that), stream-K kernels on big
    tiles come next, and a workgroup of more than 256 registers (128 x 160 with the 60 registers that
    dword-aligned rows cost) is known to run alone."""
    from mlir_roller_amd import calibrate
    data = calibrate.load(calibrate.DATA_DIR / "mi355x_f32_dword_rows.json")
    records = data["records"]
    shapes = {tuple(r["shape"]) for r in records}
    assert len(shapes) == 7 and all(s[1] % 4 or s[2] % 4 for s in shapes) and len(records) >= 600
    rows = {tuple(r["shape"]): r for r in calibrate.check(records, topk=4)}
    for shape, row in rows.items():
        # (8191 x 8193 x 8189: the estimate puts stream-K kernels on tall tiles ahead of the whole 64 x 96 and
        # 64 x 160 tiles and the eight-wave 256 x 192 that are fastest; the best of the first four is 3 % behind)
        limit = 1.04 if shape == (8191, 8193, 8189) else 1.015
        assert row["unmeasured_in_topk"] == 0 and row["topk_over_fastest"] <= limit, row
        assert row["top1_over_fastest"] <= 1.07, row
    fastest = {s: min((r for r in records if tuple(r["shape"]) == s), key=lambda r: r["ms"]) for s in shapes}
    leaders = {s: sorted((r for r in records if tuple(r["shape"]) == s), key=lambda r: r["ms"])[:3] for s in shapes}
    assert sum(1 for three in leaders.values() if any(sorted(r["block_tile"]) == [64, 96] and not r["stream_k"] for r in three)) >= 4
    # 4095 x 4097 x 4093 runs at 0.92 of the matrix peak, its aligned neighbour 4096^3 at 0.97
    best = fastest[(4095, 4097, 4093)]["ms"]
    assert 2.0 * 4095 * 4097 * 4093 / best / 1e9 > 0.9 * MI355X().peak_matrix_tflops


def test_a_hint_that_loses_its_residency_is_ranked_again():
    """Block tiles are ranked before their wave tile is known.  On 8191 x 8193 x 8189 (dword-aligned rows: 60
    more registers) the 128 x 160 tile is ranked as two workgroups per CU, and its wave tile of 64 x 80 then
    turns out to need more than half of the register file: the hint is emitted where its new estimate puts
    it, not where the tile stood, and a stream-K form never asks for more workgroups than fit."""
    arch = MI355X()
    cfg = MatmulConfig(8191, 8193, 8189, 32)
    policy = Policy(cfg, arch)
    hints = get_roller_hints(cfg, arch, topk=12)
    alone = [h for h in hints if h.block_tile == [128, 160]]
    assert alone and all(h.block_per_SM == 1 and h.stream_k <= 1 for h in alone)
    assert TileDict.from_block_tile([128, 160], 32, cfg, arch).block_per_SM == 2           # as the tile was ranked
    first = [policy.estimate_seconds(h) for h in hints[:4]]
    assert max(first) <= min(policy.estimate_seconds(h) for h in hints) * 1.005            # nothing cheaper was pushed out of the first four
    assert not any(h.block_tile == [128, 160] for h in hints[:4])
    for h in hints:
        if h.stream_k and h.threads >= 256:
            regs = int(h.wave_tile[0] * h.wave_tile[1] // 64) + policy._reg_overhead(h, h.wave_tile, h.mfma, h.threads)
            assert h.stream_k * (h.threads // 256) * regs <= arch.regs_per_lane, (h.block_tile, h.stream_k, regs)
    # an aligned neighbour keeps the tile at two per CU
    aligned = get_roller_hints(MatmulConfig(8192, 8192, 8192, 32), arch, topk=12)
    assert all(h.block_per_SM == 2 for h in aligned if h.block_tile == [128, 160])


def test_the_latency_and_cache_terms_of_the_estimate_matter_where_k_is_long_and_tiles_are_few():
    """``step_latency_seconds`` and ``cache_bandwidth_ratio`` are not fitted in closed form but chosen on
    the committed sweep; this pins what they are for.  With both switched off the first four hints of
    4096 x 64 x 4096 miss the fastest measured kernel by more than 5 %; with the committed values, and
    with any values in the ranges named beside them, they hold it."""
    import dataclasses
    from mlir_roller_amd import calibrate
    records = [r for r in calibrate.load()["records"] if tuple(r["shape"]) in {(4096, 64, 4096), (64, 4096, 4096)}]

    def worst(arch):
        return max(1e9 if row["topk_over_fastest"] is None else row["topk_over_fastest"] for row in calibrate.check(records, arch=arch, topk=4))
    base = MI355X()
    assert worst(base) <= 1.01
    assert worst(dataclasses.replace(base, step_latency_seconds=0.0, cache_bandwidth_ratio=1.0)) > 1.05
    for latency, ratio in ((0.2e-6, 2.5), (0.4e-6, 4.0)):
        assert worst(dataclasses.replace(base, step_latency_seconds=latency, cache_bandwidth_ratio=ratio)) <= 1.01, (latency, ratio)


def test_ranking_model_holds_on_a_shape_it_was_not_fitted_on():
    """Leave one shape out: refit the efficiency model without a shape's records, rank that shape with the
    refitted constants, and the first four hints still hold a kernel within three percent of the fastest
    one measured on it -- for every benchmark shape and the ragged one.  The committed constants are
    fitted on all of these; this is what says they are not merely memorised."""
    from mlir_roller_amd import calibrate
    from mlir_roller_amd.benchmark import README_SHAPES
    records = calibrate.load()["records"]
    for shape in list(README_SHAPES) + [(3000, 5000, 1536)]:
        rest = [r for r in records if tuple(r["shape"]) != shape]
        fit = calibrate.fit(rest)
        arch = MI355X()
        arch.mfma_efficiency, arch.co_resident_gain = tuple(fit["mfma_efficiency"]), fit["co_resident_gain"]
        arch.stream_k_loss = calibrate.fit_stream_k(rest)["stream_k_loss"]
        own = [r for r in records if tuple(r["shape"]) == shape]
        (row,) = calibrate.check(own, arch=arch, topk=4)
        assert row["topk_over_fastest"] is not None and row["topk_over_fastest"] <= 1.03, (shape, fit["mfma_efficiency"], row)


def test_sessions_of_a_sweep_merge_to_the_shortest_time_per_kernel():
    from mlir_roller_amd import calibrate
    rec = lambda tile, ms, sk=0, rank=1: {"shape": [2048, 2048, 2048], "block_tile": list(tile), "wave_tile": [32, 64], "mfma": 16, "rstep": 32,
                                          "threads": 256, "edge": 0, "direct": 1, "stream_k": sk, "rank_when_measured": rank, "ms": ms}
    first = {"device": {}, "records": [rec((64, 128), 0.120), rec((128, 128), 0.119, rank=2), rec((64, 128), 0.125, sk=2, rank=3)]}
    second = {"device": {}, "sessions": 2, "records": [rec((64, 128), 0.117), rec((128, 128), 0.121, rank=2), rec((128, 64), 0.118, rank=4)]}
    both = calibrate.merge(first, second)
    assert both["sessions"] == 3
    got = {(tuple(r["block_tile"]), r["stream_k"]): r["ms"] for r in both["records"]}
    assert got == {((64, 128), 0): 0.117, ((128, 128), 0): 0.119, ((64, 128), 2): 0.125, ((128, 64), 0): 0.118}
    assert [r["rank_when_measured"] for r in both["records"]] == [1, 2, 3, 4]         # in the order of the sweep


def test_refit_rejects_a_sweep_that_cannot_pin_the_model():
    from mlir_roller_amd import calibrate
    with pytest.raises(ValueError):
        calibrate.fit([])
    big_tiles_only = [r for r in calibrate.load()["records"] if min(r["block_tile"]) >= 128]
    with pytest.raises(ValueError):
        calibrate.fit_small_tiles(big_tiles_only)            # nothing below the knee
    with pytest.raises(ValueError):
        calibrate.fit_stream_k_pieces([r for r in big_tiles_only if tuple(r["shape"]) == (4096, 8192, 4096)])   # no tile split many ways
    one = [{"shape": [4096, 4096, 4096], "block_tile": [256, 256], "wave_tile": [128, 128], "mfma": 32, "rstep": 32,
            "threads": 256, "ms": 0.95}]
    with pytest.raises(ValueError):
        calibrate.fit(one)
    with pytest.raises(ValueError):
        calibrate.fit_waves_per_simd(one)
    # a synthetic sweep that follows the model exactly is recovered exactly
    arch = MI355X()
    synth = []
    shared = []
    for m, n in [(256, 256), (128, 256), (128, 128), (64, 128), (64, 64), (32, 64)]:
        rec = {"shape": [4096, 4096, 4096], "block_tile": [m, n], "wave_tile": [m // 2, n // 2], "mfma": 16,
               "rstep": 32, "threads": 256}
        per_cu = (4096 // m) * (4096 // n) // 256
        resident = min(calibrate.resident_tiles(rec, arch), per_cu)
        shared.append(resident > 1)
        eff = 0.95 - 2.5 * (1 / m + 1 / n) + (0.02 if resident > 1 else 0.0)
        t = per_cu * calibrate.ideal_tile_seconds(m, n, 4096, 32, arch) / eff + -(-per_cu // resident) * calibrate.fixed_tile_seconds(m, n, arch)
        synth.append(dict(rec, ms=t * 1e3))
    assert any(shared) and not all(shared)
    got = calibrate.fit(synth)
    assert got["mfma_efficiency"] == (0.95, 2.5) and got["co_resident_gain"] == 0.02 and got["rms_residual"] < 1e-9
