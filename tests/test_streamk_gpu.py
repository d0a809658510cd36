"""Parity of the stream-K variant of the GEMM kernel with the oracle, on an MI355X, through the C ABI.

A stream-K launch splits the K range of some tiles over workgroups and sums the pieces through a
workspace; on integer-valued inputs every partial sum is exact, so the result must equal the host
GEMM bit for bit however the split falls -- and on any input it must be the same bits from run to
run, because the pieces are added in K order whoever arrives last."""

import sys

import numpy as np
import pytest

from mlir_roller_amd import hip
from mlir_roller_amd.hip import DeviceArray, GemmConfig, GemmPlan, HipError
from oracle import gemm_oracle as go

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run(cfg, A, B, c_init=None, workspace=None):
    M, K = A.shape
    N = B.shape[1]
    dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B.T if cfg.trans_b else B)
    if c_init is None:
        dC = DeviceArray((M, N))
        dC.fill_bytes(0xFF)          # NaN pattern: every element must be overwritten
    else:
        dC = DeviceArray.from_host(c_init)
    GemmPlan(cfg).launch(dA, dB, dC, M, N, K, workspace=workspace)
    hip.synchronize()
    return dC.get()


def host_gemm(A, B):
    """Exact on integer inputs either way; the plain-C oracle for what it finishes in a moment."""
    return go.c_gemm_f32(A, B) if A.shape[0] * A.shape[1] * B.shape[1] <= 2e8 else go.gemm_f32(A, B)


# (config, shapes).  The grid is streamk workgroups per CU, cut down to one K step per workgroup on small
# problems -- so the small shapes split every tile into single K steps, the large ones split few.
CASES = [
    # aligned, no predication: 24 units on 24 workgroups; one tile per CU pair; two rounds and a bit
    (GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2), [(256, 384, 128), (1024, 1024, 2048), (2304, 2048, 512), (128, 128, 32)]),
    # ragged in every dimension, K tail in the last piece, problems smaller than a tile
    (GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2), [(200, 300, 200), (130, 260, 96), (1, 4, 4), (1000, 1000, 1000), (2100, 1900, 1124)]),
    # ragged M and N with whole K steps (no K predicates in the loop); 32x32x2 and 16x16x4; one wave along N
    (GemmConfig(96, 160, 32, 48, 80, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 2), [(3000, 5000, 1536), (200, 340, 64), (96 * 3 + 24, 160 * 2 + 40, 96)]),
    (GemmConfig(96, 160, 32, 48, 80, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 1), [(1500, 2500, 768)]),
    (GemmConfig(64, 320, 32, 16, 320, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 1), [(3000, 5000, 1536), (130, 700, 64)]),
    (GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 1), [(512, 768, 160), (1000, 1000, 500), (3000, 5000, 1536)]),
    (GemmConfig(128, 256, 32, 64, 64, 32, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 2), [(1100, 1300, 256)]),
    # register-staged loads (padded rows), dword global accesses, transposed second operand
    (GemmConfig(128, 128, 32, 64, 64, 32, 3, 4, 0, 4, 1, 3, 8, 0, 0, 0, 2), [(200, 300, 200), (1000, 900, 400)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 3, 4, 0, 1, 1, 3, 8, 0, 0, 0, 2), [(37, 53, 29), (130, 127, 17), (1001, 999, 1003)]),
    (GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1, 2), [(200, 300, 200), (1000, 900, 400)]),
    (GemmConfig(96, 96, 16, 48, 48, 16, 3, 8, 8, 1, 1, 3, 8, 0, 0, 1, 2), [(101, 99, 37), (1001, 999, 403)]),
    # no workgroup remap, panel of 3, four and eight workgroups per CU
    (GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 0, 8, 0, 1, 0, 2), [(1000, 1000, 1000)]),
    (GemmConfig(128, 64, 32, 64, 32, 16, 3, 0, 0, 4, 2, 2, 3, 0, 1, 0, 4), [(1100, 900, 512)]),
    (GemmConfig(64, 64, 32, 32, 32, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 8), [(1000, 1000, 1000), (70, 92, 52)]),
    # few tiles and a long K: every tile is split five to sixty-four ways, and the workgroup that arrives last
    # reads the pieces back four, two or one at a time (two, four or sixteen 16-byte chunks per row of blocks)
    (GemmConfig(64, 32, 32, 16, 32, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2), [(4096, 64, 4096), (256, 128, 2048), (256, 128, 1216), (256, 128, 1120)]),   # 4, 32, 19/37/38, 18/22/35 pieces
    (GemmConfig(32, 64, 32, 16, 32, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2), [(64, 4096, 4096)]),
    (GemmConfig(64, 64, 32, 32, 32, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 2), [(4096, 64, 4096), (250, 132, 2048 + 32)]),
    (GemmConfig(128, 64, 32, 32, 64, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2), [(4096, 64, 4096)]),
    (GemmConfig(64, 64, 32, 32, 32, 32, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 1), [(512, 512, 8192)]),
]
FLAT = [(cfg, shape) for cfg, shapes in CASES for shape in shapes]


@pytest.mark.parametrize("cfg,shape", FLAT, ids=[f"{c.tag()}-{s[0]}x{s[1]}x{s[2]}" for c, s in FLAT])
def test_streamk_matches_oracle_within_tolerance_and_exactly_on_integers(device, cfg, shape):
    M, N, K = shape
    sched = hip.streamk_schedule(cfg, M, N, K, device.compute_units)
    say("case", cfg.tag(), shape, "grid", sched.grid, "tiles", sched.tiles, "K steps", sched.k_steps)
    Ai, Bi = go.make_inputs(M, N, K, seed=1, distribution="integer")
    want = host_gemm(Ai, Bi)
    got = run(cfg, Ai, Bi)
    assert np.array_equal(got, want)
    assert np.array_equal(run(cfg, Ai, Bi), want)            # the arrival counters came back to zero
    if M * N * K <= 3e9:
        A, B = go.make_inputs(M, N, K, seed=M + 7 * N + 13 * K)
        first = run(cfg, A, B)
        rep = go.error_report(first, A, B)
        assert rep["ok"], rep
        assert np.array_equal(first.view(np.uint32), run(cfg, A, B).view(np.uint32))   # same bits whoever arrives last


# (config, shape, rounds of whole tiles, tiles shared out) on 256 CUs
ROUNDS = [
    (GemmConfig(32, 32, 32, 16, 16, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2), (1500, 1300, 200), 3, 391),    # 1927 tiles on 512 workgroups
    (GemmConfig(32, 32, 32, 16, 16, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2), (1024, 1024, 96), 2, 0),       # two full rounds, nothing split
    (GemmConfig(32, 32, 32, 16, 16, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2), (1600, 1632, 72), 4, 502),
    (GemmConfig(64, 64, 32, 32, 32, 16, 3, 0, 0, 1, 1, 3, 8, 0, 1, 0, 2), (2049, 2047, 131), 1, 544),    # dword-aligned rows; 32 tiles over two rounds: fewer than a quarter of the grid, so two rounds' worth is shared
    (GemmConfig(64, 32, 32, 16, 32, 16, 3, 0, 0, 4, 2, 0, 8, 0, 1, 1, 1), (1000, 1100, 160), 1, 304),    # no remap, Bt, 560 tiles on 256
    (GemmConfig(32, 64, 32, 16, 32, 16, 3, 0, 0, 4, 2, 2, 5, 1, 1, 0, 4), (3100, 2100, 64), 2, 1153),    # panels of 5, accumulate, 3201 tiles on 1024
]


@pytest.mark.parametrize("cfg,shape,rounds,shared", ROUNDS, ids=[f"{c.tag()}-{s[0]}x{s[1]}x{s[2]}" for c, s, _, _ in ROUNDS])
def test_rounds_of_whole_tiles_and_a_shared_remainder(device, cfg, shape, rounds, shared):
    """A stream-K launch works the full rounds of its grid as whole tiles (all but one, if few tiles are
    left over) and shares out the K steps of the rest: exact on integers and the same bits every run."""
    M, N, K = shape
    sched = hip.streamk_schedule(cfg, M, N, K, device.compute_units)
    say("case", cfg.tag(), shape, "grid", sched.grid, "tiles", sched.tiles, "whole", sched.whole_tiles)
    if device.compute_units == 256:
        assert (sched.whole_tiles, sched.tiles - sched.whole_tiles) == (rounds * sched.grid, shared)
    A, B = go.make_inputs(M, N, K, seed=5, distribution="integer")
    want = host_gemm(A, B)
    if cfg.accum:
        C0 = np.random.default_rng(3).integers(-9, 9, (M, N)).astype(np.float32)
        assert np.array_equal(run(cfg, A, B, c_init=C0), want + C0)
    else:
        assert np.array_equal(run(cfg, A, B), want)
        assert np.array_equal(run(cfg, A, B), want)
        A, B = go.make_inputs(M, N, K, seed=6)
        first = run(cfg, A, B)
        assert go.error_report(first, A, B)["ok"]
        assert np.array_equal(first.view(np.uint32), run(cfg, A, B).view(np.uint32))


def test_seeded_points_of_the_template_parameter_space_are_exact_as_stream_k(device):
    """Forty-eight seeded (configuration, shape) pairs from everything the configuration check accepts with
    ``streamk`` set -- both instructions, 1 to 8 waves, 1 to 7 column blocks per wave, both operand layouts,
    every edge mode, access width, remap mode and padding -- on integer inputs: bit-exact against the oracle, in
    overwrite and in accumulate mode, whatever way the split falls."""
    sys.path.insert(0, str(__import__("pathlib").Path(__file__).resolve().parent))
    from gemm_cases import seeded_streamk_cases
    seen = set()
    for case, cfg, (M, N, K) in seeded_streamk_cases():
        sched = hip.streamk_schedule(cfg, M, N, K, device.compute_units)
        say("stream-K template case", case, cfg.tag(), (M, N, K), "grid", sched.grid, "tiles", sched.tiles, "K steps", sched.k_steps)
        A, B = go.make_inputs(M, N, K, seed=3000 + case, distribution="integer")
        want = go.gemm_f32(A, B)
        if cfg.accum:
            C0 = np.random.default_rng(case).integers(0, 10, (M, N)).astype(np.float32)
            assert np.array_equal(run(cfg, A, B, c_init=C0), want + C0), (case, cfg.tag(), (M, N, K))
        else:
            assert np.array_equal(run(cfg, A, B), want), (case, cfg.tag(), (M, N, K))
        seen.add((cfg.mi, cfg.edge, cfg.vec, cfg.direct, cfg.trans_b, cfg.streamk))
    assert len(seen) >= 30          # the draw really spreads over the parameter space


def test_streamk_accumulates_into_c(device):
    cfg = GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 1, 1, 0, 2)
    M, N, K = 300, 260, 512
    A, B = go.make_inputs(M, N, K, seed=3, distribution="integer")
    C0 = np.random.default_rng(5).integers(0, 100, (M, N)).astype(np.float32)
    assert np.array_equal(run(cfg, A, B, c_init=C0), C0 + go.c_gemm_f32(A, B))


def test_streamk_is_bitwise_repeatable_and_close_to_the_plain_kernel(device):
    """Twenty launches of a problem whose tiles are all split (uniform inputs, so that a change in the
    order of the additions would show): one set of bits.  The plain kernel adds in another order; both are
    within tolerance of the float64 result."""
    cfg = GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2)
    plain = GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 0)
    M, N, K = 1536, 1536, 1536                                  # 144 tiles on 512 workgroups
    A, B = go.make_inputs(M, N, K, seed=11)
    dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((M, N))
    plan = GemmPlan(cfg)
    outs = []
    for i in range(20):
        dC.fill_bytes(0xFF)
        plan.launch(dA, dB, dC, M, N, K)
        hip.synchronize()
        outs.append(dC.get().view(np.uint32))
    for o in outs[1:]:
        assert np.array_equal(o, outs[0])
    C64 = go.c_gemm_f64(A, B) if hasattr(go, "c_gemm_f64") else None
    assert go.error_report(outs[0].view(np.float32), A, B, C64=C64)["ok"]
    assert go.error_report(run(plain, A, B), A, B, C64=C64)["ok"]


def test_streamk_with_the_callers_workspace(device):
    cfg = GemmConfig(96, 160, 32, 48, 80, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 2)
    M, N, K = 1000, 1500, 512
    A, B = go.make_inputs(M, N, K, seed=2, distribution="integer")
    want = go.c_gemm_f32(A, B)
    plan = GemmPlan(cfg)
    need, counters = plan.workspace_bytes(M, N, K)
    sched = hip.streamk_schedule(cfg, M, N, K, device.compute_units)
    assert (need, counters) == (sched.workspace_bytes, sched.counter_bytes) and need > counters > 0
    ws = DeviceArray.zeros((need // 4,), np.uint32)
    for _ in range(3):                                          # the same workspace again and again
        assert np.array_equal(run(cfg, A, B, workspace=ws), want)
        assert not ws.get()[: counters // 4].any()              # the kernel left its counters at zero
    # a smaller problem in the same (now dirty) slots
    A2, B2 = go.make_inputs(300, 400, 256, seed=4, distribution="integer")
    assert np.array_equal(run(cfg, A2, B2, workspace=ws), go.c_gemm_f32(A2, B2))
    dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((M, N))
    small = DeviceArray.zeros((need // 4 - 64,), np.uint32)
    with pytest.raises(HipError, match="workspace"):
        plan.launch(dA, dB, dC, M, N, K, workspace=small)
    # a plan without stream-K needs none and ignores what it is given
    plain = GemmPlan(GemmConfig(96, 160, 32, 48, 80, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 0))
    assert plain.workspace_bytes(M, N, K) == (0, 0)
    dC.fill_bytes(0xFF)
    plain.launch(dA, dB, dC, M, N, K, workspace=small)
    hip.synchronize()
    assert np.array_equal(dC.get(), want)


def test_launches_back_to_back_share_the_library_workspace(device):
    """The forty-eight seeded stream-K problems again, but all of them queued on one stream with no
    synchronisation in between, forwards and then backwards: tile sizes, tile counts and grids change from
    launch to launch, the library's workspace grows in the middle of the queue, and every launch has to find
    the counters at zero and nobody else's pieces in its slots."""
    sys.path.insert(0, str(__import__("pathlib").Path(__file__).resolve().parent))
    from gemm_cases import seeded_streamk_cases
    stream = hip.Stream()
    cases = [(cfg, shape) for _, cfg, shape in seeded_streamk_cases() if not cfg.accum]
    queued = []
    for order in (cases, cases[::-1]):
        for i, (cfg, (M, N, K)) in enumerate(order):
            A, B = go.make_inputs(M, N, K, seed=4000 + i, distribution="integer")
            dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B.T if cfg.trans_b else B)
            dC = DeviceArray((M, N))
            dC.fill_bytes(0xFF)
            queued.append((cfg, (M, N, K), A, B, dA, dB, dC, GemmPlan(cfg)))
    hip.synchronize()
    for cfg, (M, N, K), _, _, dA, dB, dC, plan in queued:           # nothing but launches from here to the synchronisation
        plan.launch(dA, dB, dC, M, N, K, stream=stream)
    hip.synchronize()
    assert len(queued) >= 60
    for cfg, shape, A, B, _, _, dC, _ in queued:
        assert np.array_equal(dC.get(), go.gemm_f32(A, B)), (cfg.tag(), shape)


def test_a_launch_with_more_counters_behind_one_with_fewer_on_the_same_workspace(device):
    """The library's workspace is reused from launch to launch.  A launch of more than 65536 tiles keeps
    counters where an earlier launch kept the slots of its first workgroups; the library has to zero that
    stretch again, or the tiles whose counters lie there never see their last piece arrive."""
    small = GemmConfig(16, 16, 32, 16, 16, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2)      # 1 KiB slots right behind 256 KiB of counters
    many = GemmConfig(32, 32, 32, 16, 16, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2)
    first, second = (16, 16, 2048), (8224, 8256, 96)                               # 1 tile in 64 pieces; 66306 tiles, most shares end inside a tile
    assert hip.streamk_schedule(many, *second, device.compute_units).counter_bytes > hip.streamk_schedule(small, *first, device.compute_units).counter_bytes == 256 * 1024
    A1, B1 = go.make_inputs(*first, seed=5, distribution="integer")
    A2, B2 = go.make_inputs(*second, seed=6, distribution="integer")
    for _ in range(2):                                                                # and back again: the smaller layout behind the larger
        assert np.array_equal(run(small, A1, B1), host_gemm(A1, B1))
        assert np.array_equal(run(many, A2, B2), go.gemm_f32(A2, B2))


def test_streamk_degenerate_extents(device):
    cfg = GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2)
    plan = GemmPlan(cfg)
    dA, dB, dC = DeviceArray.zeros((64,)), DeviceArray.zeros((64,)), DeviceArray((8, 8))
    dC.fill_bytes(0xFF)
    plan.launch(dA, dB, dC, 8, 8, 0)                            # K = 0: C = 0
    hip.synchronize()
    assert not dC.get().any()
    dC.fill_bytes(0xFF)
    plan.launch(dA, dB, dC, 0, 8, 8)                            # M = 0: nothing happens
    hip.synchronize()
    assert np.isnan(dC.get()).all()
    acc = GemmPlan(GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 1, 1, 0, 2))
    dC.set(np.full((8, 8), 3.0, np.float32))
    acc.launch(dA, dB, dC, 8, 8, 0)                             # K = 0, accumulating: C unchanged
    hip.synchronize()
    assert np.all(dC.get() == 3.0)


def test_streamk_on_two_streams_at_once(device):
    """Launches on different streams get different workspaces from the library, so they may overlap."""
    cfg = GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 0, 2)
    plan = GemmPlan(cfg)
    shapes = [(1000, 1000, 1000), (900, 1100, 1024)]
    streams = [hip.Stream(), hip.Stream()]
    data = []
    for shape in shapes:
        A, B = go.make_inputs(*shape, seed=shape[0], distribution="integer")
        data.append((A, B, DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((shape[0], shape[1]))))
    for _ in range(5):
        for (A, B, dA, dB, dC), shape, stream in zip(data, shapes, streams):
            plan.launch(dA, dB, dC, *shape, stream=stream)
    hip.synchronize()
    for A, B, dA, dB, dC in data:
        assert np.array_equal(dC.get(), go.c_gemm_f32(A, B))
