"""Parity of the HIP GEMM path with the oracle, on an MI355X, every call through the C ABI of
libroller_hip.so (ctypes).  Tolerances are the ones the path is specified with:

    normwise     ||C - C32||_F / ||C32||_F <= 1e-5      C32 = float32 host GEMM
    elementwise  max|C - C64| <= 1e-4 * sqrt(K) * max|A| * max|B|      C64 = float64 host GEMM

plus bit-exact equality wherever the mathematics allows it (integer-valued inputs, structured
operands, run-to-run determinism)."""

import ctypes as C
import sys

import numpy as np
import pytest

from mlir_roller_amd import hip, roller
from mlir_roller_amd import benchmark as bm
from mlir_roller_amd.analyze import MatmulConfig, get_roller_hints
from mlir_roller_amd.arch import MI355X
from mlir_roller_amd.hip import DeviceArray, GemmConfig, GemmPlan, HipError
from oracle import gemm_oracle as go

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_gemm(cfg: GemmConfig, A: np.ndarray, B: np.ndarray, c_init=None) -> np.ndarray:
    M, K = A.shape
    N = B.shape[1]
    # a trans_b kernel takes the second operand as Bt[N, K]
    dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B.T if cfg.trans_b else B)
    if c_init is None:
        dC = DeviceArray((M, N))
        dC.fill_bytes(0xFF)  # NaN pattern: every element must be overwritten
    else:
        dC = DeviceArray.from_host(c_init)
    GemmPlan(cfg).launch(dA, dB, dC, M, N, K)
    hip.synchronize()
    return dC.get()


def test_device_is_an_mi355x(device):
    assert device.arch.decode().startswith("gfx950")
    assert device.wavefront_size == 64 and device.compute_units >= 128
    assert device.lds_bytes_per_block >= 64 * 1024
    arch = MI355X.from_device(device)
    assert arch.compute_max_core == device.compute_units


# (config, shapes): aligned, ragged in every dimension, smaller than one tile, K not a multiple of BK
CASES = [
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 0), [(256, 384, 128), (128, 128, 16)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1), [(200, 300, 72), (1, 4, 4), (129, 132, 20), (64, 64, 1000)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 1, 1), [(37, 53, 29), (1, 1, 1), (130, 127, 17), (5, 700, 3)]),
    (GemmConfig(256, 256, 32, 128, 128, 32, 2, 4, 0, 4, 1), [(512, 768, 160), (300, 520, 100), (256, 256, 32)]),
    (GemmConfig(256, 256, 16, 128, 128, 32, 2, 4, 0, 4, 0), [(512, 512, 64)]),
    (GemmConfig(256, 128, 32, 64, 128, 32, 2, 4, 0, 4, 1), [(300, 260, 100)]),
    (GemmConfig(128, 256, 32, 64, 64, 32, 2, 4, 0, 4, 1), [(300, 260, 100)]),         # 8 waves
    (GemmConfig(128, 128, 16, 64, 64, 16, 2, 4, 0, 4, 1), [(200, 300, 80), (33, 36, 16)]),  # 16x16x4 MFMA
    (GemmConfig(64, 64, 16, 16, 64, 16, 2, 4, 0, 1, 1), [(70, 90, 50)]),
    (GemmConfig(128, 128, 32, 64, 32, 32, 1, 4, 0, 4, 1), [(200, 300, 72)]),           # single LDS buffer, 1 column block
    (GemmConfig(64, 64, 16, 32, 32, 32, 2, 4, 0, 4, 1), [(200, 300, 72)]),
    (GemmConfig(64, 256, 32, 64, 64, 32, 2, 4, 0, 4, 1), [(100, 600, 96)]),
    (GemmConfig(32, 512, 32, 32, 128, 32, 2, 4, 0, 4, 1), [(100, 600, 96)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1, 0, 8), [(400, 500, 48)]),     # no workgroup remap
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1, 2, 3), [(1300, 500, 48)]),    # panel walk, ragged panel
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 0, 0, 4, 1), [(200, 300, 72)]),           # unpadded LDS
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 4, 4, 1), [(200, 300, 72)]),           # padded LDS-B
]
# pipeline depth 3 (register stage + split last round): every path of its step driver -- an even and an
# odd number of fragment rounds per K step, 1, 2, 3, 4 and many K steps, ragged K, every operand width
CASES += [
    (GemmConfig(128, 128, 32, 64, 64, 32, 3, 4, 0, 4, 1), [(200, 300, 32), (200, 300, 64), (130, 260, 96), (200, 300, 200)]),
    (GemmConfig(128, 128, 8, 64, 64, 32, 3, 4, 0, 4, 1), [(140, 132, 8), (140, 132, 16), (140, 132, 24), (140, 132, 32), (140, 132, 72), (140, 132, 100)]),
    (GemmConfig(128, 128, 24, 64, 64, 32, 3, 4, 0, 4, 1), [(140, 132, 24), (140, 132, 48), (140, 132, 120), (140, 132, 100)]),
    (GemmConfig(128, 128, 16, 64, 64, 16, 3, 4, 0, 4, 1), [(200, 300, 16), (200, 300, 48), (33, 36, 80)]),
    (GemmConfig(128, 128, 32, 32, 64, 32, 3, 4, 0, 4, 0), [(256, 384, 128)]),
    (GemmConfig(128, 128, 64, 32, 64, 16, 3, 4, 0, 4, 1), [(200, 300, 136)]),
    (GemmConfig(256, 256, 32, 64, 128, 32, 3, 4, 0, 4, 1), [(512, 768, 160), (300, 520, 100)]),
    (GemmConfig(256, 256, 32, 128, 128, 32, 3, 4, 0, 4, 0), [(512, 512, 64)]),
    (GemmConfig(256, 128, 32, 64, 64, 32, 3, 4, 0, 4, 1), [(300, 260, 100)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 3, 4, 0, 1, 1), [(37, 53, 29), (130, 127, 17)]),
    (GemmConfig(32, 64, 8, 32, 32, 32, 3, 4, 0, 4, 1), [(70, 92, 52)]),          # fewer load units than threads
    (GemmConfig(64, 64, 16, 16, 64, 16, 3, 4, 0, 1, 1), [(70, 90, 50)]),
    (GemmConfig(128, 128, 32, 64, 32, 32, 3, 4, 0, 4, 1), [(200, 300, 72)]),      # one column block per wave
]
# direct-to-LDS loads with swizzled A rows: every swizzle period (K step 8, 16, 32, 64), both MFMA shapes,
# ragged edges in all three dimensions (out-of-range lanes must deposit zeros), 1..many K steps
CASES += [
    (GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 300, 32), (200, 300, 64), (130, 260, 96), (200, 300, 200), (1, 4, 4)]),
    (GemmConfig(128, 128, 8, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(140, 132, 8), (140, 132, 16), (140, 132, 24), (140, 132, 100)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(140, 132, 48), (140, 132, 100)]),
    (GemmConfig(128, 128, 64, 32, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 300, 136), (128, 128, 64)]),
    (GemmConfig(128, 128, 16, 64, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 300, 16), (33, 36, 80)]),
    (GemmConfig(256, 256, 32, 64, 128, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(512, 768, 160), (300, 520, 100)]),
    (GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 0, 3, 8, 0, 1), [(512, 512, 64)]),
    (GemmConfig(256, 128, 32, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(300, 260, 100)]),
    (GemmConfig(32, 64, 8, 32, 32, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(70, 92, 52)]),       # fewer load units than threads
    (GemmConfig(64, 64, 16, 16, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(70, 92, 52)]),
    (GemmConfig(128, 128, 32, 64, 32, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 300, 72)]),
]
# second operand stored transposed (Bt[N, K]): staged and direct-to-LDS loads, both MFMA shapes, 1, 2 and
# 4 column blocks per wave (each has its own column permutation), dword path with odd K and N, ragged edges
CASES += [
    (GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(200, 300, 32), (130, 260, 96), (200, 300, 200), (1, 4, 4)]),
    (GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 0, 3, 8, 0, 1, 1), [(512, 512, 64)]),
    (GemmConfig(256, 256, 32, 64, 128, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(300, 520, 100)]),
    (GemmConfig(128, 128, 8, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(140, 132, 8), (140, 132, 100)]),
    (GemmConfig(128, 128, 64, 32, 64, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(200, 300, 136)]),
    (GemmConfig(128, 128, 32, 64, 32, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(200, 300, 72)]),       # one column block per wave
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 4, 4, 1, 3, 8, 0, 0, 1), [(200, 300, 72), (129, 132, 20)]),
    (GemmConfig(128, 128, 16, 64, 64, 16, 3, 4, 4, 1, 1, 3, 8, 0, 0, 1), [(37, 53, 29), (130, 127, 17)]),
    (GemmConfig(64, 64, 16, 16, 64, 16, 1, 4, 4, 1, 1, 3, 8, 0, 0, 1), [(70, 90, 50)]),
    (GemmConfig(128, 128, 24, 64, 64, 32, 3, 4, 4, 4, 1, 3, 8, 0, 0, 1), [(140, 132, 100)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 0, 0, 4, 0, 3, 8, 0, 0, 1), [(256, 384, 128)]),         # unpadded, aligned
]
# 3, 5, 6 and 10 column blocks per wave: the second operand is read with dword / 64-bit LDS loads and C
# leaves in dword / 64-bit stores; direct-to-LDS, staged, dword-global and transposed-operand paths
CASES += [
    (GemmConfig(192, 320, 32, 96, 160, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(400, 700, 96), (192, 320, 32), (1, 4, 4)]),      # 3 x 5 of 32x32
    (GemmConfig(96, 160, 32, 48, 80, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 340, 72), (96, 160, 64)]),                    # 3 x 5 of 16x16
    (GemmConfig(96, 96, 32, 48, 48, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1), [(192, 288, 96)]),                                     # 3 x 3, no predication
    (GemmConfig(96, 192, 16, 48, 96, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 400, 48)]),                                    # 3 x 6: 64-bit reads
    (GemmConfig(48, 320, 32, 48, 160, 16, 3, 0, 0, 4, 1, 3, 8, 0, 1), [(100, 700, 96)]),                                   # 3 x 10
    (GemmConfig(96, 96, 16, 96, 96, 32, 2, 4, 0, 4, 1), [(200, 300, 72)]),                                                 # one wave, 3 x 3 of 32x32, staged
    (GemmConfig(96, 160, 48, 48, 80, 16, 3, 4, 0, 4, 1), [(200, 340, 100)]),                                               # odd K step: staged at depth 3
    (GemmConfig(96, 96, 16, 48, 48, 16, 1, 4, 0, 1, 1), [(101, 99, 37)]),                                                  # dword global accesses
    (GemmConfig(192, 320, 32, 96, 160, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(400, 700, 96)]),                               # transposed operand, 5 blocks
    (GemmConfig(96, 192, 16, 48, 96, 16, 2, 4, 4, 4, 1, 3, 8, 0, 0, 1), [(200, 400, 48)]),                                 # transposed, 6 blocks, staged
    (GemmConfig(96, 96, 16, 48, 48, 16, 3, 4, 4, 1, 1, 3, 8, 0, 0, 1), [(101, 99, 37)]),                                   # transposed, 3 blocks, dword
]
# edge=2 (M and N ragged, K a whole number of steps: no K predicates in the loop) and pipeline depths 4 and 5
# (three and four LDS buffers, loads two and three K steps ahead): 1, 2, 3 and many K steps, fewer steps than buffers
CASES += [
    (GemmConfig(128, 128, 32, 64, 64, 32, 3, 0, 0, 4, 2, 3, 8, 0, 1), [(200, 300, 32), (130, 260, 96), (1, 4, 64)]),
    (GemmConfig(192, 320, 32, 96, 160, 32, 3, 0, 0, 4, 2, 3, 8, 0, 1), [(400, 700, 96)]),
    (GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 2), [(200, 300, 80)]),
    (GemmConfig(128, 128, 16, 64, 64, 16, 3, 4, 4, 1, 2, 3, 8, 0, 0, 1), [(37, 53, 32)]),
    (GemmConfig(128, 128, 32, 64, 64, 16, 4, 0, 0, 4, 0, 3, 8, 0, 1), [(256, 384, 32), (256, 384, 64), (256, 384, 96), (256, 384, 512)]),
    (GemmConfig(128, 128, 32, 64, 64, 16, 5, 0, 0, 4, 1, 3, 8, 0, 1), [(200, 300, 32), (200, 300, 64), (200, 300, 96), (200, 300, 128), (200, 300, 200), (130, 260, 1000)]),
    (GemmConfig(64, 64, 64, 16, 32, 16, 5, 0, 0, 4, 2, 3, 8, 0, 1), [(200, 300, 64), (200, 300, 448)]),
    (GemmConfig(128, 128, 8, 64, 64, 32, 4, 0, 0, 4, 1, 3, 8, 0, 1), [(140, 132, 8), (140, 132, 24), (140, 132, 100)]),     # odd number of rounds per step
    (GemmConfig(256, 256, 16, 128, 128, 32, 4, 0, 0, 4, 0, 3, 8, 0, 1), [(512, 512, 160)]),
    (GemmConfig(128, 128, 32, 32, 64, 32, 4, 0, 0, 4, 1, 3, 8, 0, 1, 1), [(200, 300, 200)]),                                 # transposed operand
]
FLAT = [(cfg, shape) for cfg, shapes in CASES for shape in shapes]


@pytest.mark.parametrize("cfg,shape", FLAT, ids=[f"{c.tag()}-{s[0]}x{s[1]}x{s[2]}" for c, s in FLAT])
def test_matches_oracle_within_tolerance_and_exactly_on_integers(device, cfg, shape):
    M, N, K = shape
    say("case", cfg.tag(), shape)
    A, B = go.make_inputs(M, N, K, seed=M + 7 * N + 13 * K)
    got = run_gemm(cfg, A, B)
    rep = go.error_report(got, A, B, C64=go.c_gemm_f64(A, B))
    assert rep["ok"], rep
    Ai, Bi = go.make_inputs(M, N, K, seed=1, distribution="integer")
    assert np.array_equal(run_gemm(cfg, Ai, Bi), go.c_gemm_f32(Ai, Bi))


def test_committed_exact_cases_on_the_gpu(device):
    """The committed integer known answers (tests/golden/gemm_exact_cases.json), bit for bit, through a dword
    kernel, a 128-bit kernel where the shape allows it, the direct-to-LDS kernel and the transposed-operand kernel."""
    import json
    from pathlib import Path
    cases = json.loads((Path(__file__).resolve().parent / "golden" / "gemm_exact_cases.json").read_text())
    for case in cases:
        A, B = np.array(case["A"], np.float32), np.array(case["B"], np.float32)
        want = np.array(case["C"], np.float32)
        cfgs = [GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 1, 1), GemmConfig(64, 64, 16, 16, 64, 16, 3, 4, 4, 1, 1, 3, 8, 0, 0, 1)]
        if case["K"] % 4 == 0 and case["N"] % 4 == 0:
            cfgs += [GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1), GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1),
                     GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1)]
        for cfg in cfgs:
            say("golden", case["name"], cfg.tag())
            assert np.array_equal(run_gemm(cfg, A, B), want), (case["name"], cfg.tag())


def test_structured_operands_are_exact(device):
    cfg = GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1)
    n = 200
    B = np.random.default_rng(3).standard_normal((n, 264), dtype=np.float32)
    assert np.array_equal(run_gemm(cfg, np.eye(n, dtype=np.float32), B), B)                 # I * B = B
    A = np.random.default_rng(4).standard_normal((136, n), dtype=np.float32)
    assert np.array_equal(run_gemm(cfg, A, np.eye(n, dtype=np.float32)), A)                 # A * I = A
    ones = run_gemm(cfg, np.ones((130, 1000), np.float32), np.ones((1000, 140), np.float32))
    assert np.all(ones == 1000.0)
    # one-hot A picks single rows of B: catches any transposition or row/column permutation
    pick = np.zeros((150, n), np.float32)
    rows = np.random.default_rng(5).integers(0, n, 150)
    pick[np.arange(150), rows] = 1
    assert np.array_equal(run_gemm(cfg, pick, B), B[rows])


def test_transposed_second_operand(device):
    """C = A * Bt^T with Bt[N, ldb >= K]: one-hot operands catch a wrong column permutation, the
    leading dimension is honoured, the launch checks ldb against K, and the policy -> Compiler path
    takes the flag at full size (bit-exact on integer inputs, same bits as the B[K, N] kernel)."""
    cfg = GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1)
    n = 200
    Bt = np.random.default_rng(3).standard_normal((264, n), dtype=np.float32)           # N x K
    assert np.array_equal(run_gemm(cfg, np.eye(n, dtype=np.float32), Bt.T), Bt.T)
    pick = np.zeros((n, 140), np.float32)                                               # B = one-hot columns
    cols = np.random.default_rng(5).integers(0, n, 140)
    pick[cols, np.arange(140)] = 1
    A = np.random.default_rng(4).standard_normal((136, n), dtype=np.float32)
    assert np.array_equal(run_gemm(cfg, A, pick), A[:, cols])

    M, N, K, ldb = 200, 300, 72, 96
    rng = np.random.default_rng(21)
    hA = rng.integers(0, 10, (M, K)).astype(np.float32)
    hBt = rng.integers(0, 10, (N, ldb)).astype(np.float32)
    dA, dB, dC = DeviceArray.from_host(hA), DeviceArray.from_host(hBt), DeviceArray((M, N))
    plan = GemmPlan(cfg)
    plan.launch(dA, dB, dC, M, N, K, ldb=ldb)
    hip.synchronize()
    assert np.array_equal(dC.get(), go.c_gemm_f32(hA, np.ascontiguousarray(hBt[:, :K].T)))
    with pytest.raises(HipError):
        plan.launch(dA, dB, dC, M, N, K, ldb=K - 4)

    arch = MI355X.from_device(device)
    for shape in ((2048, 2048, 2048), (4096, 8192, 4096), (3000, 5000, 1536), (1000, 2002, 514)):
        mc = MatmulConfig(*shape, 32)
        hint = get_roller_hints(mc, arch, topk=1)[0]
        say("trans_b", shape, hint.block_tile, hint.wave_tile, hint.rstep)
        A, B = go.make_inputs(*shape, seed=2, distribution="integer")
        dA, dBt, dB = DeviceArray.from_host(A), DeviceArray.from_host(B.T), DeviceArray.from_host(B)
        outs = []
        for trans_b, operand in ((True, dBt), (False, dB)):
            func = roller.Compiler(mc, hint, bm.PIPELINE_DEPTH, trans_b=trans_b).compile()
            assert func.gemm_config.trans_b == int(trans_b)
            dC = DeviceArray((shape[0], shape[1]))
            dC.fill_bytes(0xFF)
            func(func.grid_dims(), func.block_dims(), (dA, operand, dC))
            hip.synchronize()
            outs.append(dC.get())
        assert np.array_equal(outs[0], go.gemm_f32(A, B)), shape
        assert np.array_equal(outs[0], outs[1]), shape
    mc = MatmulConfig(1024, 1024, 512, 32)
    hint = get_roller_hints(mc, arch, topk=1)[0]
    func = roller.Compiler(mc, hint, 3, trans_b=True).compile()
    roller.run_eval(func, 3, hint, repeat_times=3)                  # uniform inputs, tolerance check inside
    assert func.last_eval["ok"]


def test_seeded_random_shapes_through_policy_are_exact(device):
    """Forty seeded shapes (ragged, tiny, K and N odd or multiples of 4), each through
    get_roller_hints -> Compiler at a random pipeline depth, operand layout and accumulate mode:
    bit-exact against the host GEMM on integer inputs (sums stay far below 2^24)."""
    from gemm_cases import seeded_policy_cases
    # the data-sheet model, so that the cases (and the kernels compiled ahead for them) do not depend on the box
    for case, mc, hint, depth, trans_b, accumulate in seeded_policy_cases(MI355X()):
        M, N, K = mc.M, mc.N, mc.K
        say("random case", case, (M, N, K), "depth", depth, "trans_b", trans_b, "accumulate", accumulate,
            hint.block_tile, hint.wave_tile, hint.rstep)
        func = roller.Compiler(mc, hint, depth, accumulate=accumulate, trans_b=trans_b).compile()
        rng = np.random.default_rng(1000 + case)
        A = rng.integers(-4, 5, (M, K)).astype(np.float32)
        B = rng.integers(-4, 5, (K, N)).astype(np.float32)
        C0 = rng.integers(-50, 50, (M, N)).astype(np.float32)
        dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B.T if trans_b else B)
        dC = DeviceArray.from_host(C0)
        func(func.grid_dims(), func.block_dims(), (dA, dB, dC))
        hip.synchronize()
        want = A @ B + (C0 if accumulate else 0)
        assert np.array_equal(dC.get(), want), (case, M, N, K, func.gemm_config.tag())


def test_seeded_points_of_the_template_parameter_space_are_exact(device):
    """Two seeded draws of seventy-two (configuration, shape) pairs from everything the library's
    configuration check accepts -- not only what the policy emits -- each at two values of K:
    integer inputs, bit-exact against the oracle, in overwrite and in accumulate mode."""
    from gemm_cases import TEMPLATE_SEEDS, seeded_template_cases
    seen = set()
    draws = [(seed, *drawn) for seed in TEMPLATE_SEEDS for drawn in seeded_template_cases(seed=seed)]
    for seed, case, cfg, (M, N, K0) in draws:
        # every kernel at its drawn K and with one K step more: the loop runs its steps in pairs and
        # starts differently for an odd and an even number of them
        for K in (K0, K0 + cfg.bk):
            say("template case", seed, case, cfg.tag(), (M, N, K))
            A, B = go.make_inputs(M, N, K, seed=1000 + case + seed % 977, distribution="integer")
            want = go.gemm_f32(A, B)
            if cfg.accum:
                C0 = np.random.default_rng(case).integers(0, 10, (M, N)).astype(np.float32)
                assert np.array_equal(run_gemm(cfg, A, B, c_init=C0), want + C0), (seed, case, cfg.tag(), K)
            else:
                assert np.array_equal(run_gemm(cfg, A, B), want), (seed, case, cfg.tag(), K)
        seen.add((cfg.mi, cfg.stages, cfg.edge, cfg.vec, cfg.direct, cfg.trans_b))
    assert len(seen) >= 60          # the draw really spreads over the parameter space


def test_direct_to_lds_loads_of_dword_aligned_rows_are_exact(device):
    """Forty seeded (configuration, shape) pairs on the direct-to-LDS path with dword-aligned rows
    (any N and K; full K steps come with 16-byte loads at dword alignment, the step K ends in one
    float per lane), a third of them as stream-K: integer inputs, bit-exact against the oracle, each
    at its drawn K and with one K step more."""
    from gemm_cases import seeded_dword_direct_cases
    tails = set()
    for case, cfg, (M, N, K0) in seeded_dword_direct_cases():
        for K in (K0, K0 + cfg.bk):
            say("dword-aligned direct case", case, cfg.tag(), (M, N, K))
            A, B = go.make_inputs(M, N, K, seed=3000 + case, distribution="integer")
            want = go.gemm_f32(A, B)
            if cfg.accum:
                C0 = np.random.default_rng(case).integers(0, 10, (M, N)).astype(np.float32)
                assert np.array_equal(run_gemm(cfg, A, B, c_init=C0), want + C0), (case, cfg.tag(), K)
            else:
                assert np.array_equal(run_gemm(cfg, A, B), want), (case, cfg.tag(), K)
        tails.add((K0 % cfg.bk == 0, -(-K0 // cfg.bk) <= 2, N % 4 == 0))
    assert len(tails) >= 6          # whole and cut last steps, short and long K, N aligned or not


def test_accumulate_mode_adds_into_c(device):
    M, N, K = 300, 260, 100
    A, B = go.make_inputs(M, N, K, seed=11, distribution="integer")
    C0 = np.random.default_rng(12).integers(-50, 50, (M, N)).astype(np.float32)
    for cfg in (GemmConfig(256, 128, 32, 64, 128, 32, 2, 4, 0, 4, 1, 3, 8, 1),
                GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 1, 1, 3, 8, 1),
                GemmConfig(128, 128, 16, 64, 32, 32, 2, 4, 0, 4, 1, 3, 8, 1),
                GemmConfig(128, 128, 32, 32, 64, 32, 3, 4, 0, 4, 1, 3, 8, 1),
                GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 1, 1)):
        got = run_gemm(cfg, A, B, c_init=C0)
        assert np.array_equal(got, go.c_gemm_f32(A, B, out=C0.copy(), accumulate=True)), cfg.tag()


def test_leading_dimensions_wider_than_the_matrix(device):
    M, N, K, lda, ldb, ldc = 200, 300, 72, 96, 320, 304
    rng = np.random.default_rng(21)
    hA = rng.integers(0, 10, (M, lda)).astype(np.float32)
    hB = rng.integers(0, 10, (K, ldb)).astype(np.float32)
    hC = np.full((M, ldc), -7.0, np.float32)
    dA, dB, dC = DeviceArray.from_host(hA), DeviceArray.from_host(hB), DeviceArray.from_host(hC)
    GemmPlan(GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1)).launch(dA, dB, dC, M, N, K, lda, ldb, ldc)
    hip.synchronize()
    out = dC.get()
    assert np.array_equal(out[:, :N], go.c_gemm_f32(hA[:, :K], hB[:, :N]))
    assert np.all(out[:, N:] == -7.0)                               # padding columns untouched


def test_dword_aligned_views_with_odd_offsets_and_leading_dimensions(device):
    """Sub-matrices that start at odd float offsets inside larger buffers, with odd leading dimensions:
    every row of A, B and C is only dword-aligned, and differently so from row to row.  Through the
    direct-to-LDS kernels for dword-aligned rows -- whole tiles, stream-K, and the Bt layout -- the
    result is exact and nothing outside the C view is touched."""
    M, N, K, lda, ldb, ldc = 203, 299, 1037, 1051, 307, 311
    rng = np.random.default_rng(22)
    A, B = go.make_inputs(M, N, K, seed=23, distribution="integer")
    want = go.gemm_f32(A, B)
    for cfg in (GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 1, 1, 3, 8, 0, 1, 0, 0),
                GemmConfig(64, 96, 32, 32, 48, 16, 3, 0, 0, 1, 1, 3, 8, 0, 1, 0, 2),
                GemmConfig(64, 64, 32, 32, 32, 32, 3, 0, 0, 1, 1, 3, 8, 0, 1, 1, 0)):
        say("views", cfg.tag())
        second = np.ascontiguousarray(B.T) if cfg.trans_b else B            # Bt[N][ldb >= K] or B[K][ldb >= N]
        rows_b, width_b = second.shape
        ld_b = 1049 if cfg.trans_b else ldb
        hA = rng.integers(0, 10, (M * lda + 3,)).astype(np.float32)        # the views start 3, 1 and 5 floats in
        hB = rng.integers(0, 10, (rows_b * ld_b + 1,)).astype(np.float32)
        hC = np.full((M * ldc + 5,), -7.0, np.float32)
        hA[3:].reshape(M, lda)[:, :K] = A
        hB[1:].reshape(rows_b, ld_b)[:, :width_b] = second
        dA, dB, dC = DeviceArray.from_host(hA), DeviceArray.from_host(hB), DeviceArray.from_host(hC)
        GemmPlan(cfg).launch(hip.Ptr(dA.ptr + 12), hip.Ptr(dB.ptr + 4), hip.Ptr(dC.ptr + 20), M, N, K, lda, ld_b, ldc)
        hip.synchronize()
        out = dC.get()
        assert np.array_equal(out[5:].reshape(M, ldc)[:, :N], want), cfg.tag()
        assert np.all(out[:5] == -7.0) and np.all(out[5:].reshape(M, ldc)[:, N:] == -7.0), cfg.tag()   # nothing beside the view


def test_empty_and_zero_k(device):
    plan = GemmPlan(GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1))
    dC = DeviceArray.from_host(np.full((8, 12), 3.0, np.float32))
    plan.launch(0, 0, dC, 8, 12, 0)                                 # K = 0: C = 0
    hip.synchronize()
    assert np.all(dC.get() == 0.0)
    dC.set(np.full((8, 12), 3.0, np.float32))
    plan.launch(0, 0, dC, 0, 12, 4)                                 # M = 0: nothing to do
    plan.launch(0, 0, dC, 8, 0, 4, ldb=4, ldc=12)
    hip.synchronize()
    assert np.all(dC.get() == 3.0)


def test_launch_rejects_what_the_kernel_was_not_built_for(device):
    dA, dB, dC = DeviceArray((256, 256)), DeviceArray((256, 256)), DeviceArray((256, 256))
    vec4 = GemmPlan(GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1))
    aligned = GemmPlan(GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 0))
    for plan, args, needle in [
        (vec4, (dA, dB, dC, 100, 101, 64), "multiples of 4"),
        (vec4, (dA, dB, dC, 100, 100, 62), "multiples of 4"),
        (vec4, (dA.ptr + 4, dB, dC, 100, 100, 64), "16-byte aligned"),
        (vec4, (dA, dB, dC, 100, 100, 64, 32), "leading dimension too small"),
        (vec4, (dA, dB, dC, -1, 100, 64), "negative dimension"),
        (vec4, (0, dB, dC, 100, 100, 64), "NULL matrix pointer"),
        (aligned, (dA, dB, dC, 200, 256, 64), "edge=0 kernel needs"),
        (aligned, (dA, dB, dC, 256, 256, 24), "edge=0 kernel needs"),
    ]:
        with pytest.raises(HipError) as err:
            plan.launch(*args)
        assert err.value.status == hip.RL_ERR_INVALID_ARG and needle in str(err.value)
    hip.synchronize()


def test_results_are_bitwise_reproducible_and_independent_of_tile_order(device):
    M, N, K = 1024, 1280, 512
    A, B = go.make_inputs(M, N, K, seed=31)
    base = GemmConfig(128, 128, 32, 64, 64, 32, 2, 4, 0, 4, 0)
    first = run_gemm(base, A, B)
    assert np.array_equal(first, run_gemm(base, A, B))
    for swz, group in ((0, 8), (1, 8), (2, 4)):
        other = GemmConfig(128, 128, 32, 64, 64, 32, 2, 4, 0, 4, 0, swz, group)
        assert np.array_equal(first, run_gemm(other, A, B)), (swz, group)
    # predication does not change the arithmetic of full tiles either
    assert np.array_equal(first, run_gemm(GemmConfig(128, 128, 32, 64, 64, 32, 2, 4, 0, 4, 1), A, B))


K_TAIL_CONFIGS = [
    GemmConfig(128, 128, 32, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1),        # direct-to-LDS, four rounds per step
    GemmConfig(128, 128, 8, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1),         # direct-to-LDS, one round per step (parity flips)
    GemmConfig(128, 128, 32, 64, 64, 16, 5, 0, 0, 4, 1, 3, 8, 0, 1),        # four LDS buffers: the tail is requested three steps ahead
    GemmConfig(128, 128, 32, 32, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1, 1),     # transposed second operand, direct-to-LDS
    GemmConfig(128, 128, 16, 64, 64, 32, 3, 4, 0, 4, 1),                    # register-staged, 128-bit accesses
    GemmConfig(128, 128, 24, 64, 64, 32, 3, 4, 0, 4, 1),                    # register-staged, three rounds per step
    GemmConfig(128, 128, 16, 64, 64, 16, 3, 4, 4, 1, 1),                    # dword-aligned rows: K and N odd
    GemmConfig(128, 128, 16, 64, 64, 16, 3, 4, 4, 1, 1, 3, 8, 0, 0, 1),     # the same with the transposed operand
]


@pytest.mark.parametrize("cfg", K_TAIL_CONFIGS, ids=[c.tag() for c in K_TAIL_CONFIGS])
def test_k_tail_at_every_position_of_the_pipeline(device, cfg):
    """K ends inside the last K step; only the pipeline step that requests that tile tests its
    loads against K.  One to seven K steps put that step before the loop, at its start, in its
    middle and nowhere (fewer steps than buffers).  Exact on integers; and a row of A must not
    pick up the start of the next row: with NaN in the first column of every odd row, the even
    rows of C stay finite (a tail read as data and multiplied by the zero rows past the end of
    B would turn them into NaN)."""
    M = 130
    N = 260 if cfg.vec == 4 else 259
    tails = (4, cfg.bk - 4) if cfg.vec == 4 else (1, cfg.bk - 1)
    for steps in range(1, 8):
        for tail in tails:
            K = (steps - 1) * cfg.bk + tail
            say("case", cfg.tag(), (M, N, K))
            Ai, Bi = go.make_inputs(M, N, K, seed=steps + 10 * tail, distribution="integer")
            assert np.array_equal(run_gemm(cfg, Ai, Bi), go.c_gemm_f32(Ai, Bi)), (steps, tail)
            Ai[1::2, 0] = np.nan
            got = run_gemm(cfg, Ai, Bi)
            assert np.isnan(got[1::2]).all() and np.isfinite(got[0::2]).all(), (steps, tail)


def test_pipeline_depth_does_not_change_the_bits(device):
    """Depths 1, 2, 3 and the direct-to-LDS variant run the same MFMAs in the same order per
    accumulator; only the way operands reach LDS differs."""
    M, N, K = 384, 512, 416
    A, B = go.make_inputs(M, N, K, seed=41)
    for bk, mi in ((32, 32), (16, 16), (8, 32)):
        outs = [run_gemm(GemmConfig(128, 128, bk, 64, 64, mi, stages, 4, 0, 4, 1), A, B) for stages in (1, 2, 3)]
        outs.append(run_gemm(GemmConfig(128, 128, bk, 64, 64, mi, 3, 0, 0, 4, 1, 3, 8, 0, 1), A, B))   # direct-to-LDS
        assert all(np.array_equal(outs[0], o) for o in outs[1:]), (bk, mi)


def test_plan_cache_and_one_shot_entry_point(device):
    cfg = GemmConfig(64, 64, 16, 32, 32, 32, 2, 4, 0, 4, 1)
    p1, p2 = GemmPlan(cfg), GemmPlan(cfg)
    assert p1.handle == p2.handle and p2.compile_ms == 0.0
    res = p1.resources()
    assert res["spilled"] == 0 and res["scratch_bytes"] == 0 and 0 < res["vgprs"] <= 512
    A, B = go.make_inputs(70, 80, 48, seed=2, distribution="integer")
    dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((70, 80))
    hip.gemm_f32(cfg, dA, dB, dC, 70, 80, 48)                        # rl_gemm_f32
    hip.synchronize()
    assert np.array_equal(dC.get(), go.c_gemm_f32(A, B))


def test_released_plans_and_damaged_cache_entries(device, tmp_path):
    """rl_gemm_plans_clear leaves old handles refusable (not dangling); a cache file that fails
    its checksum is recompiled in place instead of being handed to the loader."""
    cfg = GemmConfig(64, 64, 16, 32, 32, 32, 2, 4, 0, 4, 1)
    A, B = go.make_inputs(70, 92, 52, seed=5, distribution="integer")
    want = go.gemm_f32(A, B)
    old_dir = hip.DEFAULT_CACHE_DIR
    try:
        hip.set_cache_dir(tmp_path)
        hip.lib().rl_gemm_plans_clear()
        stale = GemmPlan(cfg)
        assert np.array_equal(run_gemm(cfg, A, B), want)
        hip.lib().rl_gemm_plans_clear()
        dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((70, 92))
        with pytest.raises(HipError) as err:
            stale.launch(dA, dB, dC, 70, 92, 52)
        assert "released" in str(err.value)
        (entry,) = tmp_path.glob("gemm_*.hsaco")
        good = entry.read_bytes()
        entry.write_bytes(good[:64] + b"\0" * (len(good) - 64))
        assert np.array_equal(run_gemm(cfg, A, B), want)            # reloaded through a fresh compile
        assert entry.read_bytes() == good
    finally:
        hip.lib().rl_gemm_plans_clear()
        hip.set_cache_dir(old_dir)


def test_lds_grant_is_read_back_and_large_tiles_launch(device):
    # the sweep's winners ask for 131072 bytes of dynamic LDS; the largest legal tile for all 163840
    big = GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 0, 3, 8, 0, 1)
    full = GemmConfig(256, 256, 40, 128, 128, 32, 2, 0, 0, 4, 1)
    assert big.lds_bytes == 131072 and full.lds_bytes == 163840
    for cfg, shape in ((big, (512, 512, 128)), (full, (300, 520, 200))):
        plan = GemmPlan(cfg)
        say("lds", cfg.tag(), "needs", plan.lds_bytes, "granted", plan.lds_limit, "device", device.lds_bytes_per_block)
        assert plan.lds_bytes == cfg.lds_bytes <= plan.lds_limit <= device.lds_bytes_per_block
        A, B = go.make_inputs(*shape, seed=3, distribution="integer")
        assert np.array_equal(run_gemm(cfg, A, B), go.gemm_f32(A, B))
    # a raw module function: the same opt-in, then a refusal with text above what the CU has
    fn = GemmPlan(big).function
    fn.set_max_dynamic_lds(131072)
    with pytest.raises(HipError, match="exceed the 160 KB"):
        fn.set_max_dynamic_lds(160 * 1024 + 4)
    with pytest.raises(HipError, match="dynamic LDS exceed"):
        fn((1,), (256,), (DeviceArray((4,)),) * 3 + (0, 0, 0, 0, 0, 0), shared_mem=device.lds_bytes_per_block + 1024)


def test_calls_from_another_thread_use_the_initialised_device(device):
    # the current device is per-thread state of the runtime: every entry point selects it again
    import threading
    cfg = GemmConfig(128, 128, 32, 64, 64, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1)
    A, B = go.make_inputs(200, 300, 96, seed=11, distribution="integer")
    out = {}

    def worker():
        try:
            out["C"] = run_gemm(cfg, A, B)          # malloc, memcpy, plan launch, sync, free on this thread
            e0, e1 = hip.Event(), hip.Event()
            e0.record(); e1.record(); e1.synchronize()
            out["ms"] = hip.get_elapsed_time(e0, e1)
        except Exception as e:                       # surfaced in the main thread below
            out["error"] = e

    t = threading.Thread(target=worker)
    t.start()
    t.join(60)
    assert not t.is_alive() and "error" not in out, out.get("error")
    assert np.array_equal(out["C"], go.gemm_f32(A, B)) and out["ms"] >= 0.0
    # clearing the plans waits for the device and for launch calls in progress; old handles are refused afterwards
    plan = GemmPlan(cfg)
    hip.check(hip.lib().rl_gemm_plans_clear())
    with pytest.raises(HipError, match="released"):
        plan.launch(DeviceArray((4,)), DeviceArray((4,)), DeviceArray((4,)), 1, 4, 4)
    assert np.array_equal(run_gemm(cfg, A, B), go.gemm_f32(A, B))     # a fresh plan works


def test_low_level_module_api_like_the_reference_uses_cupy(device):
    src = r'''extern "C" __global__ void axpy(float a, const float* x, float* y, int n) {
        int i = blockIdx.x * blockDim.x + threadIdx.x;
        if (i < n) y[i] = a * x[i] + y[i];
    }'''
    code, _ = hip.compile_source(src, "axpy.hip")
    func = hip.Module(code).get_function("axpy")
    x = np.arange(1000, dtype=np.float32)
    dx, dy = DeviceArray.from_host(x), DeviceArray.from_host(np.ones(1000, np.float32))
    stream = hip.Stream()
    start, stop = hip.Event(), hip.Event()
    start.record(stream)
    func((4,), (256,), (C.c_float(2.0), dx, dy, 1000), shared_mem=0, stream=stream)
    stop.record(stream)
    stop.synchronize()
    assert hip.get_elapsed_time(start, stop) >= 0.0
    assert np.array_equal(dy.get(), 2 * x + 1)
    with pytest.raises(HipError):
        hip.Module(code).get_function("no_such_kernel")
    hip.synchronize()


# ---- the named configurations at full size -------------------------------------------------------

FULL = [
    ("cfg1", (2048, 2048, 2048), "uniform"),
    ("cfg2", (2048, 2048, 8192), "uniform"),
    ("cfg3", (4096, 8192, 4096), "uniform"),
    ("cfg4", (3000, 5000, 1536), "normal"),
]


@pytest.mark.parametrize("name,shape,dist", FULL, ids=[f[0] for f in FULL])
def test_named_configs_full_size_through_policy_and_compiler(device, name, shape, dist, tmp_path):
    cfg = MatmulConfig(*shape, 32)
    hints = get_roller_hints(cfg, MI355X.from_device(device), topk=3)
    A, B = go.make_inputs(*shape, seed=0, distribution=dist)
    C32, C64 = go.gemm_f32(A, B), go.gemm_f64(A, B)
    dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B)
    for hint in hints:
        say(name, hint)
        func = roller.Compiler(cfg, hint, bm.PIPELINE_DEPTH, dump_path=tmp_path if hint is hints[0] else None).compile()
        dC = DeviceArray((shape[0], shape[1]))
        dC.fill_bytes(0xFF)
        func(func.grid_dims(), func.block_dims(), (dA.ptr, dB.ptr, dC.ptr), shared_mem=hint.smem_cost * 2)
        hip.synchronize()
        got = dC.get()
        rep = go.error_report(got, A, B, C32=C32, C64=C64)
        assert rep["ok"], (hint, rep)
        func(func.grid_dims(), func.block_dims(), (dA.ptr, dB.ptr, dC.ptr), shared_mem=0)
        hip.synchronize()
        assert np.array_equal(got, dC.get())                         # bit-for-bit across runs
    assert (tmp_path / "kernel.hip").exists() and (tmp_path / "kernel.json").exists()
    assert (tmp_path / "build.log").read_text().strip()         # the compiler's output, or a line that says there was none


TUNER_TOPK = 8   # at least what the tuner tries by default, with room for a user's --topk 8


def test_every_kernel_the_tuner_can_pick_is_exact_at_full_size(device):
    """M0..M13 and the ragged 3000x5000x1536, every one of the policy's first hints (all the
    tuner may time and keep), through ``Compiler`` at the sweep's pipeline depth.  Size-independent
    property: with inputs in {0..9} every partial sum is an integer below 2^24, so any correct
    summation order gives the same float32 bits as the host GEMM -- a wrong kernel can never be
    timed, whatever rank it has."""
    from mlir_roller_amd import tuner
    assert TUNER_TOPK >= tuner.DEFAULT_TOPK
    arch = MI355X.from_device(device)
    launches = 0
    for i, shape in enumerate(list(bm.README_SHAPES) + [(3000, 5000, 1536)]):
        cfg = MatmulConfig(*shape, 32)
        hints = get_roller_hints(cfg, arch, topk=TUNER_TOPK, pipeline_depth=bm.PIPELINE_DEPTH)
        assert len(hints) == TUNER_TOPK
        A, B = go.make_inputs(*shape, seed=i, distribution="integer")
        want = go.gemm_f32(A, B)
        dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((shape[0], shape[1]))
        for rank, hint in enumerate(hints, 1):
            say(f"shape {i}", shape, "rank", rank, hint.block_tile, hint.wave_tile, hint.mfma, hint.rstep)
            func = roller.Compiler(cfg, hint, bm.PIPELINE_DEPTH).compile()
            dC.fill_bytes(0xFF)
            func(func.grid_dims(), func.block_dims(), (dA, dB, dC))
            hip.synchronize()
            assert np.array_equal(dC.get(), want), (shape, rank, func.gemm_config.tag())
            launches += 1
    assert launches == 15 * TUNER_TOPK


def small_integer_matrix(rows, cols, seed):
    """Integer-valued float32 matrix in {-2..2} built from two short random vectors (cheap at
    billions of elements, and not constant along any row, column or diagonal)."""
    rng = np.random.default_rng(seed)
    r = rng.integers(0, 5, size=(rows, 1), dtype=np.int8)
    c = rng.integers(0, 5, size=(1, cols), dtype=np.int8)
    return ((r + c) % 5 - 2).astype(np.float32)


# One operand beyond 4 GiB each: tile base addresses need 64-bit arithmetic and the byte ranges of
# the buffer resources exceed what their 32-bit size field holds.  (M, N, K), config.
BEYOND_4GIB = [
    ("A", (65792, 256, 16384), GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 0, 3, 8, 0, 1)),
    ("B", (256, 65792, 16384), GemmConfig(256, 256, 32, 128, 128, 32, 3, 0, 0, 4, 0, 3, 8, 0, 1)),
    ("C", (32768, 32900, 32), GemmConfig(256, 256, 32, 64, 128, 32, 3, 0, 0, 4, 1, 3, 8, 0, 1)),
    ("C-staged", (32768, 32900, 40), GemmConfig(128, 128, 16, 64, 64, 32, 2, 4, 0, 4, 1)),
    # the stream-K form: segments rebased to their first K step far into A; C beyond 4 GiB, every 130th tile split in two
    ("A-streamk", (65792, 256, 16384), GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 0, 3, 8, 0, 1, 0, 2)),
    ("C-streamk", (32768, 33028, 96), GemmConfig(128, 128, 32, 64, 64, 16, 3, 0, 0, 4, 2, 3, 8, 0, 1, 0, 2)),
]


@pytest.mark.parametrize("which,shape,cfg", BEYOND_4GIB, ids=[b[0] for b in BEYOND_4GIB])
def test_operands_larger_than_4_gib(device, which, shape, cfg):
    """Maximum sizes: with entries in {-2..2} and K <= 16384 every partial sum is an integer
    below 2^24, so the float32 host GEMM is exact in any order and the comparison is bit-for-bit."""
    M, N, K = shape
    say("beyond 4 GiB:", which, shape, cfg.tag())
    assert max(M * K, K * N, M * N) * 4 > 1 << 32
    A, B = small_integer_matrix(M, K, 1), small_integer_matrix(K, N, 2)
    want = A @ B
    dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B)
    dC = DeviceArray((M, N))
    dC.fill_bytes(0xFF)
    GemmPlan(cfg).launch(dA, dB, dC, M, N, K)
    hip.synchronize()
    got = dC.get()
    del dA, dB, dC
    for r0 in range(0, M, 4096):                       # in slabs: no 4 GiB boolean temporaries
        assert np.array_equal(got[r0:r0 + 4096], want[r0:r0 + 4096]), (which, r0)


def test_vendor_baseline_is_a_correct_row_major_gemm(device):
    """The rocBLAS column of the sweep: the column-major call really computes row-major A @ B
    (non-square, so that a swapped operand or dimension shows), and the timing helper checks it."""
    from mlir_roller_amd.vendor_blas import rocblas
    M, N, K = 200, 304, 72
    A, B = go.make_inputs(M, N, K, seed=9, distribution="integer")
    dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((M, N))
    dC.fill_bytes(0xFF)
    rocblas().sgemm_row_major(dA, dB, dC, M, N, K)
    hip.synchronize()
    assert np.array_equal(dC.get(), go.gemm_f32(A, B))
    ms, gflops = roller.run_vendor_baseline(MatmulConfig(512, 768, 256, 32), repeat_times=3)
    assert ms > 0 and gflops == pytest.approx(2 * 512 * 768 * 256 * 1e-9 / (ms / 1e3), rel=1e-6)


from gemm_cases import EXTREME_SHAPES  # noqa: E402  (beside this file; the build step compiles the same kernels ahead)


@pytest.mark.parametrize("shape", EXTREME_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_extreme_aspect_ratios_through_policy(device, shape):
    """Vectors, slivers and a very long K: the policy's first hint compiles, launches and is exact
    (entries in {-2..2}, so sums stay below 2^24 even for K = 100000)."""
    M, N, K = shape
    mc = MatmulConfig(M, N, K, 32)
    hint = get_roller_hints(mc, MI355X(), topk=1)[0]
    func = roller.Compiler(mc, hint, bm.PIPELINE_DEPTH).compile()
    say("extreme", shape, func.gemm_config.tag())
    A, B = small_integer_matrix(M, K, 3), small_integer_matrix(K, N, 4)
    dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray((M, N))
    dC.fill_bytes(0xFF)
    func(func.grid_dims(), func.block_dims(), (dA, dB, dC))
    hip.synchronize()
    assert np.array_equal(dC.get(), A @ B)


def test_handle_checks_grid_and_block(device):
    cfg = MatmulConfig(512, 512, 128, 32)
    hint = get_roller_hints(cfg, MI355X(), topk=1)[0]
    func = roller.Compiler(cfg, hint).compile()
    d = DeviceArray((512, 512))
    gx, gy = func.grid_dims()
    with pytest.raises(ValueError):
        func((max(gx - 1, 0) or 1, 1), func.block_dims(), (d, d, d))   # the reference's floor-div grid would miss tiles
    with pytest.raises(ValueError):
        func((gx, gy), (32, 1), (d, d, d))
    with pytest.raises(TypeError):
        func((gx, gy), func.block_dims(), (d, d))


def test_run_eval_and_sweep_end_to_end(device, tmp_path, capsys):
    cfg = MatmulConfig(1024, 1024, 512, 32)
    hint = get_roller_hints(cfg, MI355X.from_device(device), topk=1)[0]
    func = roller.Compiler(cfg, hint, 3).compile()
    ms, gflops = roller.run_eval(func, 3, hint, repeat_times=5)
    assert ms > 0 and gflops == pytest.approx(2 * 1024 * 1024 * 512 * 1e-9 / (ms / 1e3), rel=1e-6)
    assert func.last_eval["ok"] and func.last_eval["normwise"] <= 1e-5
    assert 0 < func.last_eval["min_ms"] <= func.last_eval["median_ms"] < 10 * ms
    df = bm.benchmark([(512, 768, 256), (300, 500, 96)], topk=4, csv_path=tmp_path / "r.csv", repeat_times=3)
    assert len(df) == 2 and (tmp_path / "r.csv").exists()
    assert all(df["Best Hint"] != "N/A") and all(df["Normwise Error"] <= 1e-5)
    assert all(df["Max Abs Error"] <= df["Max Abs Bound"])
    assert all(df["Min Launch (ms)"] <= df["Median Launch (ms)"])
