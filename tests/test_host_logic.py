"""Host logic that needs no device: hint -> template parameters, the error measures, and the
sweep's failure handling (a hint that fails to compile or to verify is skipped and the best of
the rest is still reported, as in the reference's benchmark.py:41-58)."""

import numpy as np
import pytest

from mlir_roller_amd import benchmark as bm
from mlir_roller_amd import roller
from mlir_roller_amd.analyze import MatmulConfig, get_roller_hints
from mlir_roller_amd.arch import CUDA, MI355X


def test_hint_to_gemm_config_aligned_problem():
    cfg = MatmulConfig(4096, 8192, 4096, 32)
    hint = next(h for h in get_roller_hints(cfg, MI355X(), 20) if h.block_tile == [256, 256])
    g = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=2)
    assert (g.bm, g.bn, g.bk, g.wm, g.wn, g.mi) == (256, 256, hint.rstep, *hint.wave_tile, hint.mfma)
    # the reference's depth (two shared-memory buffers, benchmark.py:29) is the pipelined direct-to-LDS kernel:
    # template STAGES 3 keeps two LDS buffers too; swizzle instead of padding
    assert (g.stages, g.vec, g.edge, g.accum, g.direct, g.pad_a, g.pad_b) == (3, 4, 0, 0, 1, 0, 0)
    g3 = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=3)
    assert g3 == g                                                       # depth 3, the sweep's, is the same kernel
    g1 = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=1)
    assert (g1.stages, g1.direct) == (1, 0) and ((g1.bk + g1.pad_a) // 4) % 2 == 1   # staged: odd number of 16-byte units per LDS-A row
    assert g.threads == hint.threads and g.lds_bytes <= 160 * 1024
    assert roller.hint_to_gemm_config(cfg, hint, pipeline_depth=1).stages == 1
    assert roller.hint_to_gemm_config(cfg, hint, pipeline_depth=3).stages == 3
    assert roller.hint_to_gemm_config(cfg, hint, pipeline_depth=5).stages == 3
    assert roller.hint_to_gemm_config(cfg, hint, pipeline_depth=3).lds_bytes == 2 * hint.smem_cost   # still two LDS buffers
    assert roller.hint_to_gemm_config(cfg, hint, accumulate=True).accum == 1


def test_direct_path_needs_a_power_of_two_k_step():
    cfg = MatmulConfig(1536, 1536, 1536, 32)
    hint = get_roller_hints(cfg, MI355X(), 1)[0].clone()
    hint.rstep = 48
    g = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=3)
    assert (g.bk, g.direct, g.mi, g.pad_a) == (48, 0, 16, 8)      # 16x16x4: rows of 2 mod 4 sixteen-byte units
    hint.rstep = 64
    assert roller.hint_to_gemm_config(cfg, hint, pipeline_depth=3).direct == 1


def test_hint_to_gemm_config_ragged_problem():
    cfg = MatmulConfig(3000, 5000, 1536, 32)
    g = roller.hint_to_gemm_config(cfg, get_roller_hints(cfg, MI355X(), 1)[0])
    assert g.edge == 2 and g.vec == 4 and 1536 % g.bk == 0   # 5000 and 1536 are multiples of 4; K is a whole number of steps
    cfg = MatmulConfig(37, 53, 29, 32)
    hint = get_roller_hints(cfg, MI355X(), 1)[0]
    g = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=3)
    assert (g.edge, g.vec, g.direct, g.stages, g.pad_a) == (1, 1, 1, 3, 0)    # dword-aligned rows still go straight to LDS ...
    g = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=5)
    assert (g.edge, g.vec, g.direct, g.stages) == (1, 1, 1, 3)               # ... on two LDS buffers, whatever depth is asked for,
    g = roller.hint_to_gemm_config(MatmulConfig(37, 53, 64, 32), hint, pipeline_depth=2)
    assert (g.edge, g.vec, g.direct) == (1, 1, 1)                            # with all three extents tested (53 is odd, 64 a whole step)
    g = roller.hint_to_gemm_config(cfg, hint, pipeline_depth=1)
    assert (g.vec, g.direct, g.stages) == (1, 0, 1) and (g.mi, g.pad_a) == (16, 8)   # the unpipelined loop stages through registers: padded rows


def test_hint_from_the_a100_model_still_maps_to_wave_tiles():
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    hint = get_roller_hints(cfg, CUDA(), 1)[0]        # [128,128] / [16,8]: 128 threads = 2 waves
    g = roller.hint_to_gemm_config(cfg, hint)
    assert (g.bm, g.bn, g.wm, g.wn, g.threads) == (128, 128, 64, 128, 128)
    bad = hint.clone()
    bad.thread_tile = [128, 128]                      # one thread: not a whole wave
    with pytest.raises(ValueError):
        roller.hint_to_gemm_config(cfg, bad)


def test_gemm_errors_verdicts():
    cfg = MatmulConfig(48, 40, 64, 32)
    A, B = roller.make_inputs(cfg, seed=1)
    good = A @ B
    assert roller.gemm_errors(good, A, B)["ok"]
    bad = good.copy()
    bad[0, 0] += 0.5
    rep = roller.gemm_errors(bad, A, B)
    assert not rep["ok"] and rep["max_abs"] > rep["bound"]
    assert rep["bound"] == pytest.approx(1e-4 * 8 * float(np.abs(A).max()) * float(np.abs(B).max()))
    An, _ = roller.make_inputs(cfg, seed=1, distribution="normal")
    assert An.dtype == np.float32 and abs(float(An.mean())) < 0.2
    with pytest.raises(ValueError):
        roller.make_inputs(cfg, distribution="cauchy")


def test_run_baseline_formula(capsys):
    ms, gflops = roller.run_baseline(MatmulConfig(64, 64, 64, 32), repeat_times=2)
    assert ms > 0 and gflops == pytest.approx(2 * 64**3 * 1e-9 / (ms / 1e3), rel=1e-9)
    assert "GFLOPS=" in capsys.readouterr().out


class _FakeFunc:
    compile_ms = 5.0

    def __init__(self, hint):
        self.hint = hint
        self.last_eval = {"normwise": 1e-7, "max_abs": 1e-6, "bound": 1e-3}


def test_sweep_survives_failing_hints(monkeypatch, tmp_path):
    calls = {"compiled": 0}

    class FakeCompiler:
        def __init__(self, config, hint, depth, dump_path=None):
            self.hint = hint

        def compile(self):
            calls["compiled"] += 1
            if calls["compiled"] % 3 == 1:
                raise RuntimeError("hiprtc says no")
            return _FakeFunc(self.hint)

    def fake_eval(func, depth, hint, repeat_times=20, seed=0, distribution="uniform"):
        if hint.block_tile == [128, 128]:
            raise AssertionError("result outside tolerance")
        ms = 1.0 + 0.01 * hint.block_tile[0]
        return ms, 2 * hint.matmul_config.M * hint.matmul_config.N * hint.matmul_config.K * 1e-9 / (ms / 1e3)

    monkeypatch.setattr(bm, "Compiler", FakeCompiler)
    monkeypatch.setattr(bm, "run_eval", fake_eval)
    monkeypatch.setattr(bm, "run_baseline", lambda config, seed=0: (_ for _ in ()).throw(MemoryError("host")))
    csv = tmp_path / "out.csv"
    df = bm.benchmark([(2048, 2048, 2048), (4096, 8192, 4096)], topk=6, csv_path=csv)
    assert len(df) == 2 and csv.exists()
    r = df.iloc[0]
    assert r["Hints Tried"] == 6 and r["Hints Failed"] >= 2
    assert r["Host Time (ms)"] == float("inf") and r["Host GFLOPS"] == 0 and r["Speedup vs Host"] == 0
    assert r["Roller Time (ms)"] < float("inf") and r["Best Hint"] != "N/A" and r["Best Hint Rank"] >= 1
    assert r["% of fp32 matrix peak"] == pytest.approx(100 * r["Roller TFLOPS"] / 157.3, rel=1e-3)
    for col in ("M", "N", "K", "Roller Time (ms)", "Roller GFLOPS", "Best Hint"):   # the reference's columns
        assert col in df.columns


def test_sweep_merges_counter_columns_and_collects_them_first(monkeypatch):
    order = []

    class FakeCompiler:
        def __init__(self, config, hint, depth, dump_path=None):
            self.hint = hint

        def compile(self):
            order.append("compile")
            return _FakeFunc(self.hint)

    def fake_collect(shapes):
        order.append("counters")
        return {tuple(s): {"MfmaUtil %": 95.0, "LdsBankConflict": 0.0, "HBM-side GB/s": 510.0} for s in shapes}

    monkeypatch.setattr(bm, "Compiler", FakeCompiler)
    monkeypatch.setattr(bm, "run_eval", lambda func, depth, hint, **k: (1.0, 1000.0))
    monkeypatch.setattr(bm, "collect_counters", fake_collect)
    df = bm.benchmark([(2048, 2048, 2048)], topk=2, baseline=False, csv_path=None, counters=True)
    assert order[0] == "counters" and "compile" in order           # profiled child runs come before any GPU work here
    assert df.iloc[0]["MfmaUtil %"] == 95.0 and df.iloc[0]["LdsBankConflict"] == 0.0 and df.iloc[0]["HBM-side GB/s"] == 510.0
    plain = bm.benchmark([(2048, 2048, 2048)], topk=1, baseline=False, csv_path=None)
    assert "MfmaUtil %" not in plain.columns


def test_counter_collection_refuses_an_initialised_process(monkeypatch):
    from mlir_roller_amd import hip
    monkeypatch.setattr(hip, "_initialised", True)
    with pytest.raises(RuntimeError, match="before this process initialises the GPU"):
        bm.collect_counters([(2048, 2048, 2048)])


def test_sweep_vendor_columns(monkeypatch):
    class FakeCompiler:
        def __init__(self, config, hint, depth, dump_path=None):
            self.hint = hint

        def compile(self):
            return _FakeFunc(self.hint)

    monkeypatch.setattr(bm, "Compiler", FakeCompiler)
    monkeypatch.setattr(bm, "run_eval", lambda func, depth, hint, **k: (2.0, 1000.0))
    monkeypatch.setattr(bm, "run_vendor_baseline", lambda config, seed=0: (3.0, 700.0))
    df = bm.benchmark([(2048, 2048, 2048)], topk=1, baseline=False, csv_path=None, vendor=True)
    r = df.iloc[0]
    assert r["rocBLAS Time (ms)"] == 3.0 and r["rocBLAS GFLOPS"] == 700.0 and r["Speedup vs rocBLAS"] == pytest.approx(1.5)

    def broken(config, seed=0):
        raise OSError("librocblas.so missing")
    monkeypatch.setattr(bm, "run_vendor_baseline", broken)          # a missing library never ends the sweep
    r = bm.benchmark([(2048, 2048, 2048)], topk=1, baseline=False, csv_path=None, vendor=True).iloc[0]
    assert r["rocBLAS Time (ms)"] == float("inf") and r["Speedup vs rocBLAS"] == 0
    assert "rocBLAS GFLOPS" not in bm.benchmark([(2048, 2048, 2048)], topk=1, baseline=False, csv_path=None).columns


def test_sweep_reports_all_failed(monkeypatch):
    class AlwaysFails:
        def __init__(self, *a, **k):
            pass

        def compile(self):
            raise RuntimeError("nope")

    monkeypatch.setattr(bm, "Compiler", AlwaysFails)
    df = bm.benchmark([(2048, 2048, 2048)], topk=3, baseline=False, csv_path=None)
    assert df.iloc[0]["Best Hint"] == "N/A" and df.iloc[0]["Roller GFLOPS"] == 0


def test_readme_shapes_are_the_fourteen():
    assert len(bm.README_SHAPES) == 14 and bm.README_SHAPES[0] == (2048, 2048, 2048)
    assert bm.README_SHAPES[10] == (4096, 8192, 4096) and bm.README_SHAPES[13] == (8192, 4096, 4096)
    assert all(d in (2048, 4096, 8192) for s in bm.README_SHAPES for d in s)


def test_plot_results_writes_an_image(tmp_path):
    import pandas as pd
    df = pd.DataFrame({"Roller TFLOPS": [139.0, 148.5, 120.0], "Speedup vs Host": [37.0, 40.2, 0]})
    out = bm.plot_results(df, tmp_path / "sweep.png")
    assert out.exists() and out.stat().st_size > 5000 and out.read_bytes()[:4] == b"\x89PNG"


def test_vendor_library_missing_is_reported_not_fatal(tmp_path):
    from mlir_roller_amd.vendor_blas import RocBLAS, VendorBlasError
    with pytest.raises(VendorBlasError, match="cannot load rocBLAS"):
        RocBLAS(library=str(tmp_path / "librocblas.so"))


@pytest.mark.parametrize("depth", [1, 2, 3])
@pytest.mark.parametrize("trans_b", [False, True])
def test_every_hint_fits_the_kernel_at_every_pipeline_depth(hip_lib, depth, trans_b):
    # the policy's LDS model follows the depth: padded rows and two buffers at depth 2, swizzled
    # unpadded rows at depth 3; no emitted hint may be refused by the library's own check
    from mlir_roller_amd import hip
    shapes = list(bm.README_SHAPES) + [(3000, 5000, 1536), (1000, 1000, 1000), (1022, 1018, 1002), (37, 53, 29)]
    for shape in shapes:
        cfg = MatmulConfig(*shape, 32)
        hints = get_roller_hints(cfg, MI355X(), 20, pipeline_depth=depth)
        assert hints, shape
        for hint in hints:
            g = roller.hint_to_gemm_config(cfg, hint, depth, trans_b=trans_b)
            lds, threads = hip.config_check(g)
            assert lds <= 160 * 1024 and threads == hint.threads
            if not trans_b:
                assert lds == min(depth, 2) * hint.smem_cost, (shape, hint)   # the model is exact, not just safe


def test_a_hint_ranked_for_another_depth_still_fits(hip_lib):
    # Compiler(config, hint, 2) with a hint that the policy sized for depth 3: padding is dropped
    # where it would overflow the CU's LDS
    from mlir_roller_amd import hip
    cfg = MatmulConfig(2048, 2048, 2048, 32)
    for hint in get_roller_hints(cfg, MI355X(), 20, pipeline_depth=3):
        for trans_b in (False, True):
            hip.config_check(roller.hint_to_gemm_config(cfg, hint, 2, trans_b=trans_b))


def test_kernel_arguments_are_typed_by_type_not_by_value():
    import ctypes as C
    from mlir_roller_amd import hip
    assert C.sizeof(hip._pack_arg(hip.Ptr(0))) == 8 and hip._pack_arg(hip.Ptr(0)).value is None   # NULL stays a pointer
    assert C.sizeof(hip._pack_arg(hip.Ptr(4096))) == 8
    # what array.ptr / array.data.ptr are: an int that launches pass as an address, as the reference's call
    # func(grid, block, (dA.data.ptr, ...)) expects (roller.py:545-550)
    small_address = hip.DevicePtr(4096)
    assert isinstance(small_address, int) and small_address + 16 == 4112
    assert C.sizeof(hip._pack_arg(small_address)) == 8 and hip._pack_arg(small_address).value == 4096
    assert hip._DataView(4096).ptr == 4096 and isinstance(hip._DataView(4096).ptr, hip.DevicePtr)
    with hip.profiler_range("a range no profiler listens to"):
        pass
    for small in (0, 7, -1, 2**31 - 1, np.int64(12)):
        packed = hip._pack_arg(small)
        assert isinstance(packed, C.c_int) and C.sizeof(packed) == 4      # a bare int is never a pointer
    for wide in (2**31, 2**40, 0x7F0000000000, -2**31 - 1):
        with pytest.raises(OverflowError):
            hip._pack_arg(wide)
    assert isinstance(hip._pack_arg(C.c_long(2**40)), C.c_long)
    assert isinstance(hip._pack_arg(1.5), C.c_float)
    with pytest.raises(TypeError):
        hip._pack_arg(True)
    with pytest.raises(TypeError):
        hip._pack_arg("x")
    with pytest.raises(ValueError):
        hip.Ptr(-1)


def test_tuner_keeps_the_policys_order_on_near_ties():
    from mlir_roller_amd import tuner
    assert tuner.DEFAULT_TOPK <= 4                                                 # the reference tries 20
    assert tuner.choose([(1, 1.000), (2, 0.997), (3, 0.996)]) == 1                 # within the spread: rank 1 stays
    assert tuner.choose([(1, 1.000), (2, 0.985), (3, 0.984)]) == 2                 # 1.5 % faster displaces; 0.1 % more does not
    assert tuner.choose([(3, 0.90), (1, 1.0), (2, 0.97)]) == 3                     # order of the list does not matter
    assert tuner.choose([(1, 1.0), (2, 0.97), (3, 0.90)]) == 3
    assert tuner.choose([(1, float("nan")), (2, 2.0), (3, float("inf")), (4, 0.0)]) == 2   # unusable timings are skipped
    assert tuner.choose([]) == -1 and tuner.choose([(1, float("nan"))]) == -1
    assert tuner.choose([(1, 1.0), (2, 0.996)], margin=0.0) == 2                   # margin 0: plain fastest
    s = tuner.summarise([(1, 1.0), (2, 0.997), (3, 0.996)], 1)
    assert s == {"kept_rank": 1, "fastest_rank": 3, "kept_over_fastest": 1.004, "top1_over_fastest": 1.004}
    assert tuner.ramp_launches((2048, 2048, 2048)) >= 250 and tuner.ramp_launches((8192, 8192, 8192), 3) >= 5


def test_sweep_applies_the_tie_rule(monkeypatch, tmp_path):
    # three hints, the third 0.3 % faster than the first: the first is reported
    times = iter([1.000, 1.002, 0.997])

    class Fake:
        compile_ms = 0.0
        last_eval = {}

    monkeypatch.setattr(bm, "Compiler", lambda *a, **k: type("C", (), {"compile": lambda self: Fake()})())
    monkeypatch.setattr(bm, "run_eval", lambda *a, **k: (next(times), 1.0))
    df = bm.benchmark([(2048, 2048, 2048)], topk=3, baseline=False, csv_path=None)
    assert int(df["Best Hint Rank"][0]) == 1 and float(df["Roller Time (ms)"][0]) == 1.000
