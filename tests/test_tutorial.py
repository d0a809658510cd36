"""The teaching ladder (C = A*B + 1): every rung compiles for gfx950 without a GPU; on the GPU
every rung is exact on integer inputs for square and non-square static shapes (the check the
reference's tutorial applies, /root/reference/src/cuda_matmul_opt.py:275-296)."""

import numpy as np
import pytest

from mlir_roller_amd import hip, tutorial
from mlir_roller_amd.tutorial import LADDER, RUNGS


def test_ladder_lists_the_reference_rungs_in_order():
    names = [r.name for r in LADDER]
    assert names[:8] == ["sgemm_naive", "sgemm_naive_row_order", "sgemm_coalesce", "sgemm_coalesce_transpose_B",
                         "sgemm_shared_mem_block", "sgemm_shared_mem_1d_block_tiling",
                         "sgemm_shared_mem_2d_block_tiling", "sgemm_shared_mem_2d_block_tiling_vectorize"]
    assert names[8:] == ["sgemm_wave_tiling", "sgemm_mfma"]
    assert [r.name for r in LADDER if r.transpose_b] == ["sgemm_coalesce_transpose_B"]


@pytest.mark.parametrize("size", [(128, 128, 128), (256, 64, 384)])
def test_every_rung_compiles_for_gfx950(hip_lib, size):
    M, K, N = size
    source = tutorial.LADDER_SOURCE.read_text()
    for rung in LADDER:
        opts = tutorial.kernel_options(rung.name, M, K, N, rung.params(M, K, N))
        code, _ = hip.compile_source(source, "sgemm_ladder.hip", opts)
        present = [other.name for other in LADDER if (other.name + "\0").encode() in code]
        assert present == [rung.name]                            # one kernel per translation unit


def test_geometry_matches_the_tile_parameters():
    for rung in LADDER:
        p = rung.params(1024, 1024, 1024)
        grid, block, lds = rung.geometry(1024, 1024, 1024, p)
        threads = int(np.prod(block))
        assert threads % 64 == 0 and threads <= 1024 and lds <= 64 * 1024, rung.name
        if "BM" in p:
            assert grid == (1024 // p["BN"], 1024 // p["BM"])
            assert lds == (p["BM"] * p["BK"] + p["BK"] * p["BN"]) * 4
    p = RUNGS["sgemm_shared_mem_2d_block_tiling"].params(64, 64, 64)
    assert (p["BM"], p["BN"]) == (64, 64)                       # small problems take the small tile
    p = RUNGS["sgemm_wave_tiling"].params(512, 512, 512)
    passes_m = p["WM"] * p["WN"] // (64 * p["TM"] * p["TN"] * p["WNITER"])
    assert (p["WM"] // passes_m // p["TM"]) * (p["WN"] // p["WNITER"] // p["TN"]) == 64   # lanes per pass


def test_prepare_refuses_sizes_the_tiles_do_not_divide():
    for name, size in (("sgemm_naive", (100, 64, 64)), ("sgemm_shared_mem_block", (64, 48, 64)),
                       ("sgemm_shared_mem_2d_block_tiling", (192, 64, 128)), ("sgemm_wave_tiling", (128, 24, 128)),
                       ("sgemm_mfma", (64, 3, 64)), ("sgemm_coalesce", (0, 32, 32))):
        with pytest.raises(ValueError):
            tutorial.prepare(name, *size)


@pytest.mark.gpu
@pytest.mark.parametrize("name", [r.name for r in LADDER])
def test_every_rung_is_exact_on_integer_inputs(device, name):
    for M, K, N in ((128, 128, 128), (256, 64, 384), (384, 160, 128)):
        print(name, (M, K, N), flush=True)
        assert tutorial.run_eval(M, K, N, *tutorial.prepare(name, M, K, N), repeat_times=0, seed=M + N) is None
    ms, gflops = tutorial.run_eval(512, 512, 512, *tutorial.prepare(name, 512, 512, 512), repeat_times=3)
    assert ms > 0 and gflops == pytest.approx(2 * 512 ** 3 * 1e-9 / (ms / 1e3), rel=1e-6)
