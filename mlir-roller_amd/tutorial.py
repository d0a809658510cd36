"""The teaching ladder of fp32 kernels (C = A*B + 1), compiled and run through the same low-level
calls as the GEMM path: ``rl_compile`` (hiprtc) -> ``rl_module_load`` -> ``rl_module_get_function``
-> ``rl_launch``.

Counterpart of /root/reference/src/cuda_matmul_opt.py: ``prepare_*`` there lowers one MLIR kernel
for static (M, K, N) and returns ``(cuda_func, grid_dims, block_dims, shared_mem, npy_dtype,
transpose_B)`` (:128-257); ``run_eval`` checks ``C == A @ B + 1`` exactly on integer inputs, then
times ``repeat_times`` launches between two events (:260-315).  ``prepare`` and ``run_eval`` here
keep those shapes; the kernels are HIP (csrc/sgemm_ladder.hip), sized for 64-lane wavefronts, and
two rungs are added at the top (wave tiling, MFMA).  The kernels are not bounds-checked, so
``prepare`` refuses sizes that a rung's tiles do not divide.
"""

from __future__ import annotations

import argparse
from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import numpy as np

from . import hip
from .hip import DeviceArray, Event, Function, Module

LADDER_SOURCE = hip.CSRC_DIR / "sgemm_ladder.hip"


@dataclass(frozen=True)
class Rung:
    """One kernel of the ladder: its tile parameters for a size, launch geometry and LDS bytes."""
    name: str
    params: Callable[[int, int, int], Dict[str, int]]
    geometry: Callable[[int, int, int, Dict[str, int]], Tuple[tuple, tuple, int]]
    divisors: Callable[[Dict[str, int]], Tuple[int, int, int]]      # what M, N, K must be multiples of
    transpose_b: bool = False


def _square(M, K, N):
    return {"BLOCK": 32}


def _square_geometry(shared: bool, by_columns: bool = False):
    def geometry(M, K, N, p):
        b = p["BLOCK"]
        grid = (N // b, M // b) if by_columns else (M // b, N // b)
        return grid, (b, b), (2 * b * b * 4 if shared else 0)
    return geometry


def _tiled_1d(M, K, N):
    return {"BM": 64, "BN": 64, "BK": 8, "TM": 8}


def _tiled_2d(M, K, N):
    big = M >= 128 and N >= 128          # the reference's choice (cuda_matmul_opt.py:176-181)
    return {"BM": 128 if big else 64, "BN": 128 if big else 64, "BK": 8, "TM": 8, "TN": 8}


def _wave_tiled(M, K, N):
    # 2 x 2 waves of 64 x 64; a lane holds 2 x 2 passes of 4 x 4 results (8 x 8 lanes per 32 x 32 pass)
    return {"BM": 128, "BN": 128, "BK": 16, "WM": 64, "WN": 64, "WNITER": 2, "TM": 4, "TN": 4}


def _tile_geometry(threads: Callable[[Dict[str, int]], tuple]):
    def geometry(M, K, N, p):
        lds = (p["BM"] * p["BK"] + p["BK"] * p["BN"]) * 4
        return (N // p["BN"], M // p["BM"]), threads(p), lds
    return geometry


_tile_divisors = lambda p: (p["BM"], p["BN"], max(p["BK"], 4))

LADDER = [
    Rung("sgemm_naive", _square, _square_geometry(False), lambda p: (p["BLOCK"], p["BLOCK"], 1)),
    Rung("sgemm_naive_row_order", _square, _square_geometry(False, by_columns=True), lambda p: (p["BLOCK"], p["BLOCK"], 1)),
    Rung("sgemm_coalesce", _square, _square_geometry(False), lambda p: (p["BLOCK"], p["BLOCK"], 1)),
    Rung("sgemm_coalesce_transpose_B", _square, _square_geometry(False), lambda p: (p["BLOCK"], p["BLOCK"], 1), True),
    Rung("sgemm_shared_mem_block", _square, _square_geometry(True), lambda p: (p["BLOCK"], p["BLOCK"], p["BLOCK"])),
    Rung("sgemm_shared_mem_1d_block_tiling", _tiled_1d,
         _tile_geometry(lambda p: (p["BM"] // p["TM"], p["BN"])), _tile_divisors),
    Rung("sgemm_shared_mem_2d_block_tiling", _tiled_2d,
         _tile_geometry(lambda p: (p["BM"] // p["TM"], p["BN"] // p["TN"])), _tile_divisors),
    Rung("sgemm_shared_mem_2d_block_tiling_vectorize", _tiled_2d,
         _tile_geometry(lambda p: (p["BM"] // p["TM"], p["BN"] // p["TN"])), _tile_divisors),
    Rung("sgemm_wave_tiling", _wave_tiled,
         _tile_geometry(lambda p: (64 * (p["BM"] // p["WM"]) * (p["BN"] // p["WN"]),)), _tile_divisors),
    Rung("sgemm_mfma", lambda M, K, N: {}, lambda M, K, N, p: ((N // 64, M // 64), (256,), 0), lambda p: (64, 64, 2)),
]
RUNGS = {r.name: r for r in LADDER}


def kernel_options(kernel: str, M: int, K: int, N: int, params: Dict[str, int]):
    """hiprtc defines for one rung: the static shape, which kernel of the file to build, its tiles."""
    rung = [r.name for r in LADDER].index(kernel) + 1
    return [f"-D{k}={v}" for k, v in {"M": M, "K": K, "N": N, "RUNG": rung, **params}.items()]


def prepare(kernel: str, M: int, K: int, N: int):
    """Compiles one rung for a static size and returns what the reference's ``prepare_*`` return:
    ``(cuda_func, grid_dims, block_dims, shared_mem, npy_dtype, transpose_B)``."""
    rung = RUNGS[kernel]
    params = rung.params(M, K, N)
    dm, dn, dk = rung.divisors(params)
    if M <= 0 or N <= 0 or K <= 0 or M % dm or N % dn or K % dk:
        raise ValueError(f"{kernel} needs M, N, K to be positive multiples of {dm}, {dn}, {dk}; got {M}, {N}, {K}")
    if max(M * K, K * N, M * N) >= 2 ** 31:
        raise ValueError("the ladder kernels index with 32-bit integers")
    code, _ = hip.compile_source(LADDER_SOURCE.read_text(), "sgemm_ladder.hip", kernel_options(kernel, M, K, N, params))
    func = Module(code).get_function(kernel)
    grid_dims, block_dims, shared_mem = rung.geometry(M, K, N, params)
    return func, grid_dims, block_dims, shared_mem, np.float32, rung.transpose_b


def run_eval(M: int, K: int, N: int, cuda_func: Function, grid_dims, block_dims, shared_mem: int,
             npy_dtype, transpose_B: bool, repeat_times: Optional[int] = None, seed: int = 0):
    """Exact check on integer-valued inputs (every partial sum stays below 2^24, so any summation
    order gives the same bits), then ``repeat_times`` timed launches (default 50; below 1 skips
    the timing).  Returns ``(ms_per_launch, gflops)`` or ``None``."""
    if repeat_times is None:
        repeat_times = 50
    if 81 * K >= 2 ** 24:
        raise ValueError("K too large for the exact integer check")
    rng = np.random.default_rng(seed)
    A = rng.integers(0, 10, (M, K)).astype(npy_dtype)
    B = rng.integers(0, 10, (K, N)).astype(npy_dtype)
    dA = DeviceArray.from_host(A)
    dB = DeviceArray.from_host(np.ascontiguousarray(B.T) if transpose_B else B)
    dC = DeviceArray.zeros((M, N), npy_dtype)
    args = (dA, dB, dC)
    cuda_func(grid_dims, block_dims, args, shared_mem=shared_mem)
    hip.synchronize()
    C = dC.get()
    if not np.array_equal(C, A @ B + 1):
        raise AssertionError(f"kernel result differs from A @ B + 1 (max |diff| {np.max(np.abs(C - (A @ B + 1)))})")
    if repeat_times < 1:
        return None
    start, end = Event(), Event()
    start.record()
    for _ in range(repeat_times):
        cuda_func(grid_dims, block_dims, args, shared_mem=shared_mem)
    end.record()
    end.synchronize()
    t_gpu = hip.get_elapsed_time(start, end)
    gflops = repeat_times * 2 * M * N * K * 1e-9 / (t_gpu / 1000)
    print(f"t={t_gpu / repeat_times:.6f} ms GFLOPS={gflops:.6f}")
    return t_gpu / repeat_times, gflops


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description="fp32 matmul teaching ladder on MI355X")
    ap.add_argument("--sizes", type=int, nargs="+", default=[1024])
    ap.add_argument("--kernels", nargs="+", default=[r.name for r in LADDER], choices=list(RUNGS))
    ap.add_argument("--repeats", type=int, default=None)
    args = ap.parse_args(argv)
    hip.init(0)
    for name in args.kernels:
        print(f"\n{name}")
        for s in args.sizes:
            print(f"{s=}", end=" ")
            run_eval(s, s, s, *prepare(name, s, s, s), repeat_times=args.repeats)


if __name__ == "__main__":
    main()
