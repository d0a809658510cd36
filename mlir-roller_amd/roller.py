"""Compile, launch and time one Roller hint on MI355X.

Keeps the call surface of /root/reference/src/roller.py -- ``Compiler(config, hint,
pipeline_depth, dump_path).compile()`` (:345-387), the returned handle's
``f(grid, block, (ptrA, ptrB, ptrC), shared_mem=)`` (:545-550), ``time_cuda`` (:514-522),
``run_eval`` (:525-586) and ``run_baseline`` (:589-607) -- and replaces what is behind it:
instead of building a linalg.matmul plus a transform-dialect schedule, lowering it to PTX and
loading that with CuPy, the hint selects the parameters of a hand-written gfx950 kernel template
that libroller_hip.so JIT-compiles with hiprtc, caches, loads and launches.
"""

from __future__ import annotations

import json
import shutil
import subprocess
import time
from contextlib import contextmanager
from pathlib import Path
from typing import Optional, Tuple

import numpy as np

from . import hip
from .analyze import (MatmulConfig, TileDict, get_roller_hints, kernel_stages, lds_row_pad, loads_go_direct_to_lds,
                      split_block_over_waves)
from .arch import MI355X
from .hip import DeviceArray, Event, GemmConfig, GemmPlan
from .utils import get_block_dims

KERNEL_NAME = "gemm_kernel"  # the symbol the reference looks up (roller.py:499)

# numerical gates of the GEMM path
NORMWISE_TOL = 1e-5          # ||C - C32||_F / ||C32||_F against a float32 host GEMM
ELEMENTWISE_FACTOR = 1e-4    # max|C - C64| <= factor * sqrt(K) * max|A| * max|B| against float64
WARMUP_MS = 40.0             # load queued ahead of the timed launches of run_eval


def hint_to_gemm_config(config: MatmulConfig, hint: TileDict, pipeline_depth: int = 2,
                        accumulate: bool = False, trans_b: bool = False) -> GemmConfig:
    """Template parameters for one hint.

    block_tile -> BM, BN; rstep -> BK; wave_tile -> WM, WN (derived from the thread count when
    the hint comes from a device model without matrix cores); pipeline_depth -> pipeline stages
    (``kernel_stages``: the reference's depth 2 and the sweep's depth 3 are the same kernel, two LDS
    buffers and the pipelined loop; 4 and 5 add buffers).  Ragged problems switch on predication, and
    problems whose K, N are not multiples of 4 get the kernel for dword-aligned rows (vec=1; it keeps
    the direct-to-LDS loads with two LDS buffers).  ``trans_b`` selects the kernel
    whose second operand is stored as Bt[N, K].
    """
    bm, bn = hint.block_tile
    bk = hint.rstep
    if hint.wave_tile:
        (wm, wn), mi = hint.wave_tile, hint.mfma
    else:
        threads = 1
        for d in get_block_dims(hint.block_tile + [0], hint.thread_tile + [0]):
            threads *= d
        if threads % 64:
            raise ValueError(f"{threads} threads per block is not a whole number of 64-lane waves")
        split = split_block_over_waves(hint.block_tile, threads // 64, bk, MI355X())
        if split is None:
            raise ValueError(f"block tile {hint.block_tile} cannot be split into MFMA wave tiles "
                             f"for {threads} threads and reduce step {bk}")
        (wm, wn), mi = split
    M, N, K = config.M, config.N, config.K
    stages = min(GemmConfig.MAX_STAGES, kernel_stages(pipeline_depth))
    vec = 4 if (K % 4 == 0 and N % 4 == 0) else 1
    # Depths 4 and 5 (three and four LDS buffers) exist on the direct-to-LDS path only, for tiles
    # that divide evenly over the threads and fit the CU's LDS; otherwise the deepest depth that
    # does fit is taken.
    threads = 64 * (bm // wm) * (bn // wn)
    while stages > 3:
        loads = (bm * bk // 4) // threads + (bk * bn // 4) // threads
        if (loads_go_direct_to_lds(config, (bm, bn), bk, stages) and (bm * bk // 4) % threads == 0
                and (bk * bn // 4) % threads == 0 and (stages - 3) * loads <= 63
                and (stages - 1) * (bm * bk + bk * bn) * 4 <= MI355X().lds_bytes):
            break
        stages -= 1
    # On the pipelined loop the global loads go straight to LDS (swizzled A rows, no padding)
    # whenever both operand tiles are whole waves of 16-byte units and the K step is a power of
    # two (the swizzle is an XOR).
    direct = int(loads_go_direct_to_lds(config, (bm, bn), bk, stages))
    # otherwise padded rows keep the 128-bit reads of LDS-A free of bank conflicts
    pad_a = 0 if direct else lds_row_pad(bk, mi)
    # a transposed second operand sits in LDS like A and wants the same padding
    pad_b = pad_a if trans_b else 0
    # Padding is an optimisation, fitting the CU is not: a hint whose policy ran for another depth
    # or layout may leave no room for it.
    lds_cap = MI355X().lds_bytes
    buffers = stages - 1 if stages >= 3 else stages
    footprint = lambda pa, pb: buffers * (bm * (bk + pa) + (bn * (bk + pb) if trans_b else bk * (bn + pb))) * 4
    if pad_b and footprint(pad_a, pad_b) > lds_cap:
        pad_b = 0
    if pad_a and footprint(pad_a, pad_b) > lds_cap:
        pad_a = 0
    return GemmConfig(
        bm=bm, bn=bn, bk=bk, wm=wm, wn=wn, mi=mi, stages=stages, pad_a=pad_a, pad_b=pad_b, vec=vec,
        # 0: every extent is a whole number of tiles; 2: only M or N is ragged; 1: K is ragged too
        # (the direct-to-LDS loads of dword-aligned rows come with all three tests)
        edge=(0 if (M % bm == 0 and N % bn == 0) else 2) if K % bk == 0 and not (direct and vec == 1) else 1,
        swz=3, group=8, accum=1 if accumulate else 0, direct=direct, trans_b=1 if trans_b else 0,
        # the stream-K form of the kernel exists on the pipelined loop only
        streamk=int(getattr(hint, "stream_k", 0)) if stages == 3 else 0,
    )


class KernelHandle:
    """What ``Compiler.compile()`` returns: a loaded GEMM kernel that is called like the
    reference's ``cp.cuda.Function``::

        func(grid_dims, block_dims, (ptrA, ptrB, ptrC), shared_mem=nbytes)

    The three pointers are device addresses (ints or ``DeviceArray``).  The kernel takes the
    problem size at run time, so the handle appends M, N, K and the leading dimensions of the
    ``MatmulConfig`` it was compiled for (pass nine arguments to override them).  ``grid_dims``
    and ``block_dims`` are checked -- the grid must cover ceil(N/bn) x ceil(M/bm) tiles and the
    block must hold the kernel's thread count -- while the launch itself uses the geometry and
    the (padded) LDS size of the compiled plan.
    """

    def __init__(self, plan: GemmPlan, config: MatmulConfig, gemm_config: GemmConfig, hint: TileDict):
        self.plan = plan
        self.config = config
        self.gemm_config = gemm_config
        self.hint = hint
        self.compile_ms = plan.compile_ms
        self.last_eval: dict = {}

    @property
    def shared_mem_bytes(self) -> int:
        return self.plan.lds_bytes

    @property
    def threads(self) -> int:
        return self.plan.threads

    def grid_dims(self) -> Tuple[int, int]:
        c, g = self.config, self.gemm_config
        return (-(-c.N // g.bn), -(-c.M // g.bm))

    def block_dims(self) -> Tuple[int, int]:
        x, y, _ = get_block_dims(self.hint.block_tile + [0], self.hint.thread_tile + [0])
        return (x, y) if x * y == self.plan.threads else (self.plan.threads, 1)

    def __call__(self, grid_dims, block_dims, args, shared_mem: int = 0, stream=None) -> None:
        if len(args) == 3:
            c = self.config
            dims = (c.M, c.N, c.K, c.K, c.K if self.gemm_config.trans_b else c.N, c.N)
        elif len(args) == 9:
            dims = tuple(int(v) for v in args[3:])
        else:
            raise TypeError("args must be (A, B, C) or (A, B, C, M, N, K, lda, ldb, ldc)")
        M, N, K, lda, ldb, ldc = dims
        g = self.gemm_config
        need = (-(-N // g.bn)) * (-(-M // g.bm))
        have = 1
        for d in grid_dims:
            have *= int(d)
        if have < need:
            raise ValueError(f"grid {tuple(grid_dims)} has {have} workgroups, the problem needs {need}")
        lanes = 1
        for d in block_dims:
            lanes *= int(d)
        if lanes != self.plan.threads:
            raise ValueError(f"block {tuple(block_dims)} has {lanes} threads, the kernel needs {self.plan.threads}")
        self.plan.launch(args[0], args[1], args[2], M, N, K, lda, ldb, ldc, stream=stream)


class Compiler:
    """Same constructor and ``compile()`` as the reference's ``Compiler`` (roller.py:345-387).

    ``dump_path`` receives ``kernel.hip`` (template source with the chosen parameters as
    defines), ``kernel.json`` (parameters and register/LDS usage), ``build.log`` (what hiprtc
    printed for this kernel, or a line saying that the code object came from the cache) and, when
    ``hipcc`` is on the PATH, ``kernel.s`` (gfx950 assembly) -- the counterparts of the reference's
    ``transformed.mlir`` / ``llvm.mlir`` / ``kernel.ptx`` dumps (roller.py:369-371, :480-495, :502).
    """

    def __init__(self, config: MatmulConfig, hint: TileDict, pipeline_depth: int = 2,
                 dump_path: Optional[Path] = None, accumulate: bool = False, trans_b: bool = False):
        self.config = config
        self.hint = hint
        self.pipeline_depth = pipeline_depth
        self.dump_path = Path(dump_path) if dump_path else None
        self.accumulate = accumulate
        self.trans_b = trans_b

    def compile(self) -> KernelHandle:
        gemm_config = hint_to_gemm_config(self.config, self.hint, self.pipeline_depth, self.accumulate, self.trans_b)
        hip.config_check(gemm_config)
        plan = GemmPlan(gemm_config)
        handle = KernelHandle(plan, self.config, gemm_config, self.hint)
        if self.dump_path:
            self._dump(handle)
        return handle

    def _dump(self, handle: KernelHandle) -> None:
        out = self.dump_path
        out.mkdir(parents=True, exist_ok=True)
        g = handle.gemm_config
        defines = {k.upper(): v for k, v in vars(g).items()}
        header = "".join(f"#define {k} {v}\n" for k, v in defines.items())
        (out / "kernel.hip").write_text(header + hip.template_source())
        info = {"config": vars(g), "lds_bytes": handle.shared_mem_bytes, "threads": handle.threads,
                "resources": handle.plan.resources(), "compile_ms": handle.compile_ms}
        (out / "kernel.json").write_text(json.dumps(info, indent=1))
        log = handle.plan.build_log()
        if not log:
            log = ("(no compiler output: the code object came from the in-process or on-disk cache)\n" if handle.compile_ms == 0
                   else "(hiprtc compiled this kernel without a message)\n")
        (out / "build.log").write_text(log)
        hipcc = shutil.which("hipcc")
        if hipcc:
            subprocess.run([hipcc, "--offload-arch=gfx950", "-O3", "--cuda-device-only", "-S",
                            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                            str(out / "kernel.hip"), "-o", str(out / "kernel.s")],
                           check=False, capture_output=True)


@contextmanager
def time_cuda(stream=None):
    """Event pair around a region (name kept from roller.py:514-522); read the result with
    ``hip.get_elapsed_time(start, end)`` after the block."""
    start, end = Event(), Event()
    start.record(stream)
    yield start, end
    end.record(stream)
    end.synchronize()


time_hip = time_cuda


def make_inputs(config: MatmulConfig, seed: int = 0, distribution: str = "uniform"):
    """Seeded row-major fp32 operands: uniform[-1, 1), standard normal, or small integers
    (0..9, for which every fp32 partial sum is exact and any summation order agrees bitwise)."""
    rng = np.random.default_rng(seed)
    shape_a, shape_b = (config.M, config.K), (config.K, config.N)
    if distribution == "uniform":
        draw = lambda s: rng.uniform(-1.0, 1.0, s).astype(np.float32)
    elif distribution == "normal":
        draw = lambda s: rng.standard_normal(s, dtype=np.float32)
    elif distribution == "integer":
        draw = lambda s: rng.integers(0, 10, s).astype(np.float32)
    else:
        raise ValueError(f"unknown distribution {distribution!r}")
    return draw(shape_a), draw(shape_b)


def gemm_errors(C: np.ndarray, A: np.ndarray, B: np.ndarray, C32: Optional[np.ndarray] = None,
                C64: Optional[np.ndarray] = None) -> dict:
    """Both error measures of the path and their verdicts: normwise against a float32 host GEMM,
    elementwise against a float64 host GEMM (either may be passed in when already computed)."""
    if C32 is None:
        C32 = A @ B
    K = A.shape[1]
    ref_norm = float(np.linalg.norm(C32.astype(np.float64)))
    normwise = float(np.linalg.norm(C.astype(np.float64) - C32.astype(np.float64))) / max(ref_norm, 1e-300)
    if C64 is None:
        C64 = A.astype(np.float64) @ B.astype(np.float64)
    max_abs = float(np.max(np.abs(C.astype(np.float64) - C64))) if C.size else 0.0
    amax = float(np.max(np.abs(A))) if A.size else 0.0
    bmax = float(np.max(np.abs(B))) if B.size else 0.0
    bound = ELEMENTWISE_FACTOR * np.sqrt(max(K, 1)) * amax * bmax
    return {"normwise": normwise, "max_abs": max_abs, "bound": float(bound),
            "ok": bool(normwise <= NORMWISE_TOL and max_abs <= bound)}


_reference_cache: dict = {}


def _host_case(config: MatmulConfig, seed: int, distribution: str):
    """Inputs and float32 host result for a shape; the last one is kept because a sweep
    evaluates up to ``topk`` hints on the same shape."""
    key = (config.M, config.N, config.K, seed, distribution)
    if key not in _reference_cache:
        _reference_cache.clear()
        A, B = make_inputs(config, seed, distribution)
        _reference_cache[key] = [A, B, A @ B, None]
    return _reference_cache[key]


def _host_case_f64(case) -> np.ndarray:
    """float64 host GEMM of a cached case, computed on first use."""
    if case[3] is None:
        case[3] = case[0].astype(np.float64) @ case[1].astype(np.float64)
    return case[3]


def run_eval(cuda_func: KernelHandle, pipeline_depth, hint: TileDict, repeat_times: int = 20,
             seed: int = 0, distribution: str = "uniform", check: bool = True):
    """Protocol of the reference's ``run_eval`` (roller.py:525-586): one checked launch, one
    more single launch, warm-ups (ten, or as many as fill ``WARMUP_MS``), then ``repeat_times``
    launches between two events.
    Returns ``(ms_per_launch, gflops)``; details (error measures, minimum and median of
    per-launch event pairs) land in ``cuda_func.last_eval``.

    Unlike the reference, which only prints on a mismatch, a result outside the tolerances
    raises, so that a wrong kernel can never be picked as the fastest one.
    """
    cfg = hint.matmul_config
    M, N, K = cfg.M, cfg.N, cfg.K
    case = _host_case(cfg, seed, distribution)
    A, B, C32 = case[0], case[1], case[2]
    g = cuda_func.gemm_config
    dA, dB = DeviceArray.from_host(A), DeviceArray.from_host(B.T if g.trans_b else B)
    dC = DeviceArray.zeros((M, N))

    grid_dims = (-(-N // g.bn), -(-M // g.bm))  # the reference floors here; ragged tiles exist now
    block_dims = cuda_func.block_dims()
    shared_memory_usage = max(hint.smem_cost * int(pipeline_depth), cuda_func.shared_mem_bytes)
    args = (dA.ptr, dB.ptr, dC.ptr)

    cuda_func(grid_dims, block_dims, args, shared_mem=shared_memory_usage)
    hip.synchronize()
    info: dict = {}
    if check:
        info = gemm_errors(dC.get(), A, B, C32, _host_case_f64(case))
        if not info["ok"]:
            raise AssertionError(f"GEMM result outside tolerance for {hint}: {info}")

    # one launch inside a named range, for a profiler to find (the reference: an NVTX range "roller",
    # roller.py:556-562; here a roctx range of the same name when the marker library is there)
    with hip.profiler_range("roller"):
        cuda_func(grid_dims, block_dims, args, shared_mem=shared_memory_usage)
    # The reference warms up with 10 launches.  On MI355X the engine clock drops as soon as the
    # GPU idles (here: during the check above) and needs about 25 ms of load to come back, so
    # the warm-up is extended to cover WARMUP_MS; it runs straight into the timed launches.
    est_ms = 2.0 * M * N * K / 120e9
    for _ in range(max(10, int(WARMUP_MS / est_ms) + 1)):
        cuda_func(grid_dims, block_dims, args, shared_mem=shared_memory_usage)
    with time_cuda() as (start_gpu, end_gpu):
        for _ in range(repeat_times):
            cuda_func(grid_dims, block_dims, args, shared_mem=shared_memory_usage)
    t_gpu = hip.get_elapsed_time(start_gpu, end_gpu)
    # Per-launch spread: a second batch with an event after every launch (recording an event
    # does not idle the GPU, so the clock stays up), read back after one final wait.
    marks = [Event() for _ in range(repeat_times + 1)]
    marks[0].record()
    for mark in marks[1:]:
        cuda_func(grid_dims, block_dims, args, shared_mem=shared_memory_usage)
        mark.record()
    marks[-1].synchronize()
    each = sorted(hip.get_elapsed_time(a, b) for a, b in zip(marks, marks[1:]))

    flops = 2 * M * N * K
    gflops = repeat_times * flops * 1e-9 / (t_gpu / 1000)
    print(f"t={t_gpu / repeat_times:.6f} ms GFLOPS={gflops:.6f}")
    info.update(ms=t_gpu / repeat_times, gflops=gflops)
    if each:
        info.update(min_ms=each[0], median_ms=each[len(each) // 2])
    cuda_func.last_eval = info
    return t_gpu / repeat_times, gflops


def run_baseline(config: MatmulConfig, repeat_times: int = 3, seed: int = 0):
    """Baseline column of the sweep.  The reference times cuBLAS through ``cp.matmul``
    (roller.py:589-607); here it is numpy's float32 ``A @ B`` (its BLAS, all host cores) on the
    same seeded inputs: one warm-up, then the best of ``repeat_times`` wall-clock runs.
    Returns ``(ms, gflops)``."""
    A, B = _host_case(config, seed, "uniform")[:2]
    out = np.empty((config.M, config.N), dtype=np.float32)
    np.matmul(A, B, out=out)
    best = float("inf")
    for _ in range(max(1, repeat_times)):
        t0 = time.perf_counter()
        np.matmul(A, B, out=out)
        best = min(best, time.perf_counter() - t0)
    gflops = 2 * config.M * config.N * config.K * 1e-9 / best
    print(f"t={best * 1e3:.6f} ms GFLOPS={gflops:.6f}")
    return best * 1e3, gflops


def run_vendor_baseline(config: MatmulConfig, repeat_times: int = 50, seed: int = 0, check: bool = True):
    """The reference's baseline proper (roller.py:589-607): the vendor BLAS on the GPU -- there
    cuBLAS through ``cp.matmul``, here rocBLAS ``sgemm`` -- on the same seeded inputs, timed like
    the kernels (clock ramp queued ahead, ``repeat_times`` launches between two events).
    Returns ``(ms, gflops)``; raises if rocBLAS is missing or its result is outside the tolerances."""
    from .vendor_blas import rocblas

    M, N, K = config.M, config.N, config.K
    case = _host_case(config, seed, "uniform")
    A, B, C32 = case[0], case[1], case[2]
    dA, dB, dC = DeviceArray.from_host(A), DeviceArray.from_host(B), DeviceArray.zeros((M, N))
    blas = rocblas()
    blas.sgemm_row_major(dA, dB, dC, M, N, K)
    hip.synchronize()
    if check:
        info = gemm_errors(dC.get(), A, B, C32, _host_case_f64(case))
        if not info["ok"]:
            raise AssertionError(f"rocBLAS result outside tolerance: {info}")
    est_ms = 2.0 * M * N * K / 120e9
    for _ in range(max(10, int(WARMUP_MS / est_ms) + 1)):
        blas.sgemm_row_major(dA, dB, dC, M, N, K)
    with time_cuda() as (start_gpu, end_gpu):
        for _ in range(repeat_times):
            blas.sgemm_row_major(dA, dB, dC, M, N, K)
    t = hip.get_elapsed_time(start_gpu, end_gpu) / repeat_times
    gflops = 2 * M * N * K * 1e-9 / (t / 1000)
    print(f"t={t:.6f} ms GFLOPS={gflops:.6f}")
    return t, gflops


if __name__ == "__main__":
    S = 4096
    config = MatmulConfig(M=S, N=S, K=S, el_bits=32)
    pipeline_depth = 3
    hints = get_roller_hints(config, MI355X(), topk=20)
    run_baseline(config)
    timings = {}
    for hint in hints:
        func = Compiler(config, hint, pipeline_depth, dump_path=Path("log")).compile()
        print(hint)
        timings[hint] = run_eval(func, pipeline_depth, hint)
        print("---\n")
    if timings:
        best_hint = min(timings, key=lambda h: timings[h][0])
        print(f"Best hint: {best_hint}, time: {timings[best_hint][0]}, GFLOPS: {timings[best_hint][1]}")
