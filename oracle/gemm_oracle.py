"""CPU oracle of the fp32 GEMM path -- TEST INFRASTRUCTURE, not product code.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this module; the product (``mlir_roller_amd``) never does and has no CPU fallback.

What the path computes is the reference's payload ``linalg.matmul(A, B, C)`` on row-major fp32
``A[M,K]``, ``B[K,N]``, ``C[M,N]`` (/root/reference/src/roller.py:50-62), checked by the reference
against ``dA @ dB`` (roller.py:552).  The kernel that the reference generates comes out of an
IREE fork that is not in its tree (empty submodule third_party/iree, .gitmodules:1-3, no commit
pinned), and the reference holds no tests or golden vectors for it, so the oracle is the
definition of that payload:

* ``gemm_f32``  -- numpy float32 ``A @ B`` (the "reference path's result" of the acceptance
  bound ``||C - C_ref||_F / ||C_ref||_F <= 1e-5``),
* ``gemm_f64``  -- float64 host GEMM (for ``max|C - C64| <= 1e-4 * sqrt(K) * max|A| * max|B|``),
* ``c_gemm_f32`` / ``c_gemm_f64`` / ``c_gemm_naive`` -- the plain-C restatement in
  ``gemm_oracle.c`` (k-ascending fp32 accumulation, float64 accumulation, one dot product per
  element), which shares no code with numpy's BLAS and cross-checks it,
* ``gemm_exact`` -- exact integer arithmetic on Python ints for tiny cases.

Pinned by tests/test_oracle_gemm.py (closed forms, exact cases, algebraic identities).
"""

from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path
from typing import Optional, Tuple

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB_PATH = ORACLE_DIR / "_build" / "liboracle_gemm.so"

NORMWISE_TOL = 1e-5
ELEMENTWISE_FACTOR = 1e-4


# ---- inputs -----------------------------------------------------------------------------------

def make_inputs(M: int, N: int, K: int, seed: int = 0, distribution: str = "uniform") -> Tuple[np.ndarray, np.ndarray]:
    """Seeded row-major fp32 operands: one generator, A drawn first, then B.
    "uniform" = U[-1, 1), "normal" = N(0, 1), "integer" = {0..9} (fp32 sums of such products are
    exact for any K below 207126, so every summation order gives the same bits)."""
    rng = np.random.default_rng(seed)
    if distribution == "uniform":
        draw = lambda s: rng.uniform(-1.0, 1.0, s).astype(np.float32)
    elif distribution == "normal":
        draw = lambda s: rng.standard_normal(s, dtype=np.float32)
    elif distribution == "integer":
        draw = lambda s: rng.integers(0, 10, s).astype(np.float32)
    else:
        raise ValueError(distribution)
    return draw((M, K)), draw((K, N))


# ---- numpy restatement --------------------------------------------------------------------------

def gemm_f32(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    return np.matmul(np.asarray(A, np.float32), np.asarray(B, np.float32))


def gemm_f64(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    return np.matmul(np.asarray(A, np.float64), np.asarray(B, np.float64))


def gemm_exact(A, B):
    """Triple loop on Python ints (inputs must be integer-valued); list of lists."""
    A = [[int(v) for v in row] for row in np.asarray(A).tolist()]
    B = [[int(v) for v in row] for row in np.asarray(B).tolist()]
    M, K, N = len(A), len(B), len(B[0]) if B else 0
    return [[sum(A[i][k] * B[k][j] for k in range(K)) for j in range(N)] for i in range(M)]


# ---- acceptance bounds --------------------------------------------------------------------------

def error_report(Cg: np.ndarray, A: np.ndarray, B: np.ndarray, C32: Optional[np.ndarray] = None,
                 C64: Optional[np.ndarray] = None) -> dict:
    """Both error measures of a computed ``Cg`` and whether it meets both bounds."""
    C32 = gemm_f32(A, B) if C32 is None else C32
    C64 = gemm_f64(A, B) if C64 is None else C64
    K = A.shape[1]
    ref_norm = float(np.linalg.norm(C32.astype(np.float64)))
    normwise = float(np.linalg.norm(Cg.astype(np.float64) - C32.astype(np.float64))) / max(ref_norm, 1e-300)
    max_abs = float(np.max(np.abs(Cg.astype(np.float64) - C64))) if Cg.size else 0.0
    amax = float(np.max(np.abs(A))) if A.size else 0.0
    bmax = float(np.max(np.abs(B))) if B.size else 0.0
    bound = ELEMENTWISE_FACTOR * float(np.sqrt(max(K, 1))) * amax * bmax
    finite = bool(np.all(np.isfinite(Cg)))
    return {"normwise": normwise, "max_abs": max_abs, "bound": bound,
            "ok": finite and normwise <= NORMWISE_TOL and max_abs <= bound}


# ---- plain-C restatement ------------------------------------------------------------------------

_lib: Optional[C.CDLL] = None


def build(verbose: bool = False) -> Path:
    """``make -C oracle`` (gcc)."""
    subprocess.run(["make", "-C", str(ORACLE_DIR)] + ([] if verbose else ["-s"]), check=True)
    return LIB_PATH


def _clib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = C.CDLL(str(LIB_PATH))
        fp, dp = C.POINTER(C.c_float), C.POINTER(C.c_double)
        ints, longs = [C.c_int] * 3, [C.c_long] * 3
        lib.oracle_gemm_f64.argtypes = [fp, fp, dp] + ints + longs + [C.c_int]
        lib.oracle_gemm_f32.argtypes = [fp, fp, fp] + ints + longs + [C.c_int]
        lib.oracle_gemm_naive.argtypes = [fp, fp, fp] + ints + longs
        lib.oracle_compare.argtypes = [fp, dp, C.c_int, C.c_int, C.c_long, C.c_long, dp, dp, dp]
        for f in (lib.oracle_gemm_f64, lib.oracle_gemm_f32, lib.oracle_gemm_naive, lib.oracle_compare):
            f.restype = None
        _lib = lib
    return _lib


def _f32(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float32)
    if x.ndim != 2 or x.strides[1] != 4 or x.strides[0] % 4 or (x.shape[0] > 1 and x.strides[0] < 4 * x.shape[1]):
        x = np.ascontiguousarray(x)
    return x


def _ld(x: np.ndarray) -> int:
    return x.strides[0] // x.itemsize if x.shape[0] > 1 else max(x.shape[1], 1)


def _ptr(x: np.ndarray, ctype):
    return x.ctypes.data_as(C.POINTER(ctype))


def c_gemm_f64(A: np.ndarray, B: np.ndarray, out: Optional[np.ndarray] = None, accumulate: bool = False) -> np.ndarray:
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[1]
    if out is None:
        out = np.zeros((M, N), dtype=np.float64)
    _clib().oracle_gemm_f64(_ptr(A, C.c_float), _ptr(B, C.c_float), _ptr(out, C.c_double), M, N, K,
                            _ld(A), _ld(B), _ld(out), int(accumulate))
    return out


def c_gemm_f32(A: np.ndarray, B: np.ndarray, out: Optional[np.ndarray] = None, accumulate: bool = False) -> np.ndarray:
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[1]
    if out is None:
        out = np.zeros((M, N), dtype=np.float32)
    _clib().oracle_gemm_f32(_ptr(A, C.c_float), _ptr(B, C.c_float), _ptr(out, C.c_float), M, N, K,
                            _ld(A), _ld(B), _ld(out), int(accumulate))
    return out


def c_gemm_naive(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[1]
    out = np.zeros((M, N), dtype=np.float32)
    _clib().oracle_gemm_naive(_ptr(A, C.c_float), _ptr(B, C.c_float), _ptr(out, C.c_float), M, N, K,
                              _ld(A), _ld(B), _ld(out))
    return out


def c_compare(Cg: np.ndarray, R: np.ndarray) -> dict:
    """max |Cg - R| and the normwise relative difference, computed by the C side."""
    Cg = _f32(Cg)
    R = np.ascontiguousarray(R, dtype=np.float64)
    mx, d2, r2 = C.c_double(), C.c_double(), C.c_double()
    _clib().oracle_compare(_ptr(Cg, C.c_float), _ptr(R, C.c_double), Cg.shape[0], Cg.shape[1],
                           _ld(Cg), _ld(R), C.byref(mx), C.byref(d2), C.byref(r2))
    return {"max_abs": mx.value, "normwise": (d2.value ** 0.5) / max(r2.value ** 0.5, 1e-300)}
