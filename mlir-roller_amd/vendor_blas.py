"""rocBLAS ``sgemm`` through ctypes -- the vendor-library baseline of the sweep.

The reference times cuBLAS next to its own kernels (``cp.matmul`` in ``run_baseline``,
/root/reference/src/roller.py:589-607) and tabulates the speedup (benchmark.py:69-85).  This
module is the same yardstick on MI355X: nothing in the GEMM path itself calls it.

rocBLAS is column-major.  A row-major ``C[M,N] = A[M,K] @ B[K,N]`` is the column-major product
``C^T[N,M] = B^T[N,K] @ A^T[K,M]``, and a row-major matrix read as column-major *is* its
transpose, so the call is ``sgemm(N, N, m=N, n=M, k=K, B, ldb=N, A, lda=K, C, ldc=N)``.
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path
from typing import Optional

from . import hip
from .hip import _address

OPERATION_NONE = 111          # rocblas_operation_none
STATUS_SUCCESS = 0            # rocblas_status_success


class VendorBlasError(RuntimeError):
    pass


class RocBLAS:
    """One rocBLAS handle on the library's device.  Loading rocBLAS and its first GEMM are slow
    (the kernel library for the GPU is read lazily); both happen outside any timed region."""

    def __init__(self, library: Optional[str] = None):
        path = library or str(Path(hip.ROCM) / "lib" / "librocblas.so")
        try:
            self._lib = C.CDLL(path)
        except OSError as e:
            raise VendorBlasError(f"cannot load rocBLAS ({path}): {e}") from e
        hip.init()
        L = self._lib
        L.rocblas_create_handle.argtypes = [C.POINTER(C.c_void_p)]
        L.rocblas_destroy_handle.argtypes = [C.c_void_p]
        L.rocblas_set_stream.argtypes = [C.c_void_p, C.c_void_p]
        L.rocblas_sgemm.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                    C.POINTER(C.c_float), C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                    C.POINTER(C.c_float), C.c_void_p, C.c_int]
        for f in (L.rocblas_create_handle, L.rocblas_destroy_handle, L.rocblas_set_stream, L.rocblas_sgemm):
            f.restype = C.c_int
        self._handle = C.c_void_p()
        self._check(L.rocblas_create_handle(C.byref(self._handle)), "rocblas_create_handle")
        self._one, self._zero = C.c_float(1.0), C.c_float(0.0)

    @staticmethod
    def _check(status: int, what: str) -> None:
        if status != STATUS_SUCCESS:
            raise VendorBlasError(f"{what} failed with rocblas_status {status}")

    def set_stream(self, stream) -> None:
        self._check(self._lib.rocblas_set_stream(self._handle, hip._stream_handle(stream)), "rocblas_set_stream")

    def sgemm_row_major(self, A, B, Cm, M: int, N: int, K: int, lda: Optional[int] = None,
                        ldb: Optional[int] = None, ldc: Optional[int] = None) -> None:
        """Enqueues ``C = A @ B`` for row-major fp32 device matrices (pointers or ``DeviceArray``)."""
        ptr = _address
        self._check(self._lib.rocblas_sgemm(
            self._handle, OPERATION_NONE, OPERATION_NONE, N, M, K, C.byref(self._one),
            ptr(B), N if ldb is None else ldb, ptr(A), K if lda is None else lda,
            C.byref(self._zero), ptr(Cm), N if ldc is None else ldc), "rocblas_sgemm")

    def close(self) -> None:
        if getattr(self, "_handle", None) and self._handle.value:
            self._lib.rocblas_destroy_handle(self._handle)
            self._handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_shared: Optional[RocBLAS] = None


def rocblas() -> RocBLAS:
    """Process-wide handle (created on first use)."""
    global _shared
    if _shared is None:
        _shared = RocBLAS()
    return _shared
