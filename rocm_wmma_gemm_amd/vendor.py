"""ctypes binding of ``lib/libvendor_gemm.so``: rocBLAS and hipBLASLt behind the GEMM
library's argument conventions, for the context numbers of the benchmarks.

Counterpart of the reference's rocblas_wrapper (reference
rocblas_wrapper/include/rocblas_wrapper/gemm.hpp:33-107), which its rocBLAS test and
benchmark drive (reference test/rocblas/test.cpp, benchmark/rocblas/bench.cpp).  Not used by
the GEMM library itself.
"""
from __future__ import annotations

import ctypes
import os

from .loader import _type_slot, library_dir

ROCBLAS, HIPBLASLT = 0, 1
BACKENDS = {"rocblas": ROCBLAS, "hipblaslt": HIPBLASLT}


class VendorGemmError(RuntimeError):
    pass


class VendorGemm:
    """init on construction (reference init_rocblas), cleanup on close()."""

    def __init__(self, lib_dir: str | None = None):
        path = os.path.join(lib_dir if lib_dir is not None else library_dir(), "libvendor_gemm.so")
        try:
            self._lib = ctypes.CDLL(path)
        except OSError as e:
            raise VendorGemmError(f"could not open {path}: {e}")
        L = self._lib
        L.vendor_gemm_init.restype = ctypes.c_int
        L.vendor_gemm_init.argtypes = []
        L.vendor_gemm_cleanup.restype = None
        L.vendor_gemm_cleanup.argtypes = []
        L.vendor_gemm.restype = ctypes.c_int
        L.vendor_gemm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                  ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t,
                                  ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                  ctypes.c_void_p]
        if L.vendor_gemm_init() != 0:
            raise VendorGemmError("vendor_gemm_init failed (rocBLAS / hipBLASLt handle)")

    def close(self) -> None:
        if self._lib is not None:
            self._lib.vendor_gemm_cleanup()
            self._lib = None

    def gemm(self, backend, C, A, B, M: int, N: int, K: int, layout_c=0, layout_a=0, layout_b=0,
             batch_count: int = 1, stream=None) -> None:
        """C = A * B through rocBLAS or hipBLASLt, enqueued on ``stream`` (default: torch's
        current stream); tensors are flat packed storage as for ``Loader.gemm``."""
        import torch

        if isinstance(backend, str):
            backend = BACKENDS[backend]
        if stream is None:
            stream = torch.cuda.current_stream()
        handle = ctypes.c_void_p(int(stream.cuda_stream) if hasattr(stream, "cuda_stream") else int(stream))
        rc = self._lib.vendor_gemm(backend, _type_slot(C.dtype, A.dtype), C.data_ptr(), A.data_ptr(),
                                   B.data_ptr(), M, N, K, batch_count, int(layout_c), int(layout_a),
                                   int(layout_b), ctypes.byref(handle))
        if rc != 0:
            raise VendorGemmError(f"vendor_gemm returned {rc}")
