"""TEST INFRASTRUCTURE ONLY: ctypes front end of the CPU GEMM oracle.

The arithmetic lives in ``gemm_oracle.c`` (a restatement of the reference's
``test/test.hpp:33-215`` and ``common/matrix.hpp:154-164``).  Only tests, the
smoke check and the benchmark's ``cpu_baseline`` leg may import this module; the
product package never does.

Half and bfloat16 matrices are carried as ``numpy.uint16`` arrays of raw bits so
that no third-party conversion sits between the oracle and its checks.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_gemm.so")

F16, BF16, F32 = 0, 1, 2
ROW, COL = 0, 1
DTYPE_NAMES = {"f16": F16, "bf16": BF16, "f32": F32}


def build(force: bool = False) -> str:
    """Compile the oracle's C source next to it and return the library path."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "gemm_oracle.c"))
    ):
        subprocess.run(["make", "-C", _HERE, "-B", "liboracle_gemm.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, i32, u32, f32, vp = (ctypes.c_size_t, ctypes.c_int, ctypes.c_uint32, ctypes.c_float,
                                 ctypes.c_void_p)
        L.oracle_f16_to_f32.restype = f32
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f32_to_f16.argtypes = [f32]
        L.oracle_bf16_to_f32.restype = f32
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f32_to_bf16.argtypes = [f32]
        L.oracle_raw_draws.restype = None
        L.oracle_raw_draws.argtypes = [u32, sz, vp]
        L.oracle_uniform_draws.restype = None
        L.oracle_uniform_draws.argtypes = [u32, f32, f32, sz, vp]
        L.oracle_init_matrix.restype = None
        L.oracle_init_matrix.argtypes = [vp, sz, sz, i32, i32, u32, i32, f32, f32]
        L.oracle_gemm_naive.restype = None
        L.oracle_gemm_naive.argtypes = [vp, vp, vp, sz, sz, sz, i32, i32, i32, i32, i32]
        L.oracle_gemm.restype = i32
        L.oracle_gemm.argtypes = [vp, vp, vp, sz, sz, sz, i32, i32, i32, i32, i32, i32, vp]
        L.oracle_gemm_rows.restype = i32
        L.oracle_gemm_rows.argtypes = [vp, vp, vp, sz, sz, sz, i32, i32, i32, i32, i32, sz, sz,
                                       i32, vp]
        L.oracle_cosine_similarity.restype = f32
        L.oracle_cosine_similarity.argtypes = [vp, vp, sz, sz, i32, i32]
        L.oracle_cosine_threshold.restype = f32
        L.oracle_cosine_threshold.argtypes = [i32]
        L.oracle_fnv1a64.restype = ctypes.c_uint64
        L.oracle_fnv1a64.argtypes = [vp, sz]
        L.oracle_fnv1a64_basis.restype = ctypes.c_uint64
        L.oracle_fnv1a64_basis.argtypes = [vp, sz, ctypes.c_uint64]
        _lib = L
    return _lib


def _np_dtype(dtype: int):
    return np.float32 if dtype == F32 else np.uint16


def _ptr(a: np.ndarray) -> ctypes.c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def default_threads() -> int:
    return max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "64"))))


# ---------------------------------------------------------------- scalars
def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    L = lib()
    flat = np.asarray(x, dtype=np.float32).ravel()
    return np.array([L.oracle_f32_to_f16(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(x))


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    L = lib()
    flat = np.asarray(x, dtype=np.float32).ravel()
    return np.array([L.oracle_f32_to_bf16(float(v)) for v in flat], dtype=np.uint16).reshape(np.shape(x))


def bits_to_f32(bits: np.ndarray, dtype: int) -> np.ndarray:
    """Widen raw f16/bf16 bits to float32 (vectorised numpy, exact)."""
    if dtype == F32:
        return np.asarray(bits, dtype=np.float32)
    bits = np.asarray(bits, dtype=np.uint16)
    if dtype == BF16:
        return (bits.astype(np.uint32) << 16).view(np.float32)
    return bits.view(np.float16).astype(np.float32)


# ---------------------------------------------------------------- generator
def raw_draws(seed: int, count: int) -> np.ndarray:
    out = np.empty(count, dtype=np.uint32)
    lib().oracle_raw_draws(seed, count, _ptr(out))
    return out


def uniform_draws(seed: int, lo: float, hi: float, count: int) -> np.ndarray:
    out = np.empty(count, dtype=np.float32)
    lib().oracle_uniform_draws(seed, lo, hi, count, _ptr(out))
    return out


def init_matrix(m: int, n: int, layout: int, dtype: int, seed: int = 1, dist: str = "uniform",
                lo: float = -1.0, hi: float = 1.0) -> np.ndarray:
    """Flat storage (length m*n) of an m x n matrix filled like test/test.hpp:33-54.

    ``dist='normal'`` draws normal(mean=lo, std=hi) instead (harness-only)."""
    out = np.empty(m * n, dtype=_np_dtype(dtype))
    lib().oracle_init_matrix(_ptr(out), m, n, layout, dtype, seed, 0 if dist == "uniform" else 1,
                             lo, hi)
    return out


# ---------------------------------------------------------------- gemm
def gemm(A: np.ndarray, B: np.ndarray, M: int, N: int, K: int, layout_c: int, layout_a: int,
         layout_b: int, in_dtype: int, out_dtype: int, *, threads: int | None = None,
         want_scale: bool = False, rows: tuple[int, int] | None = None, naive: bool = False):
    """C = A*B per test/test.hpp:59-129.  Returns flat C storage (and S if asked).

    With ``rows=(r0, r1)`` only those rows of C are computed (others are zero)."""
    assert A.size == M * K and B.size == K * N
    C = np.zeros(M * N, dtype=_np_dtype(out_dtype))
    if naive:
        lib().oracle_gemm_naive(_ptr(C), _ptr(A), _ptr(B), M, N, K, layout_c, layout_a, layout_b,
                                in_dtype, out_dtype)
        return C
    S = np.zeros(M * N, dtype=np.float32) if want_scale else None
    r0, r1 = rows if rows is not None else (0, M)
    rc = lib().oracle_gemm_rows(_ptr(C), _ptr(A), _ptr(B), M, N, K, layout_c, layout_a, layout_b,
                                in_dtype, out_dtype, r0, r1,
                                threads if threads is not None else default_threads(),
                                _ptr(S) if S is not None else None)
    if rc != 0:
        raise MemoryError("oracle_gemm_rows: allocation failed")
    return (C, S) if want_scale else C


def logical(flat: np.ndarray, m: int, n: int, layout: int) -> np.ndarray:
    """View flat storage as the logical m x n matrix (common/matrix.hpp:154-164)."""
    return flat.reshape(m, n) if layout == ROW else flat.reshape(n, m).T


# ---------------------------------------------------------------- verification
def cosine_similarity(gpu: np.ndarray, cpu: np.ndarray, m: int, n: int, layout: int,
                      dtype: int) -> float:
    return float(lib().oracle_cosine_similarity(_ptr(gpu), _ptr(cpu), m, n, layout, dtype))


def cosine_threshold(dtype: int) -> float:
    return float(lib().oracle_cosine_threshold(dtype))


def fnv1a64(a: np.ndarray, basis: int | None = None) -> str:
    a = np.ascontiguousarray(a)
    if basis is None:
        return "%016x" % lib().oracle_fnv1a64(_ptr(a), a.nbytes)
    return "%016x" % lib().oracle_fnv1a64_basis(_ptr(a), a.nbytes, basis)


def ulp_out(values_f32: np.ndarray, dtype: int) -> np.ndarray:
    """One unit in the last place of the output type at |values| (0 for fp32 C)."""
    v = np.abs(np.asarray(values_f32, dtype=np.float64))
    if dtype == F32:
        return np.zeros_like(v)
    mant, min_exp = (10, -14) if dtype == F16 else (7, -126)
    e = np.floor(np.log2(np.maximum(v, 2.0 ** min_exp)))
    return 2.0 ** (np.maximum(e, min_exp) - mant)


def tolerance(S: np.ndarray, K: int, cpu_f32: np.ndarray, out_dtype: int) -> np.ndarray:
    """|gpu - cpu| bound: 2*K*2^-24*sum_k|a*b| + 1 ulp of the C type.

    Any two fp32 summation orders of K products differ by at most 2*K*u*S with
    u = 2^-24; rounding to a narrower C type adds at most one output ulp."""
    return 2.0 * K * 2.0 ** -24 * np.asarray(S, dtype=np.float64) + ulp_out(cpu_f32, out_dtype)
