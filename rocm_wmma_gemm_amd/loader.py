"""Python mirror of ``rocm_wmma_gemm::loader``.

Reference interface: rocm_wmma_gemm/include/rocm_wmma_gemm/kernel_loader.hpp:51-182
 - library name ``librocm_wmma_gemm_<arch>.so`` with ``<arch>`` taken from device 0's
   architecture string cut at the first ':' (:74-91);
 - search order: the configured library directory first, then the dynamic linker's
   own path (:93-102);
 - the four ``rocm_wmma_gemm_<Ctype>_<ABtype>`` symbols are resolved eagerly and a
   missing library or symbol raises (:104-113) -- here ``GemmLibraryError``;
 - ``gemm`` takes (C, A, B, M, N, K[, batch_count], stream) with the layouts in
   C, A, B order and passes the ADDRESS of the stream handle (:138-154).

There is no CPU fallback: if the library cannot be loaded every call fails.
"""
from __future__ import annotations

import ctypes
import enum
import os
import subprocess
from dataclasses import dataclass

_HERE = os.path.dirname(os.path.abspath(__file__))
_DEFAULT_LIB_DIR = os.path.join(_HERE, "lib")

ENTRY_SUFFIXES = ("f16_f16", "f32_f16", "bf16_bf16", "f32_bf16")

# status codes and the fixed scratch size of include/rocm_wmma_gemm_c.h
OK, ERR_VARIANT, ERR_ARGUMENT, ERR_SCRATCH, ERR_RUNTIME, ERR_LIMIT = 0, -1, -2, -3, -4, -5
NOALLOC_SCRATCH_BYTES = 64 << 20


class GemmLibraryError(RuntimeError):
    """Library or symbol could not be loaded (the C++ loader throws std::runtime_error)."""


class m_layout(enum.IntEnum):
    row_major = 0
    col_major = 1


row_major = m_layout.row_major
col_major = m_layout.col_major


class _VariantInfoC(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "block_m", "block_n", "block_k", "warps_m", "warps_n", "warp_tile_m", "warp_tile_n",
        "pipeline", "lds_bytes", "threads")]


@dataclass(frozen=True)
class VariantInfo:
    index: int
    block_m: int
    block_n: int
    block_k: int
    warps_m: int
    warps_n: int
    warp_tile_m: int
    warp_tile_n: int
    pipeline: int
    lds_bytes: int
    threads: int


def library_dir() -> str:
    """Directory searched first (the C++ loader's ROCM_WMMA_GEMM_LIB_DIR define)."""
    return os.environ.get("ROCM_WMMA_GEMM_LIB_DIR", _DEFAULT_LIB_DIR)


def library_path(arch: str = "gfx950") -> str:
    return os.path.join(library_dir(), f"librocm_wmma_gemm_{arch}.so")


def build_library(jobs: int = 8, force: bool = False) -> str:
    """Compile the HIP library in-tree (cross-compiles without a GPU)."""
    cmd = ["make", "-C", os.path.join(_HERE, "csrc"), f"-j{jobs}", "all"]
    if force:
        cmd.insert(1, "-B")
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)
    return os.path.join(_DEFAULT_LIB_DIR, "librocm_wmma_gemm_gfx950.so")


def source_stamp() -> str:
    """Sixteen hex digits over everything a kernel launch of the library depends on: the
    kernel and host sources under csrc/ (the generated table left out) and the tuned
    tables.  A counter summary under profiles/ records the stamp of the tree it was measured
    on, so that a reader (and bench.py) can tell whether it still describes this library."""
    import glob
    import hashlib

    files = []
    for pattern in ("csrc/*.hip", "csrc/*.hpp", "csrc/*.cpp", "csrc/*.def", "csrc/kernel/*.hpp",
                    "config/gemm_config_gfx950_*.json", "config/model_gfx950.json"):
        files += glob.glob(os.path.join(_HERE, pattern))
    h = hashlib.sha256()
    for path in sorted(f for f in files if not f.endswith("config_generated.hpp")):
        h.update(os.path.relpath(path, _HERE).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def detect_arch() -> str:
    import torch

    if not torch.cuda.is_available():
        raise GemmLibraryError("rocm_wmma_gemm::loader: hipGetDeviceProperties failed (no GPU)")
    name = torch.cuda.get_device_properties(0).gcnArchName
    return name.split(":", 1)[0]


def _type_slot(c_dtype, ab_dtype) -> int:
    import torch

    table = {(torch.float16, torch.float16): 0, (torch.float32, torch.float16): 1,
             (torch.bfloat16, torch.bfloat16): 2, (torch.float32, torch.bfloat16): 3}
    try:
        return table[(c_dtype, ab_dtype)]
    except KeyError:
        raise TypeError(f"Unsupported type pair for rocm_wmma_gemm loader: C={c_dtype}, A/B={ab_dtype}")


class Loader:
    """Opens the per-architecture library and forwards gemm calls through its C ABI."""

    _ENTRY_ARGS = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                   ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_int, ctypes.c_int,
                   ctypes.c_int, ctypes.c_void_p]

    def __init__(self, arch: str | None = None, lib_dir: str | None = None):
        self.arch = arch if arch is not None else detect_arch()
        name = f"librocm_wmma_gemm_{self.arch}.so"
        first = os.path.join(lib_dir if lib_dir is not None else library_dir(), name)
        errors = []
        self._lib = None
        for candidate in (first, name):
            try:
                self._lib = ctypes.CDLL(candidate, mode=os.RTLD_NOW | os.RTLD_LOCAL)
                self.path = candidate
                break
            except OSError as e:
                errors.append(str(e))
        if self._lib is None:
            raise GemmLibraryError(f"rocm_wmma_gemm::loader: could not open {name}: " + "; ".join(errors))
        self._entries = []
        for suffix in ENTRY_SUFFIXES:
            sym = "rocm_wmma_gemm_" + suffix
            try:
                fn = getattr(self._lib, sym)
            except AttributeError as e:
                raise GemmLibraryError(f"rocm_wmma_gemm::loader: symbol not found: {sym} ({e})")
            fn.restype = None
            fn.argtypes = self._ENTRY_ARGS
            self._entries.append(fn)
        self._bind_extras()

    # ------------------------------------------------------------------ extras
    def _bind_extras(self):
        L = self._lib
        self._has_extras = hasattr(L, "rocm_wmma_gemm_run_variant")
        if not self._has_extras:
            return
        L.rocm_wmma_gemm_arch.restype = ctypes.c_char_p
        L.rocm_wmma_gemm_arch.argtypes = []
        L.rocm_wmma_gemm_variant_count.restype = ctypes.c_int
        L.rocm_wmma_gemm_variant_count.argtypes = []
        L.rocm_wmma_gemm_variant_info_get.restype = ctypes.c_int
        L.rocm_wmma_gemm_variant_info_get.argtypes = [ctypes.c_int, ctypes.POINTER(_VariantInfoC)]
        L.rocm_wmma_gemm_select.restype = ctypes.c_int
        L.rocm_wmma_gemm_select.argtypes = [ctypes.c_size_t] * 3 + [ctypes.c_int] * 4 + [
            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.rocm_wmma_gemm_select_batched.restype = ctypes.c_int
        L.rocm_wmma_gemm_select_batched.argtypes = [ctypes.c_size_t] * 4 + [ctypes.c_int] * 4 + [
            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.rocm_wmma_gemm_run_variant.restype = ctypes.c_int
        L.rocm_wmma_gemm_run_variant.argtypes = [ctypes.c_int] * 4 + self._ENTRY_ARGS
        if hasattr(L, "rocm_wmma_gemm_run_variant_ex"):
            L.rocm_wmma_gemm_run_variant_ex.restype = ctypes.c_int
            L.rocm_wmma_gemm_run_variant_ex.argtypes = [ctypes.c_int] * 5 + self._ENTRY_ARGS
            L.rocm_wmma_gemm_select_ex.restype = ctypes.c_int
            L.rocm_wmma_gemm_select_ex.argtypes = [ctypes.c_size_t] * 4 + [ctypes.c_int] * 4 + [
                ctypes.POINTER(ctypes.c_int)] * 3
        if hasattr(L, "rocm_wmma_gemm_workspace_release"):
            L.rocm_wmma_gemm_workspace_release.restype = ctypes.c_int
            L.rocm_wmma_gemm_workspace_release.argtypes = []
        if hasattr(L, "rocm_wmma_gemm_noalloc"):
            L.rocm_wmma_gemm_noalloc.restype = ctypes.c_int
            L.rocm_wmma_gemm_noalloc.argtypes = [ctypes.c_int] + self._ENTRY_ARGS

    def library_arch(self) -> str:
        return self._lib.rocm_wmma_gemm_arch().decode()

    def variants(self) -> list[VariantInfo]:
        out = []
        for i in range(self._lib.rocm_wmma_gemm_variant_count()):
            c = _VariantInfoC()
            if self._lib.rocm_wmma_gemm_variant_info_get(i, ctypes.byref(c)) != 0:
                raise GemmLibraryError(f"variant {i} not described by the library")
            out.append(VariantInfo(i, *[getattr(c, n) for n, _ in _VariantInfoC._fields_]))
        return out

    def select(self, M: int, N: int, K: int, type_idx: int, layout_c: int, layout_a: int,
               layout_b: int, batch_count: int = 1) -> tuple[int, int, int]:
        """(variant, swizzle, split_k) the dispatcher picks for this problem (for a strided
        batch of batch_count such problems)."""
        swz, sk = ctypes.c_int(0), ctypes.c_int(0)
        v = self._lib.rocm_wmma_gemm_select_batched(
            M, N, K, batch_count, type_idx, int(layout_c), int(layout_a), int(layout_b),
            ctypes.byref(swz), ctypes.byref(sk))
        return v, swz.value, sk.value

    # ------------------------------------------------------------------ gemm
    @staticmethod
    def _stream_handle(stream) -> int:
        import torch

        if stream is None:
            stream = torch.cuda.current_stream()
        return int(stream.cuda_stream) if hasattr(stream, "cuda_stream") else int(stream)

    @staticmethod
    def _check(C, A, B, M, N, K, batch):
        for name, t, need in (("A", A, M * K * batch), ("B", B, K * N * batch), ("C", C, M * N * batch)):
            if not t.is_cuda:
                raise ValueError(f"{name} must be a device tensor")
            if not t.is_contiguous():
                raise ValueError(f"{name} must be densely packed")
            if t.numel() < need:
                raise ValueError(f"{name} holds {t.numel()} elements, the problem needs {need}")
        if A.dtype != B.dtype:
            raise TypeError("A and B must share an element type")
        # the library's own limits: beyond them its C++ side throws, which a caller that
        # came in through ctypes could not catch
        for name, v in (("M", M), ("N", N), ("K", K)):
            if v < 0 or v > 0x7FFFFFFF:
                raise ValueError(f"{name} = {v} does not fit in 31 bits")
        if batch < 0:
            raise ValueError("batch_count must not be negative")

    def gemm(self, C, A, B, M: int, N: int, K: int, layout_c=row_major, layout_a=row_major,
             layout_b=row_major, batch_count: int = 1, stream=None) -> None:
        """C = A * B, enqueued on ``stream`` (default: torch's current stream).

        C, A, B are device tensors used as flat packed storage in the stated layouts."""
        self._check(C, A, B, M, N, K, batch_count)
        slot = _type_slot(C.dtype, A.dtype)
        handle = ctypes.c_void_p(self._stream_handle(stream))
        self._entries[slot](C.data_ptr(), A.data_ptr(), B.data_ptr(), M, N, K, batch_count,
                            int(layout_c), int(layout_a), int(layout_b), ctypes.byref(handle))

    def gemm_raw(self, slot: int, c_ptr: int, a_ptr: int, b_ptr: int, M: int, N: int, K: int,
                 batch_count: int, layout_c: int, layout_a: int, layout_b: int,
                 stream_handle: int) -> None:
        """Direct C-ABI call with raw device addresses (no checks)."""
        handle = ctypes.c_void_p(stream_handle)
        self._entries[slot](c_ptr, a_ptr, b_ptr, M, N, K, batch_count, layout_c, layout_a,
                            layout_b, ctypes.byref(handle))

    def workspace_release(self) -> int:
        """Frees the current device's library-owned scratch buffer (0), unless a captured
        graph may hold its address (1)."""
        return self._lib.rocm_wmma_gemm_workspace_release()

    def gemm_noalloc(self, C, A, B, M: int, N: int, K: int, layout_c=row_major,
                     layout_a=row_major, layout_b=row_major, batch_count: int = 1,
                     stream=None) -> int:
        """gemm() through the entry point that allocates nothing: scratch memory comes from
        a fixed per-GPU array of NOALLOC_SCRATCH_BYTES.  Returns the library's status code
        (0 = enqueued, ERR_SCRATCH = the call needs more scratch memory than that)."""
        self._check(C, A, B, M, N, K, batch_count)
        slot = _type_slot(C.dtype, A.dtype)
        handle = ctypes.c_void_p(self._stream_handle(stream))
        return self._lib.rocm_wmma_gemm_noalloc(
            slot, C.data_ptr(), A.data_ptr(), B.data_ptr(), M, N, K, batch_count,
            int(layout_c), int(layout_a), int(layout_b), ctypes.byref(handle))

    def select_ex(self, M: int, N: int, K: int, type_idx: int, layout_c: int, layout_a: int,
                  layout_b: int, batch_count: int = 1) -> tuple[int, int, int, int]:
        """(variant, swizzle, split_k, touch_ahead) the dispatcher picks for this problem."""
        swz, sk, touch = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
        v = self._lib.rocm_wmma_gemm_select_ex(
            M, N, K, batch_count, type_idx, int(layout_c), int(layout_a), int(layout_b),
            ctypes.byref(swz), ctypes.byref(sk), ctypes.byref(touch))
        return v, swz.value, sk.value, touch.value

    def run_variant(self, variant: int, swizzle: int, split_k: int, C, A, B, M: int, N: int,
                    K: int, layout_c=row_major, layout_a=row_major, layout_b=row_major,
                    batch_count: int = 1, stream=None, touch_ahead: int = 0) -> int:
        """Same as gemm() with the tile variant, swizzle, split-K form and line touches forced
        (tuner hook)."""
        self._check(C, A, B, M, N, K, batch_count)
        slot = _type_slot(C.dtype, A.dtype)
        handle = ctypes.c_void_p(self._stream_handle(stream))
        return self._lib.rocm_wmma_gemm_run_variant_ex(
            slot, variant, swizzle, split_k, touch_ahead, C.data_ptr(), A.data_ptr(), B.data_ptr(),
            M, N, K, batch_count, int(layout_c), int(layout_a), int(layout_b), ctypes.byref(handle))
