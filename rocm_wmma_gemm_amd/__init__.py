"""MI355X (gfx950) GEMM behind the rocm_wmma_gemm host interface.

The product is the shared library ``lib/librocm_wmma_gemm_gfx950.so`` (hand-written
HIP, built by ``csrc/Makefile``).  This package is the Python-side mirror of the
reference's header-only runtime loader: it finds the library for the GPU in the
machine and forwards typed ``gemm`` calls through the library's C ABI.  PyTorch is
used only to own device memory and streams.
"""
from .loader import (  # noqa: F401
    GemmLibraryError,
    Loader,
    VariantInfo,
    build_library,
    col_major,
    library_path,
    m_layout,
    row_major,
    source_stamp,
)

__all__ = ["Loader", "GemmLibraryError", "VariantInfo", "m_layout", "row_major", "col_major",
           "library_path", "build_library", "source_stamp"]
