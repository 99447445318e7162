// Shared vocabulary of the gfx950 GEMM library: layout enum, operand tags and the
// element-type mapping used by the public API and by the kernels.
//
// Interface parity: reference rocm_wmma_gemm/include/rocm_wmma_gemm/kernel/common.hpp:38-86.
// The numeric values of m_layout are part of the C ABI (0 = row-major, 1 = column-major).
#ifndef ROCM_WMMA_GEMM_COMMON_HPP
#define ROCM_WMMA_GEMM_COMMON_HPP

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace rocm_wmma_gemm
{

enum class m_layout
{
    row_major = 0, // element (i,j) of an m x n matrix lives at i*n + j
    col_major = 1 // element (i,j) lives at j*m + i
};

enum class m_input
{
    matrix_a = 0,
    matrix_b = 1
};

// Device-side storage type behind each host-visible element type.  16-bit types
// are moved as raw bits; arithmetic happens in fp32 inside the matrix cores.
template<class T>
struct type_selector
{
    using type = T;
};
template<>
struct type_selector<half>
{
    using type = _Float16;
};
template<>
struct type_selector<__hip_bfloat16>
{
    using type = __bf16;
};

// Edge of the square MFMA output tile the kernels are built from
// (v_mfma_f32_32x32x16_{f16,bf16}) and the CDNA wavefront width.
constexpr int mfma_tile = 32;
constexpr int mfma_k    = 16;
constexpr int warp_size = 64;

// Name kept for sources written against the RDNA library, where the matrix
// instruction tile was called wmma_tile; here it is the MFMA tile edge.
constexpr int wmma_tile = mfma_tile;

} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_COMMON_HPP
