// Public C++ entry points: C = A * B on one MI355X (gfx950).
//
// Interface parity: reference rocm_wmma_gemm/include/rocm_wmma_gemm/gemm.hpp:50-73
// (template parameter order C, A, B; non-const operand pointers; stream by
// reference) and :76-217 (the set of explicit instantiations).
//
//   A is M x K, B is K x N, C is M x N, each densely packed in its own layout.
//   C is overwritten.  Batched calls step A, B, C by M*K, K*N, M*N elements.
//   The call enqueues on `stream` and returns; it does not synchronise.
#ifndef ROCM_WMMA_GEMM_HPP
#define ROCM_WMMA_GEMM_HPP

#include "kernel/common.hpp"

namespace rocm_wmma_gemm
{

template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T, class U>
__host__ void gemm(T* C, U* A, U* B, size_t M, size_t N, size_t K, hipStream_t& stream);

template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T, class U>
__host__ void
    gemm(T* C, U* A, U* B, size_t M, size_t N, size_t K, size_t batch_count, hipStream_t& stream);

// The shared library carries these 4 type pairs x 8 layout triples x {plain, batched}.
#define ROCM_WMMA_GEMM_FOR_EACH_LAYOUT(X, T, U)                                   \
    X(m_layout::row_major, m_layout::row_major, m_layout::row_major, T, U)        \
    X(m_layout::row_major, m_layout::row_major, m_layout::col_major, T, U)        \
    X(m_layout::row_major, m_layout::col_major, m_layout::row_major, T, U)        \
    X(m_layout::row_major, m_layout::col_major, m_layout::col_major, T, U)        \
    X(m_layout::col_major, m_layout::row_major, m_layout::row_major, T, U)        \
    X(m_layout::col_major, m_layout::row_major, m_layout::col_major, T, U)        \
    X(m_layout::col_major, m_layout::col_major, m_layout::row_major, T, U)        \
    X(m_layout::col_major, m_layout::col_major, m_layout::col_major, T, U)

#define ROCM_WMMA_GEMM_FOR_EACH_TYPE_PAIR(X)                         \
    ROCM_WMMA_GEMM_FOR_EACH_LAYOUT(X, half, half)                    \
    ROCM_WMMA_GEMM_FOR_EACH_LAYOUT(X, float, half)                   \
    ROCM_WMMA_GEMM_FOR_EACH_LAYOUT(X, __hip_bfloat16, __hip_bfloat16) \
    ROCM_WMMA_GEMM_FOR_EACH_LAYOUT(X, float, __hip_bfloat16)

#define ROCM_WMMA_GEMM_DECLARE(LC, LA, LB, T, U)                                              \
    extern template void gemm<LC, LA, LB, T, U>(T*, U*, U*, size_t, size_t, size_t,           \
                                                hipStream_t&);                                \
    extern template void gemm<LC, LA, LB, T, U>(T*, U*, U*, size_t, size_t, size_t, size_t,   \
                                                hipStream_t&);

ROCM_WMMA_GEMM_FOR_EACH_TYPE_PAIR(ROCM_WMMA_GEMM_DECLARE)

#undef ROCM_WMMA_GEMM_DECLARE

} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_HPP
