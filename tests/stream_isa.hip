// Instantiates the whole-K streaming kernel for a few tiles and layouts so that the host
// test can look at the generated assembly (see test_host.py).
#include "kernel_table.hpp"

using namespace rocm_wmma_gemm;

template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::f16, float, 64, 64, true, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::f16, _Float16, 32, 32, true, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::bf16, __bf16, 32, 128, true, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::bf16, float, 16, 64, false, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::f16, _Float16, 64, 32, false, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::f16, float, 32, 64, true, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::bf16, __bf16, 16, 32, true, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::bf16, float, 32, 16, false, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::f16, _Float16, 64, 16, true, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::f16, float, 128, 64, true, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::bf16, __bf16, 64, 128, false, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::stream_gemm<device::in_kind::bf16, float, 128, 32, false, true>>(device::gemm_args);
