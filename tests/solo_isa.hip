// Instantiates the hand-scheduled kernel for a few type/layout/guard combinations so
// that the host test can look at the generated assembly (see test_host.py).
#include "kernel_table.hpp"

using namespace rocm_wmma_gemm;

template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::f16, _Float16, true, true, 256, 256, 64, 2, 2, 2, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::bf16, float, false, false, 256, 256, 64, 2, 2, 2, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::f16, _Float16, true, false, 256, 256, 64, 2, 2, 2, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::f16, _Float16, true, true, 256, 256, 64, 2, 2, 2, true>>(device::gemm_args);
template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::bf16, __bf16, true, true, 256, 192, 64, 2, 2, 2, false>>(device::gemm_args);
// the twin that walks K in runs and groups (its loop carries a few scalar instructions more)
template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::bf16, __bf16, true, true, 256, 256, 64, 2, 2, 2, false, true>>(device::gemm_args);
// the same twin with non-temporal loads of B
template __global__ void device::gemm_entry<device::solo_gemm<device::in_kind::bf16, __bf16, true, true, 256, 256, 64, 2, 2, 2, false, true, 1>>(device::gemm_args);
