// Instantiates direct-to-LDS kernels with an operand that is contiguous along M or N so
// that the host test can look at the generated assembly (see test_host.py).
#include "kernel_table.hpp"

using namespace rocm_wmma_gemm;

template __global__ void device::gemm_entry<device::direct_gemm<device::in_kind::f16, _Float16, false, true, 128, 128, 64, 2, 2, 4, false>>(device::gemm_args);
template __global__ void device::gemm_entry<device::direct_gemm<device::in_kind::bf16, float, false, false, 128, 128, 64, 2, 2, 2, false>>(device::gemm_args);
