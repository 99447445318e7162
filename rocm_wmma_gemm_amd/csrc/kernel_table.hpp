// Host-side view of the compiled kernels: a table of launchable entry points
// indexed by (type pair, A K-contiguous, B K-contiguous, tile variant, load mode).
//
// Stands where the reference has kernel_lookup / kernel_launcher (reference
// rocm_wmma_gemm/include/rocm_wmma_gemm/kernel_lookup.hpp:41,
// kernel_launcher.hpp:64-130): index arithmetic -> function pointer -> launch.
#ifndef ROCM_WMMA_GEMM_KERNEL_TABLE_HPP
#define ROCM_WMMA_GEMM_KERNEL_TABLE_HPP

#include "kernel/direct_kernel.hpp"
#include "kernel/pingpong_kernel.hpp"
#include "kernel/solo_kernel.hpp"
#include "kernel/stream_kernel.hpp"
#include "kernel/gemm_kernel.hpp"

namespace rocm_wmma_gemm
{
namespace host
{

struct variant_desc
{
    int block_m, block_n, block_k;
    int waves_m, waves_n;
    int pipeline;
    int lds_bytes;
    int threads;
};

#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE) +1
constexpr int num_variants = 0
#include "variants.def"
    ;
#undef RWG_VARIANT

constexpr int num_types = 4; // f16_f16, f32_f16, bf16_bf16, f32_bf16
constexpr int num_load_modes = 3; // device::load_mode
// kernels per variant: one per load mode, then the twins of the 16-byte unguarded and guarded
// kernels that walk K in runs and groups (persistent 256 x 256 x 64 kernel only; nullptr
// elsewhere), then those twins with non-temporal loads of B, then of A
constexpr int num_modes     = 9;
constexpr int k_runs_twin   = 3; // mode m < 2 has its twin at m + k_runs_twin
constexpr int once_stride   = 2; // and the twin that reads B (1) or A (2) once at m + k_runs_twin + once_stride * which

using kernel_fn = void (*)(const device::gemm_args);

extern const variant_desc variant_table[num_variants];

// Entry point of one compiled kernel, or nullptr if that combination is not built.
kernel_fn lookup_kernel(int type_idx, bool a_kmajor, bool b_kmajor, int variant, int mode);

// Per-(type, layout) tables, each defined in its own translation unit.
#define RWG_DECLARE_SLICE(T, AK, BK_) \
    extern const kernel_fn kernel_slice_##T##_##AK##_##BK_[num_variants][num_modes];
RWG_DECLARE_SLICE(0, 0, 0)
RWG_DECLARE_SLICE(0, 0, 1)
RWG_DECLARE_SLICE(0, 1, 0)
RWG_DECLARE_SLICE(0, 1, 1)
RWG_DECLARE_SLICE(1, 0, 0)
RWG_DECLARE_SLICE(1, 0, 1)
RWG_DECLARE_SLICE(1, 1, 0)
RWG_DECLARE_SLICE(1, 1, 1)
RWG_DECLARE_SLICE(2, 0, 0)
RWG_DECLARE_SLICE(2, 0, 1)
RWG_DECLARE_SLICE(2, 1, 0)
RWG_DECLARE_SLICE(2, 1, 1)
RWG_DECLARE_SLICE(3, 0, 0)
RWG_DECLARE_SLICE(3, 0, 1)
RWG_DECLARE_SLICE(3, 1, 0)
RWG_DECLARE_SLICE(3, 1, 1)
#undef RWG_DECLARE_SLICE

} // namespace host
} // namespace rocm_wmma_gemm

#endif
