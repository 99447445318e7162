// entry<>: the launchable kernel for one tile variant and load mode of the type pair and
// operand layouts a translation unit is compiled for (-DRWG_TYPE=<0..3> -DRWG_AK=<0|1>
// -DRWG_BK=<0|1>), or nullptr where the pipeline is not built for that combination.
// Shared by the ahead-of-time slices (kernel_slice.hip) and the tuner's one-variant
// translation unit (kernel_jit.hip).
#ifndef ROCM_WMMA_GEMM_KERNEL_ENTRY_HPP
#define ROCM_WMMA_GEMM_KERNEL_ENTRY_HPP

#include "kernel_table.hpp"

#ifndef RWG_TYPE
#error "compile with -DRWG_TYPE=0..3 -DRWG_AK=0|1 -DRWG_BK=0|1"
#endif

namespace rocm_wmma_gemm
{
namespace host
{

namespace
{
constexpr device::in_kind kIn = (RWG_TYPE < 2) ? device::in_kind::f16 : device::in_kind::bf16;
using out_t = std::conditional<RWG_TYPE == 0, _Float16,
                               std::conditional<RWG_TYPE == 2, __bf16, float>::type>::type;

template<int BM, int BN, int BK, int WM, int WN, int PIPE, device::load_mode MODE, bool K_RUNS = false, int ONCE = 0>
constexpr kernel_fn entry()
{
    static_assert(PIPE >= 0 && PIPE <= 7, "unknown pipeline");
    if constexpr(K_RUNS)
    {
        // the twin that walks K in runs and groups (ONCE: with non-temporal loads of B, 1, or
        // A, 2): the large persistent tile only
        if constexpr(MODE != device::load_mode::scalar && PIPE == 5 && BM == 256 && BN == 256 && BK == 64)
        {
            return &device::gemm_entry<
                device::solo_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN, 2,
                                  MODE == device::load_mode::vec_guarded, true, ONCE>>;
        }
        else
        {
            return nullptr;
        }
    }
    else if constexpr(PIPE == 0)
    {
        return &device::gemm_entry<
            device::staged_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN, MODE>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 1)
    {
        // vec_guarded here means: operands are whole aligned tiles (the host padded
        // them if need be) but C is ragged, so the stores are guarded
        return &device::gemm_entry<
            device::direct_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN,
                                (BK == 64 ? 2 : 4), MODE == device::load_mode::vec_guarded>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 2)
    {
        return &device::gemm_entry<
            device::pingpong_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN,
                                  (BK == 64 ? 2 : 4), MODE == device::load_mode::vec_guarded>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 3)
    {
        return &device::gemm_entry<
            device::direct_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN,
                                (BK == 64 ? 2 : 4), MODE == device::load_mode::vec_guarded, 16>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 4)
    {
        return &device::gemm_entry<
            device::pingpong_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN,
                                  (BK == 64 ? 2 : 4), MODE == device::load_mode::vec_guarded, 16>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 5
                      && (BM % 128 == 0 || RWG_AK != 0) && (BN % 128 == 0 || RWG_BK != 0))
    {
        // (the LDS layout of an M/N-contiguous operand works in 128-row halves)
        return &device::gemm_entry<
            device::solo_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN,
                              (BK == 64 ? 2 : 4), MODE == device::load_mode::vec_guarded>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 6
                      && (BM % 128 == 0 || RWG_AK != 0) && (BN % 128 == 0 || RWG_BK != 0))
    {
        return &device::gemm_entry<device::direct_gemm<kIn, out_t, RWG_AK != 0, RWG_BK != 0, BM, BN, BK, WM, WN, 4,
                                                       MODE == device::load_mode::vec_guarded>>;
    }
    else if constexpr(MODE != device::load_mode::scalar && PIPE == 7)
    {
        // (one kernel for whole and ragged tiles: its loads and stores are always guarded)
        static_assert(BK == 128, "the streaming kernel's stages are 128 wide");
        return &device::gemm_entry<device::stream_gemm<kIn, out_t, BM, BN, RWG_AK != 0, RWG_BK != 0>>;
    }
    else
    {
        return nullptr; // the direct pipelines never load 2 bytes at a time
    }
}
} // namespace
} // namespace host
} // namespace rocm_wmma_gemm

#endif
