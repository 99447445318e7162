// One translation unit per (type pair, A layout, B layout): instantiates every
// tile variant and load mode for that combination.  Compiled 16 times with
//   -DRWG_TYPE=<0..3> -DRWG_AK=<0|1> -DRWG_BK=<0|1>
// so the kernels build in parallel.  (The reference generates one source file per
// tuned config instead: reference rocm_wmma_gemm/config/generate_config.py:375-391.)
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

template<int BM, int BN, int BK, int WM, int WN, int PIPE, device::load_mode MODE>
constexpr kernel_fn entry()
{
    static_assert(PIPE >= 0 && PIPE <= 6, "unknown pipeline");
    if constexpr(PIPE == 0)
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
    else
    {
        return nullptr; // the direct pipelines never load 2 bytes at a time
    }
}
} // namespace

#define RWG_CAT2(a, b, c, d) a##b##_##c##_##d
#define RWG_CAT(a, b, c, d) RWG_CAT2(a, b, c, d)

#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE)                              \
    {entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_unguarded>(),       \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_guarded>(),         \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::scalar>()},

const kernel_fn RWG_CAT(kernel_slice_, RWG_TYPE, RWG_AK, RWG_BK)[num_variants][num_modes] = {
#include "variants.def"
};
#undef RWG_VARIANT

} // namespace host
} // namespace rocm_wmma_gemm
