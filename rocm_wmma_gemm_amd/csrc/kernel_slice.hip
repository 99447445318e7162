// One translation unit per (type pair, A layout, B layout): instantiates every
// tile variant and load mode for that combination.  Compiled 16 times with
//   -DRWG_TYPE=<0..3> -DRWG_AK=<0|1> -DRWG_BK=<0|1>
// so the kernels build in parallel.  (The reference generates one source file per
// tuned config instead: reference rocm_wmma_gemm/config/generate_config.py:375-391.)
#include "kernel_entry.hpp"

namespace rocm_wmma_gemm
{
namespace host
{

#define RWG_CAT2(a, b, c, d) a##b##_##c##_##d
#define RWG_CAT(a, b, c, d) RWG_CAT2(a, b, c, d)

#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE)                              \
    {entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_unguarded>(),       \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_guarded>(),         \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::scalar>(),             \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_unguarded, true>(), \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_guarded, true>(),      \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_unguarded, true, 1>(), \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_guarded, true, 1>(),   \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_unguarded, true, 2>(), \
     entry<BM, BN, BK, WM, WN, PIPE, device::load_mode::vec_guarded, true, 2>()},

const kernel_fn RWG_CAT(kernel_slice_, RWG_TYPE, RWG_AK, RWG_BK)[num_variants][num_modes] = {
#include "variants.def"
};
#undef RWG_VARIANT

} // namespace host
} // namespace rocm_wmma_gemm
