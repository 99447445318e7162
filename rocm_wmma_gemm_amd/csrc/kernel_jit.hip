// One tile variant for one (type pair, A layout, B layout), compiled at tune time into a
// small shared library of its own so that the tuner can time kernels that the shipped
// library does not hold.  Compile with
//   -DRWG_TYPE=<0..3> -DRWG_AK=<0|1> -DRWG_BK=<0|1>
//   -DRWG_JIT_BM=.. -DRWG_JIT_BN=.. -DRWG_JIT_BK=.. -DRWG_JIT_WM=.. -DRWG_JIT_WN=.. -DRWG_JIT_PIPE=..
// and hand rwg_jit_kernels to rocm_wmma_gemm_register_variant of the loaded library.  A
// tuple that a pipeline's template does not take fails to compile (its static_asserts):
// the tuner counts that as "not feasible".
//
// Role of the reference's hipRTC step: reference rocm_wmma_gemm/config/tuner.cpp:237-395
// instantiates kernel_gemm_impl for one (warps, warp tiles, swizzle, bits) tuple from the
// kernel headers at run time.
#include "kernel_entry.hpp"

#if !defined(RWG_JIT_BM) || !defined(RWG_JIT_BN) || !defined(RWG_JIT_BK) || !defined(RWG_JIT_WM) \
    || !defined(RWG_JIT_WN) || !defined(RWG_JIT_PIPE)
#error "compile with -DRWG_JIT_BM/BN/BK/WM/WN/PIPE"
#endif

using namespace rocm_wmma_gemm;

extern "C" {

// (const objects have internal linkage unless declared extern)
extern const void* const rwg_jit_kernels[host::num_modes];
extern const int         rwg_jit_description[9];

// kernels by load mode: 16-byte unguarded, 16-byte guarded, 2-byte, then the K-run twins of
// the first two, and those twins with non-temporal loads of B and of A (null for every tuple
// but the persistent 256 x 256 x 64 tile)
const void* const rwg_jit_kernels[host::num_modes] = {
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_unguarded>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_guarded>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::scalar>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_unguarded, true>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_guarded, true>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_unguarded, true, 1>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_guarded, true, 1>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_unguarded, true, 2>()),
    reinterpret_cast<const void*>(host::entry<RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                              RWG_JIT_PIPE, device::load_mode::vec_guarded, true, 2>()),
};

// block_m, block_n, block_k, warps_m, warps_n, pipeline, type pair, A K-contiguous, B K-contiguous
const int rwg_jit_description[9] = {RWG_JIT_BM, RWG_JIT_BN, RWG_JIT_BK, RWG_JIT_WM, RWG_JIT_WN,
                                    RWG_JIT_PIPE, RWG_TYPE,   RWG_AK != 0, RWG_BK != 0};
}
