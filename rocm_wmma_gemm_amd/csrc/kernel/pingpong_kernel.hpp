// Ping-pong MFMA GEMM kernel for gfx950: two waves per SIMD that take turns.
//
// Same data path as the direct kernel (direct_kernel.hpp: global -> LDS with
// global_load_lds_dwordx4, swizzled LDS layouts, ds_read_b64_tr_b16 for operands
// that are contiguous along M or N) but a different schedule.  In the direct kernel
// every wave interleaves its loads with its MFMAs; a load that cannot issue (the
// CU's miss queue is full of lines still on their way from the fabric) then holds
// up the MFMAs queued behind it in the same wave, and both waves of a SIMD hit that
// at the same time.  Here a wave alternates between two kinds of interval:
//
//   MEM(u)      read ALL MFMA operands of tile u from LDS into registers, issue its
//               share of the global -> LDS loads of tile u+STAGES-1, wait for its
//               share of tile u+1 to have landed
//   COMPUTE(u)  nothing but the TM*TN*KK MFMAs of tile u, back to back
//
// with a workgroup barrier between intervals.  Waves 0-3 (one per SIMD) and waves
// 4-7 (their SIMD partners) run half a period apart -- the second group passes one
// extra barrier before its loop -- so in every interval one wave of each SIMD feeds
// the MFMA pipe without touching memory while its partner does memory work that may
// stall as long as it likes within that interval.
//
// Hazards (tile t lives in stage t % STAGES; interval k lies between barriers k and
// k+1; group 0 runs MEM(t) in interval 2t, group 1 in interval 2t+1):
//   * tile t is last read in interval 2t+1, so its stage is free from barrier 2t+2;
//     MEM(u) overwrites stage (u-1) % STAGES, i.e. tile u-1, in interval >= 2u. OK.
//   * a wave waits for its own share of tile u+1 at the end of MEM(u) (the loads of
//     STAGES-2 later tiles may still be in flight: vmcnt((STAGES-2)*loads)); the
//     barrier that ends that interval comes before any wave reads tile u+1.
//
// Role with respect to the reference: as the other kernels, its gemm_impl (reference
// rocm_wmma_gemm/include/rocm_wmma_gemm/kernel/kernel.hpp:108-556).
#ifndef ROCM_WMMA_GEMM_PINGPONG_KERNEL_HPP
#define ROCM_WMMA_GEMM_PINGPONG_KERNEL_HPP

#include <utility>

#include "direct_kernel.hpp"

namespace rocm_wmma_gemm
{
namespace device
{

template<in_kind IN,
         class OutT,
         bool A_KMAJOR,
         bool B_KMAJOR,
         int  BM,
         int  BN,
         int  BK,
         int  WAVES_M,
         int  WAVES_N,
         int  STAGES,
         bool GUARD_C = false,
         int  MI      = 32>
struct pingpong_gemm
{
    using InT = typename std::conditional<IN == in_kind::f16, _Float16, __bf16>::type;

    static constexpr int WAVES     = WAVES_M * WAVES_N;
    static constexpr int THREADS   = 64 * WAVES;
    static constexpr int WTM       = BM / WAVES_M;
    static constexpr int WTN       = BN / WAVES_N;
    static constexpr int TM        = WTM / MI;
    static constexpr int TN        = WTN / MI;
    static constexpr int KK        = BK / (MI == 32 ? 16 : 32);
    static constexpr int A_BYTES   = BM * BK * 2;
    static constexpr int B_BYTES   = BN * BK * 2;
    static constexpr int STAGE     = A_BYTES + B_BYTES;
    static constexpr int LDS_BYTES = STAGES * STAGE;
    static_assert(WAVES == 8, "two groups of four waves: one wave of each group per SIMD");
    static_assert(STAGES == 4 || STAGES == 2, "stage ring must be a power of two");
    static_assert(LDS_BYTES <= 160 * 1024, "tile ring does not fit the 160 KB LDS");

    using op_a  = direct_operand<A_KMAJOR, BM, BK, WTM, WAVES, MI>;
    using op_b  = direct_operand<B_KMAJOR, BN, BK, WTN, WAVES, MI>;
    using acc_t = mfma_acc<MI>;

    static constexpr int VM_LOADS = op_a::PER_WAVE + op_b::PER_WAVE; // per wave, per tile
    static_assert((STAGES - 1) * VM_LOADS < 64, "vmcnt is a 6-bit counter");

    static constexpr int waitcnt_imm(int vmcnt)
    {
        return (vmcnt & 15) | (7 << 4) | (0 << 8) | ((vmcnt >> 4) << 14);
    }

    // All MFMA operands of the tile at LDS byte address `stage`, as pinned reads (see
    // direct_operand::fragment_pinned): the s_waitcnt at the end of the memory
    // interval covers them, and the compiler does not put a wait for all outstanding
    // global -> LDS loads in front of them.
    template<int... X, int... Y>
    __device__ __forceinline__ static void read_fragments(std::integer_sequence<int, X...>,
                                                          std::integer_sequence<int, Y...>,
                                                          const op_a&  oa,
                                                          const op_b&  ob,
                                                          unsigned int stage,
                                                          u32x4 (&fa)[KK][TM],
                                                          u32x4 (&fb)[KK][TN])
    {
        ((fa[X / TM][X % TM] = oa.template fragment_pinned<X % TM, X / TM>(stage)), ...);
        ((fb[Y / TN][Y % TN] = ob.template fragment_pinned<Y % TN, Y / TN>(stage + A_BYTES)), ...);
    }

    __device__ __forceinline__ static void run(const gemm_args& args)
    {
        __shared__ __attribute__((aligned(1024))) char lds_raw[LDS_BYTES];
        lds_char_ptr       lds      = (lds_char_ptr)lds_raw;
        const unsigned int lds_addr = (unsigned int)(size_t)lds;

        const int tid     = threadIdx.x;
        const int lane    = tid & 63;
        const int wave    = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int group   = wave >> 2; // waves w and w+4 share a SIMD
        const int wave_m  = wave / WAVES_N;
        const int wave_n  = wave % WAVES_N;

        const block_work w = decode_block(args);
        const int slice    = w.slice;
        const tile_coord t = map_tile(w.tile_id, args.grid_m, args.grid_n, args.group);
        const int row0 = t.m * BM;
        const int col0 = t.n * BN;

        const int k_steps_total = args.K / BK;
        const int steps_per     = (k_steps_total + w.slices - 1) / w.slices;
        const int step_begin    = slice * steps_per;
        int       step_end      = step_begin + steps_per;
        if(step_end > k_steps_total)
        {
            step_end = k_steps_total;
        }
        const int nk = step_end - step_begin;

        const long long batch = blockIdx.y;
        const InT* A = static_cast<const InT*>(args.A) + batch * args.batch_stride_a;
        const InT* B = static_cast<const InT*>(args.B) + batch * args.batch_stride_b;

        const long long a_ld = args.lda;
        const long long b_ld = args.ldb;
        const long long a_sr = A_KMAJOR ? a_ld : 1, a_sk = A_KMAJOR ? 1 : a_ld;
        const long long b_sr = B_KMAJOR ? b_ld : 1, b_sk = B_KMAJOR ? 1 : b_ld;

        op_a oa;
        op_b ob;
        oa.init(wave, lane, a_ld, wave_m * WTM);
        ob.init(wave, lane, b_ld, wave_n * WTN);

        const InT* a_src = A + row0 * a_sr + (long long)step_begin * BK * a_sk;
        const InT* b_src = B + col0 * b_sr + (long long)step_begin * BK * b_sk;
        const long long a_step = BK * a_sk, b_step = BK * b_sk;

        acc_t acc[TM][TN];
#pragma unroll
        for(int i = 0; i < TM; ++i)
        {
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
#pragma unroll
                for(int v = 0; v < (MI == 32 ? 16 : 4); ++v)
                {
                    acc[i][j][v] = 0.0f;
                }
            }
        }

        if(nk > 0)
        {
            // Source pointers never move past the last tile of this K range: the
            // redundant loads at the end land in stages nobody reads again and keep
            // the number of loads in flight a compile-time constant.
            const InT* a_last = a_src + (long long)(nk - 1) * a_step;
            const InT* b_last = b_src + (long long)(nk - 1) * b_step;

            // prologue: tiles 0 .. STAGES-2, then everyone's share of tile 0 must land
#pragma unroll
            for(int s = 0; s < STAGES - 1; ++s)
            {
                oa.issue(a_src, lds + s * STAGE, wave);
                ob.issue(b_src, lds + s * STAGE + A_BYTES, wave);
                a_src = a_src + a_step > a_last ? a_last : a_src + a_step;
                b_src = b_src + b_step > b_last ? b_last : b_src + b_step;
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2) * VM_LOADS));
            __builtin_amdgcn_s_barrier(); // barrier 0
            if(group == 1)
            {
                __builtin_amdgcn_s_barrier(); // barrier 1: group 1 idles through interval 0
            }

            u32x4 fa[KK][TM], fb[KK][TN];
            for(int u = 0; u < nk; ++u)
            {
                lds_char_ptr fill = lds + ((u + STAGES - 1) & (STAGES - 1)) * STAGE;
                // ---- MEM(u)
                read_fragments(std::make_integer_sequence<int, KK * TM>{},
                               std::make_integer_sequence<int, KK * TN>{}, oa, ob,
                               lds_addr + (u & (STAGES - 1)) * STAGE, fa, fb);
                oa.issue(a_src, fill, wave);
                ob.issue(b_src, fill + A_BYTES, wave);
                a_src = a_src + a_step > a_last ? a_last : a_src + a_step;
                b_src = b_src + b_step > b_last ? b_last : b_src + b_step;
                __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2) * VM_LOADS));
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                // ---- COMPUTE(u)
                __builtin_amdgcn_s_setprio(2);
#pragma unroll
                for(int kk = 0; kk < KK; ++kk)
                {
#pragma unroll
                    for(int i = 0; i < TM; ++i)
                    {
#pragma unroll
                        for(int j = 0; j < TN; ++j)
                        {
                            acc[i][j] = mfma_tile<IN, MI>(fa[kk][i], fb[kk][j], acc[i][j]);
                        }
                    }
                }
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            if(group == 0)
            {
                __builtin_amdgcn_s_barrier(); // matches group 1's extra barrier
            }
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0)); // redundant tail loads
        }

        if(w.slices == 1)
        {
            OutT* C = static_cast<OutT*>(args.C) + batch * args.batch_stride_c;
            write_out<MI, GUARD_C>(
                acc, C, args.M, args.N, args.N, row0 + wave_m * WTM, col0 + wave_n * WTN, lane);
        }
        else
        {
            long long pitch;
            float*    P = partial_base<BM, BN>(args, w, batch, row0, col0, pitch);
            write_out<MI, GUARD_C>(
                acc, P, args.M, args.N, pitch, row0 + wave_m * WTM, col0 + wave_n * WTN, lane);
        }
    }
};

} // namespace device
} // namespace rocm_wmma_gemm

#endif // ROCM_WMMA_GEMM_PINGPONG_KERNEL_HPP
